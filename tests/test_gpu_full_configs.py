"""The large benchmark configurations at their full shapes (needs an MI355X): configs[2] (E8 two-stage
4 bpw, 4096 <-> 14336, M = 1, 4, 16) and configs[3] (the same shapes, trellis and E8, M = 256 and
1024) against the oracle's fp32 CPU path, plus properties that do not need an oracle at these
sizes: linearity in x, rows of a batch equal to single-token calls, repeated runs bit-identical."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t, e8_prepared

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e

TOL = 1e-2                                  # relative Frobenius error, bf16 I/O, fp32 accumulation

SHAPES = [(14336, 4096), (4096, 14336)]


def _e8_layer(m, n, seed):
    rng = np.random.default_rng(seed)
    lo = rng.integers(0, 30000, size=(2, m, n // 8))
    hi = rng.integers(0, 65536, size=(2, m, n // 8))
    q = np.where(rng.random((2, m, n // 8)) < 0.7, lo, hi).astype(np.uint16).view(np.int16)
    su, sv = O.rht_signs(m, n, 42)
    return q[0], q[1], su.astype(np.float16), sv.astype(np.float16)


def _e8_forward(ext, x, q1, q2, su, sv, m, n, dtype):
    from glq_amd import hadamard as H
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    cb = e8_table_f16()
    d1, d2, _, _ = e8_prepared(ext, cb, q1, q2)                   # folded once per layer, then looked up
    return ext.glq_fused_linear_block_diag_cuda(
        x, t(sv), t(su), d1, cb, 0.02, n, m, n, m, torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), d2, cb, 1 / 3.0,
        out_dtype=dtype)


@pytest.mark.parametrize("m,n", SHAPES)
def test_e8_two_stage_full_shapes(ext, m, n):
    say("e8 full", m, n)
    q1, q2, su, sv = _e8_layer(m, n, m)
    art = {"Qidxs": q1, "Qidxs2": q2, "inv_resid_scale": np.float32(1 / 3.0), "SU": su, "SV": sv,
           "Wscale": np.float32(0.02), "blocks_m": O.block_decompose(m), "blocks_n": O.block_decompose(n)}
    x = torch.randn(1024, n, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    ref = O.e8_linear_forward(x[:272].float().numpy(), art, n, m)
    xd = x.to(DEV)
    ys = {}
    for M in (1, 4, 16, 40, 256, 1024):                    # indices -> MFMA up to 16 tokens, dense route above
        y = _e8_forward(ext, xd[:M], q1, q2, su, sv, m, n, torch.bfloat16)
        assert y.shape == (M, m)
        assert rel(y[:min(M, 272)], ref[:min(M, 272)]) < TOL
        assert torch.equal(y, _e8_forward(ext, xd[:M], q1, q2, su, sv, m, n, torch.bfloat16))
        ys[M] = y.float()
    # rows of the 16-token call are the single-token results (same kernel family, same K order)
    assert rel(ys[16][:1], ys[1].cpu().numpy()) < 4e-3 and rel(ys[16][:4], ys[4].cpu().numpy()) < 4e-3
    assert rel(ys[1024][:256], ys[256].cpu().numpy()) < 4e-3
    # linearity: f(a x0 + b x1) = a f(x0) + b f(x1) up to bf16 rounding of inputs and outputs
    x0, x1 = xd[0:1].float(), xd[1:2].float()
    mix = (0.5 * x0 - 2.0 * x1).to(torch.bfloat16)
    lhs = _e8_forward(ext, mix, q1, q2, su, sv, m, n, torch.bfloat16).float()
    rhs = 0.5 * ys[4][0:1] - 2.0 * ys[4][1:2]
    assert rel(lhs, rhs.cpu().numpy()) < 2e-2


@pytest.mark.parametrize("m,n", SHAPES)
def test_trellis_full_shapes_many_tokens(ext, m, n):
    from glq_amd import hadamard as H
    say("trellis full", m, n)
    p = O.random_packed(m, n, 4, seed=n)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": p, "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
           "Wscale": np.float32(0.018), "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(1024, n, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    # the oracle's forward with its vectorised state unpacking (pinned against the plain one
    # in the oracle's own tests): glq/quantized_linear.py:986-1010
    W = (O.decode_layer(p, m, n, fast=True) * np.float32(art["Wscale"])).astype(np.float32)
    ref = O.linear_forward_rht(x[:272].float().numpy(), W, su.astype(np.float32), sv.astype(np.float32), bn, bm, n, m)
    del W
    args = (t(art["SV"]), t(art["SU"]), t(p), torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV),
            H.pack_block_meta(bm).to(DEV), 0.018, n, m, n, m)
    xd = x.to(DEV)
    ys = {}
    for M in (1, 3, 16, 40, 64, 256, 1024):                # GEMV forms, 32+ tokens: whole-block finishing on tall layers, 128-token tiles, dense
        y = ext.glq_fused_linear_trellis_3inst_cuda(xd[:M], *args, out_dtype=torch.bfloat16)
        assert rel(y[:min(M, 272)], ref[:min(M, 272)]) < TOL
        assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_cuda(xd[:M], *args, out_dtype=torch.bfloat16))
        ys[M] = y.float()
    assert rel(ys[16][:1], ys[1].cpu().numpy()) < 6e-3
    assert rel(ys[1024][:256], ys[256].cpu().numpy()) < 6e-3
    # the dequantizer at this size: every weight an exact fp16 value of the 3INST code
    W = ext.glq_decompress_trellis_3inst_cuda(t(p), m, n)
    ref_w = O.decode_layer(p[: (64 // 16) * (n // 16)], 64, n, fast=True)      # first four tile rows
    assert np.array_equal(W[:64].float().cpu().numpy(), ref_w)
