"""Seeded sweeps over layer shapes, rates and token counts that straddle every route switch of the fused
linears (fused-input GEMV, small-batch MFMA kernel, small and large tile kernels, K slots, block-diagonal
transforms of odd sizes), each against the oracle's fp32 CPU forward within the 1e-2 bound, plus the
many-token paths that only large layers reach (fp16 sums, the tail-round launch) through their properties
(needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t

pytestmark = pytest.mark.gpu
TOL = 1e-2
TOKENS = [1, 2, 3, 4, 5, 8, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 257, 300]


def _trellis_cases():
    rng = np.random.default_rng(2024)
    cases = []
    for i in range(36):
        m = int(rng.integers(1, 40)) * 32
        n = int(rng.integers(1, 48)) * 64
        K = int(rng.integers(2, 5))
        K2 = int(rng.choice([0, 0, 1, 2, 3, 4]))
        B = TOKENS[(i * 7) % len(TOKENS)]
        cases.append((m, n, K, K2, B, i))
    return cases


@pytest.mark.parametrize("m,n,K,K2,B,seed", _trellis_cases())
def test_trellis_fused_linear_random_shapes(m, n, K, K2, B, seed):
    from glq_amd import ext, hadamard as H
    say("random trellis", m, n, K, K2, B)
    su, sv = O.rht_signs(m, n, 300 + seed)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": O.random_packed(m, n, K, seed), "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
           "Wscale": np.float32(0.02), "blocks_m": bm, "blocks_n": bn}
    if K2:
        art["trellis_packed2"] = O.random_packed(m, n, K2, 1000 + seed)
        art["inv_resid_scale2"] = np.float32(0.25)
    dtype = torch.bfloat16 if seed % 2 else torch.float16
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(seed)) * 0.7).to(dtype)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    meta = (torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV))
    if K2:
        y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
            x.to(DEV), t(art["SV"]), t(art["SU"]), t(art["trellis_packed"]), t(art["trellis_packed2"]), *meta, 0.02, 0.25,
            n, m, n, m, out_dtype=dtype)
    else:
        y = ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), t(art["SV"]), t(art["SU"]), t(art["trellis_packed"]), *meta,
                                                    0.02, n, m, n, m, out_dtype=dtype)
    assert y.shape == (B, m) and y.dtype == dtype
    e = rel(y, ref)
    assert e < TOL, e


def _e8_cases():
    rng = np.random.default_rng(77)
    cases = []
    for i in range(30):
        m = int(rng.integers(1, 300)) * (8 if i % 3 else 1)
        n = int(rng.integers(1, 300)) * 8 if i % 4 else int(rng.integers(1, 12)) * 256
        stages = int(rng.integers(1, 5))
        B = TOKENS[(i * 11) % len(TOKENS)]
        cases.append((m, n, stages, B, i))
    return cases


@pytest.mark.parametrize("m,n,stages,B,seed", _e8_cases())
def test_e8_fused_linear_random_shapes(m, n, stages, B, seed):
    """Rows and widths that are not multiples of anything but 8 columns, 1-4 stages, prepared (folded where
    the kernels take it) and not."""
    from glq_amd import ext, hadamard as H
    say("random e8", m, n, stages, B)
    rng = np.random.default_rng(seed)
    q = [rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16) for _ in range(stages)]
    inv = [1 / 3.0, 1 / 9.0, 1 / 27.0]
    su, sv = O.rht_signs(m, n, 500 + seed)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"Qidxs": q[0], "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.015),
           "blocks_m": bm, "blocks_n": bn}
    W = O.e8_dequant(q[0], q[1] if stages > 1 else None, inv[0] if stages > 1 else 0.0, q[2] if stages > 2 else None,
                     inv[1] if stages > 2 else 0.0, q[3] if stages > 3 else None, inv[2] if stages > 3 else 0.0)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(seed)) * 0.7).to(torch.bfloat16)
    ref = O.linear_forward_rht(x.float().numpy(), W * np.float32(0.015), su.astype(np.float32), sv.astype(np.float32),
                               bn, bm, n, m)
    cb = e8_table_f16()
    d = [t(a) for a in q] + [None] * (4 - stages)
    if seed % 2 == 0:
        ext.e8_prepare(d[0], cb, d[1], cb, d[2], d[3])
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("ignore", RuntimeWarning)       # the unprepared half runs on its indices, by design
        y = ext.glq_fused_linear_block_diag_cuda(
            x.to(DEV), t(art["SV"]), t(art["SU"]), d[0], cb, 0.015, n, m, n, m, torch.tensor(bn), torch.tensor(bm),
            H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), d[1], cb, inv[0] if stages > 1 else 0.0,
            d[2], cb, inv[1] if stages > 2 else 0.0, d[3], cb, inv[2] if stages > 3 else 0.0, out_dtype=torch.bfloat16)
    assert y.shape == (B, m)
    e = rel(y, ref)
    assert e < TOL, e


@pytest.mark.parametrize("m,n,M,K", [(14336, 512, 4096, 4), (14336, 256, 4096, 2), (11008, 512, 8192, 3),
                                     (1088, 2368, 333, 2), (2368, 1088, 1100, 4)])
def test_many_token_trellis_paths_of_large_layers(m, n, M, K):
    """The last two: rows of several Hadamard blocks of which some are small (2368 = 2048 + 256 + 64,
    1088 = 1024 + 64), whose transforms take many tokens per workgroup, written straight into the tile
    kernel's operand layout, at token counts that end inside such a group.  Tile counts that trigger the tail-round launch (896 = 3.5 rounds, 1376 = 5.4 rounds of 256 CUs) on
    narrow layers, so that the oracle stays cheap: sampled rows of every token tile and of both launches' row
    ranges against the oracle; the fused linear (fp16 sums between tile kernel and output transform) against
    the unfused pipeline (fp32 sums) on all rows; repeated runs bit-identical."""
    from glq_amd import ext, hadamard as H
    say("many-token trellis", m, n, M, K)
    packed = O.random_packed(m, n, K, 5)
    su, sv = O.rht_signs(m, n, 9)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    meta = (torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV))
    x = (torch.randn(M, n, generator=torch.Generator().manual_seed(3)) * 0.7).to(torch.bfloat16)
    xd, pd, sud, svd = x.to(DEV), t(packed), t(su.astype(np.float16)), t(sv.astype(np.float16))
    old = ext.TRELLIS_BATCH_MAX
    ext.TRELLIS_BATCH_MAX = 1 << 30
    try:
        y = ext.glq_fused_linear_trellis_3inst_cuda(xd, svd, sud, pd, *meta, 0.02, n, m, n, m, out_dtype=torch.bfloat16)
        assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_cuda(xd, svd, sud, pd, *meta, 0.02, n, m, n, m,
                                                                      out_dtype=torch.bfloat16))
    finally:
        ext.TRELLIS_BATCH_MAX = old
    rows = np.unique(np.concatenate([np.arange(0, M, 509 if M > 2000 else 37), [M - 1, 255, 256, min(511, M - 1), min(512, M - 1)]]))
    art = {"trellis_packed": packed, "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": bm, "blocks_n": bn}
    ref = O.trellis_linear_forward(x[rows].float().numpy(), art, n, m)
    assert rel(y[torch.from_numpy(rows).to(DEV)], ref) < TOL
    # the unfused pipeline keeps fp32 sums: input transform, matmul entry, output transform
    x_rht = torch.empty(M, n, dtype=torch.float16, device=DEV)
    ext.glq_input_rht_blockdiag_cuda(xd, svd, x_rht, n, n, meta[0], meta[2])
    y_rht = ext.glq_decode_matmul_trellis_3inst_cuda(x_rht, pd, m, n, 0.02)
    y2 = torch.empty(M, m, dtype=torch.bfloat16, device=DEV)
    ext.glq_output_rht_blockdiag_cuda(y_rht, sud, y2, m, m, meta[1], meta[3])
    assert rel(y, y2.float().cpu().numpy()) < 4e-3
    # every row range of the two launches is written: no row of the output is left at its initial value
    assert bool(torch.isfinite(y.float()).all()) and float(y.float().abs().sum(0).min()) > 0.0


@pytest.mark.parametrize("m,n,K,K2,in_f", [
    (32, 64, 4, 1, 64), (64, 4096, 4, 2, 4096), (160, 2368, 4, 3, 2300), (512, 2048, 4, 4, 2048),
    (960, 2560, 4, 2, 2560), (2048, 2048, 4, 1, 2048), (4096, 4096, 4, 2, 4000), (2048, 11008, 4, 4, 11008),
    (1088, 1088, 3, 2, 1088), (2048, 2048, 2, 2, 2048)])
def test_few_tokens_of_two_stage_layers(m, n, K, K2, in_f):
    """1, 3 and 16 tokens through a stacked layer: with a first stage of 4 bits/weight both streams are decoded in
    one launch (at one token with the input transform folded in, at every height; at 2..16 tokens against the
    staged transformed activations); the last two cases, other first stages, take a launch per stage.  Against
    the oracle, through the finished output and through the RHT-domain product written into a wider row, and
    equal bit for bit on a second call."""
    from glq_amd import ext, hadamard as H
    say("few tokens two stages", m, n, K, K2, in_f)
    su, sv = O.rht_signs(m, n, 41)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": O.random_packed(m, n, K, 11), "trellis_packed2": O.random_packed(m, n, K2, 12),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16)}
    W = (O.decode_layer(art["trellis_packed"], m, n, fast=True) +
         O.decode_layer(art["trellis_packed2"], m, n, fast=True) * np.float32(0.3)).astype(np.float32)
    bnt, bmt, bnm, bmm = torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV)
    p1, p2, svd, sud = t(art["trellis_packed"]), t(art["trellis_packed2"]), t(art["SV"]), t(art["SU"])
    for B in (1, 3, 16):
        x = (torch.randn(B, in_f, generator=torch.Generator().manual_seed(m + n + B)) * 0.7).to(torch.bfloat16)
        xp = np.zeros((B, n), np.float32)                     # columns past in_features are zero padding
        xp[:, :in_f] = x.float().numpy()
        ref = O.linear_forward_rht(xp, W * np.float32(0.02), su.astype(np.float32), sv.astype(np.float32), bn, bm, n, m)
        y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(x.to(DEV), svd, sud, p1, p2, bnt, bmt, bnm, bmm, 0.02, 0.3,
                                                         in_f, m, n, m, out_dtype=torch.bfloat16)
        assert y.shape == (B, m)
        assert rel(y, ref) < TOL, (B, rel(y, ref))
        assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_rvq2_cuda(x.to(DEV), svd, sud, p1, p2, bnt, bmt, bnm, bmm,
                                                                           0.02, 0.3, in_f, m, n, m, out_dtype=torch.bfloat16))
        # the product before the output transform, into columns [32, 32 + m) of a wider row
        wide = torch.full((B, m + 64), 7.0, dtype=torch.float32, device=DEV)
        ext.glq_fused_linear_trellis_3inst_yrht_rvq2_cuda(x.to(DEV), svd, p1, p2, bnt, bnm, 0.02, 0.3, in_f, n, m, wide, 32)
        xr = O.block_diag_fht(xp * sv.astype(np.float16).astype(np.float32)[None, :], bn)
        assert rel(wide[:, 32:32 + m], (xr @ W.T) * np.float32(0.02)) < TOL, B
        assert float(wide[:, :32].min()) == 7.0 and float(wide[:, 32 + m:].max()) == 7.0


def test_two_stage_layers_with_a_launch_per_stage_in_a_fresh_process():
    """GLQ_TRELLIS_FUSE_STAGES=0 (read once by the library): two-stage layers decode their stages in two launches
    at every token count; the two-stage cases of this file and of the module tests against the oracle that way, in
    a process of their own."""
    import os
    import subprocess
    import sys
    say("two-stage layers, a launch per stage, child process")
    here = os.path.dirname(os.path.abspath(__file__))
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.abspath(__file__), os.path.join(here, "test_gpu_module.py"),
                        "-x", "-q", "-m", "gpu", "-k", "two_stage and not fresh_process", "--timeout", "300",
                        "--timeout-method", "thread", "-p", "no:cacheprovider"],
                       env={**os.environ, "GLQ_TRELLIS_FUSE_STAGES": "0"}, capture_output=True, text=True, timeout=900,
                       cwd=os.path.dirname(here))
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-1000:])
    assert " passed" in r.stdout and "no tests ran" not in r.stdout, r.stdout[-500:]


@pytest.mark.parametrize("env", [{"GLQ_TT_PC_STEPS": "1"}, {"GLQ_TT_PC": "0"}])
def test_tile_kernels_with_either_split_of_the_waves_in_a_fresh_process(env):
    """Tiles of up to 256 tokens run with four decoding and four multiplying waves when their K slots are long
    enough, with eight waves that do both otherwise (switches read once by the library).  GLQ_TT_PC_STEPS=1: the
    split form wherever the tile allows it; GLQ_TT_PC=0: never.  The many-token cases of this file and the grouped
    many-token calls against the oracle under both, each in a process of its own."""
    import os
    import subprocess
    import sys
    say("tile kernels, wave roles, child process", env)
    here = os.path.dirname(os.path.abspath(__file__))
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.abspath(__file__), os.path.join(here, "test_gpu_group_many.py"),
                        "-x", "-q", "-m", "gpu", "-k",
                        "(trellis_fused_linear_random_shapes or large_activations or ragged_out or grouped_many_tokens) and not fresh_process",
                        "--timeout", "300", "--timeout-method", "thread", "-p", "no:cacheprovider"],
                       env={**os.environ, **env}, capture_output=True, text=True, timeout=900, cwd=os.path.dirname(here))
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-1000:])
    assert " passed" in r.stdout and "no tests ran" not in r.stdout, r.stdout[-500:]


def test_large_activations_stay_finite_at_many_tokens():
    """Activations of a few thousand: the unscaled sum over a row of 2048 columns passes the fp16 range, the
    layer's output (the sum times Wscale) does not.  The fp16 sums between the tile kernel and the output transform
    carry the scale, so the many-token path stays finite and inside the bound, one- and two-stage layers alike."""
    from glq_amd import ext, hadamard as H
    m, n, B = 1024, 2048, 100
    say("large activations", m, n, B)
    su, sv = O.rht_signs(m, n, 5)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    p1, p2 = O.random_packed(m, n, 4, 21), O.random_packed(m, n, 2, 22)
    W1 = O.decode_layer(p1, m, n, fast=True)
    W2 = O.decode_layer(p2, m, n, fast=True)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(1)) * 3000.0).to(torch.bfloat16)
    meta = (torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV))
    svd, sud = t(sv.astype(np.float16)), t(su.astype(np.float16))
    for W, call in ((W1, lambda: ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), svd, sud, t(p1), *meta, 0.02, n, m, n, m,
                                                                        out_dtype=torch.bfloat16)),
                    (W1 + np.float32(0.3) * W2,
                     lambda: ext.glq_fused_linear_trellis_3inst_rvq2_cuda(x.to(DEV), svd, sud, t(p1), t(p2), *meta, 0.02, 0.3,
                                                                          n, m, n, m, out_dtype=torch.bfloat16))):
        ref = O.linear_forward_rht(x.float().numpy(), W.astype(np.float32) * np.float32(0.02), su.astype(np.float32),
                                   sv.astype(np.float32), bn, bm, n, m)
        assert float(np.abs(ref).max()) < 6.0e4 and float(np.abs(ref).max()) / 0.02 > 7.0e4   # the case is what it claims
        y = call()
        assert bool(torch.isfinite(y.float()).all())
        assert rel(y, ref) < TOL, rel(y, ref)


def test_ragged_out_features_at_many_tokens():
    """out_features that is not a multiple of 8 (rows of y that do not start on 16 bytes) at more than 64 tokens:
    the whole-block output transform that reads fp16 sums does not apply, the sums stay fp32; one layer and two
    layers through the grouped call (the second layer's columns start at an odd offset)."""
    from glq_amd import ext, hadamard as H
    m, n, B, out_f = 1856, 2496, 513, 1853
    say("ragged out_features, many tokens", m, n, B, out_f)
    su, sv = O.rht_signs(m, n, 8)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    p1 = O.random_packed(m, n, 4, 31)
    W = O.decode_layer(p1, m, n, fast=True).astype(np.float32)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(2)) * 0.7).to(torch.bfloat16)
    ref = O.linear_forward_rht(x.float().numpy(), W * np.float32(0.02), su.astype(np.float32), sv.astype(np.float32), bn, bm, n, m)
    bnt, bnm = torch.tensor(bn), H.pack_block_meta(bn).to(DEV)
    svd, sud, pd = t(sv.astype(np.float16)), t(su.astype(np.float16)), t(p1)
    y = ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), svd, sud, pd, bnt, torch.tensor(bm), bnm, H.pack_block_meta(bm).to(DEV),
                                                0.02, n, out_f, n, m, out_dtype=torch.bfloat16)
    assert y.shape == (B, out_f) and rel(y, ref[:, :out_f]) < TOL
    yg = ext.glq_fused_linear_trellis_3inst_group(x.to(DEV), [(svd, sud, pd, 0.02, out_f, m), (svd, sud, pd, 0.02, m, m)],
                                                  bnt, bnm, n, n, out_dtype=torch.bfloat16)
    assert yg.shape == (B, out_f + m)
    assert rel(yg[:, :out_f], ref[:, :out_f]) < TOL and rel(yg[:, out_f:], ref) < TOL
