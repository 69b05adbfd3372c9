"""The benchmark configurations on really quantized weights at their full shapes (needs an MI355X).

Weights are N(0, 0.02) from seed 0, transformed by the oracle's seeded RHT and quantized by the
GPU encoders (tail-biting Viterbi for the trellis, nearest-E8 search with a x3 residual stage for
the shell codebook), which are bit-equal to the oracle's encoders on the small cases of
test_gpu_encode.py.  Every check here is of the DECODE side against the oracle on whole layers:

* the dequantizer, bit for bit, on every weight of the layer;
* the fused linear against the oracle's fp32 CPU forward on the whole output (1e-2 relative
  Frobenius error, bf16 in and out, fp32 accumulation);
* the reference's quality gates (tests/test_trellis_3inst_kernel.py:309-312, 353-365, 383-395,
  846-859 in the reference checkout): SQNR > 40 dB of the GEMV / batched product against
  x @ W_dec.T, and > 35 dB of the fused layer against x @ W_hat.T with W_hat the quantizer's own
  reconstruction carried back to the weight domain -- never one decode against another;
* 4096-token calls of configs[3] against the oracle on rows sampled from every 128-token tile
  position class, and against the 1024-token call row by row.
"""
import math

import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t, e8_prepared

pytestmark = pytest.mark.gpu

TOL = 1e-2                                  # relative Frobenius error, bf16 I/O, fp32 accumulation


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e


def sqnr(ref, got):
    ref = np.asarray(ref, np.float64)
    got = np.asarray(got, np.float64)
    return 10 * math.log10((ref ** 2).mean() / ((got - ref) ** 2).mean())


def gauss_weight(m, n):
    return (torch.randn(m, n, generator=torch.Generator().manual_seed(0)) * 0.02).numpy()


def to_weight_domain(W_rht, su, sv, bm, bn):
    """diag(su) H_m W_rht H_n diag(sv): the inverse of rht_transform_weights (H is symmetric and
    its own inverse), glq/rht.py:124-138."""
    A = O.block_diag_fht(W_rht, bn)
    A = O.block_diag_fht(A.T.copy(), bm).T
    return A * su[:, None] * sv[None, :]


_CACHE = {}


def trellis_layer(ext, m, n, K=4):
    """(W, art, W_dec): art in the oracle's artifact layout, W_dec the oracle's decode of the
    packed bits (normalised RHT domain)."""
    key = ("tr", m, n, K)
    if key not in _CACHE:
        W = gauss_weight(m, n)
        bm, bn = O.block_decompose(m), O.block_decompose(n)
        su, sv = O.rht_signs(m, n, 42)
        Wt = O.rht_transform_weights(W, su, sv, bm, bn)
        wscale = float(np.sqrt((Wt ** 2).mean(dtype=np.float32))) * O.trellis_opt_scale()
        Wr = (Wt / np.float32(wscale)).astype(np.float32)
        packed, recon = ext.trellis_quantize_matrix(t(Wr), K)
        torch.cuda.synchronize()
        art = {"trellis_packed": packed.cpu().numpy(), "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
               "Wscale": np.float32(wscale), "blocks_m": bm, "blocks_n": bn}
        W_dec = O.decode_layer(art["trellis_packed"], m, n, fast=True)
        # the encoder's reconstruction is what the packed bits decode to
        assert np.array_equal(W_dec, recon.cpu().numpy())
        # ... and it is a 4-bit quantization of the weight, not noise: QTIP reports an MSE of about
        # 0.005 for the 3INST code at 4 bits on unit Gaussians
        assert O.rel_fro(W_dec, Wr) < 0.12, O.rel_fro(W_dec, Wr)
        _CACHE[key] = (W, art, W_dec)
    return _CACHE[key]


def trellis_args(art, m, n):
    from glq_amd import hadamard as H
    bn, bm = art["blocks_n"], art["blocks_m"]
    return (t(art["SV"]), t(art["SU"]), t(art["trellis_packed"]), torch.tensor(bn), torch.tensor(bm),
            H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), float(art["Wscale"]), n, m, n, m)


# ------------------------------------------------------------------ configs[1]: SmolLM3-3B shapes
@pytest.mark.parametrize("m,n", [(2048, 2048), (512, 2048), (11008, 2048), (2048, 11008)])
def test_trellis_smollm3_layer_whole_layer_oracle_and_quality_gates(ext, m, n):
    say("quantized smollm3", m, n)
    W, art, W_dec = trellis_layer(ext, m, n)
    su, sv = art["SU"].astype(np.float32), art["SV"].astype(np.float32)
    bn, bm = art["blocks_n"], art["blocks_m"]
    args = trellis_args(art, m, n)
    # dequantizer: every weight of the layer
    Wg = ext.glq_decompress_trellis_3inst_cuda(args[2], m, n)
    assert np.array_equal(Wg.float().cpu().numpy(), W_dec)
    # whole-layer forward, batch 1 and a few tokens (GEMV forms), bf16
    x = torch.randn(5, n, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    ref = O.linear_forward_rht(x.float().numpy(), W_dec * art["Wscale"], su, sv, bn, bm, n, m)
    for B in (1, 2, 5):
        y = ext.glq_fused_linear_trellis_3inst_cuda(x[:B].to(DEV), *args, out_dtype=torch.bfloat16)
        assert rel(y, ref[:B]) < TOL, (B, rel(y, ref[:B]))
        assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_cuda(x[:B].to(DEV), *args, out_dtype=torch.bfloat16))
    # gate: GEMV and batched product on RHT-domain activations against x @ W_dec.T
    xr = (torch.randn(9, n, generator=torch.Generator().manual_seed(7)) * 0.5).to(torch.float16)
    pref = xr.float().numpy() @ W_dec.T
    out = ext.glq_decode_matvec_trellis_3inst_cuda(xr[0].to(DEV), args[2], m, n)
    assert sqnr(pref[0], out.cpu().numpy()) > 40.0, sqnr(pref[0], out.cpu().numpy())
    outb = ext.glq_decode_matmul_trellis_3inst_cuda(xr.to(DEV), args[2], m, n)
    assert sqnr(pref, outb.cpu().numpy()) > 40.0, sqnr(pref, outb.cpu().numpy())
    assert torch.equal(outb[0], out)                         # row of the batch == GEMV, bit for bit
    # gate: the fused layer against the quantizer's reconstruction in the weight domain
    W_hat = to_weight_domain(W_dec * art["Wscale"], su, sv, bm, bn)
    xh = x.to(torch.float16)
    for B in (1, 4):
        y = ext.glq_fused_linear_trellis_3inst_cuda(xh[:B].to(DEV), *args)
        r = xh[:B].float().numpy() @ W_hat.T
        assert sqnr(r, y.float().cpu().numpy()) > 35.0, (B, sqnr(r, y.float().cpu().numpy()))
    # and against the unquantized layer: 4 bits keep well over 20 dB
    y = ext.glq_fused_linear_trellis_3inst_cuda(xh[:4].to(DEV), *args)
    assert sqnr(xh[:4].float().numpy() @ W.T, y.float().cpu().numpy()) > 20.0


def test_trellis_smollm3_group_calls_on_quantized_layers(ext):
    """q/k/v as one grouped call (the form bench.py times) against the oracle, whole outputs."""
    n = 2048
    shards, refs = [], []
    x = torch.randn(1, n, generator=torch.Generator().manual_seed(11)).to(torch.bfloat16)
    for m in (2048, 512):
        _, art, W_dec = trellis_layer(ext, m, n)
        refs.append(O.linear_forward_rht(x.float().numpy(), W_dec * art["Wscale"], art["SU"].astype(np.float32),
                                         art["SV"].astype(np.float32), art["blocks_n"], art["blocks_m"], n, m))
        shards.append((t(art["SV"]), t(art["SU"]), t(art["trellis_packed"]), float(art["Wscale"]), m, m))
    from glq_amd import hadamard as H
    bn = O.block_decompose(n)
    group = [shards[0], shards[1], shards[1]]                # q, k, v (k and v share one layer here)
    y = ext.glq_fused_linear_trellis_3inst_group(x.to(DEV), group, torch.tensor(bn), H.pack_block_meta(bn).to(DEV),
                                                 n, n, out_dtype=torch.bfloat16)
    ref = np.concatenate([refs[0], refs[1], refs[1]], axis=1)
    assert rel(y, ref) < TOL, rel(y, ref)


# ------------------------------------------------------------------ configs[2]: E8 two-stage
def e8_layer(ext, m, n):
    key = ("e8", m, n)
    if key not in _CACHE:
        W = gauss_weight(m, n)
        bm, bn = O.block_decompose(m), O.block_decompose(n)
        su, sv = O.rht_signs(m, n, 42)
        Wt = O.rht_transform_weights(W, su, sv, bm, bn)
        wscale = float(np.sqrt((Wt ** 2).mean(dtype=np.float32)))
        Wr = (Wt / np.float32(wscale)).astype(np.float32)
        table = t(O.e8_table())
        v = t(Wr).reshape(-1, 8)
        dec1, i1 = ext.e8_quantize(v, table)
        dec2, i2 = ext.e8_quantize((v - dec1) * 3.0, table)
        torch.cuda.synchronize()
        art = {"Qidxs": i1.reshape(m, n // 8).cpu().numpy().astype(np.uint16).view(np.int16),
               "Qidxs2": i2.reshape(m, n // 8).cpu().numpy().astype(np.uint16).view(np.int16),
               "inv_resid_scale": np.float32(1 / 3.0), "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
               "Wscale": np.float32(wscale), "blocks_m": bm, "blocks_n": bn}
        W_dec = O.e8_dequant(art["Qidxs"], art["Qidxs2"], 1 / 3.0)
        hat = (dec1 + dec2 / 3.0).reshape(m, n).cpu().numpy()
        assert np.allclose(W_dec, hat, atol=1e-6)
        assert O.rel_fro(W_dec, Wr) < 0.12, O.rel_fro(W_dec, Wr)   # two E8 stages: about 4 bits
        # the encoder on a sample of this very layer against the oracle's search
        rows = np.arange(0, m * n // 8, max(1, m * n // 8 // 2000))[:2000]
        _, oi = O.e8_quantize(Wr.reshape(-1, 8)[rows])
        assert np.array_equal(oi, i1.cpu().numpy()[rows])
        _CACHE[key] = (W, art, W_dec)
    return _CACHE[key]


def e8_forward(ext, x, art, m, n, dtype):
    from glq_amd import hadamard as H
    bn, bm = art["blocks_n"], art["blocks_m"]
    cb = e8_table_f16()
    q1, q2, _, _ = e8_prepared(ext, cb, art["Qidxs"], art["Qidxs2"])     # load-time step once, then looked up
    return ext.glq_fused_linear_block_diag_cuda(
        x, t(art["SV"]), t(art["SU"]), q1, cb, float(art["Wscale"]), n, m, n, m, torch.tensor(bn),
        torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), q2, cb,
        1 / 3.0, out_dtype=dtype)


@pytest.mark.parametrize("m,n", [(14336, 4096), (4096, 14336)])
def test_e8_two_stage_llama_mlp_whole_layer_oracle_and_quality_gates(ext, m, n):
    say("quantized e8", m, n)
    W, art, W_dec = e8_layer(ext, m, n)
    su, sv = art["SU"].astype(np.float32), art["SV"].astype(np.float32)
    bn, bm = art["blocks_n"], art["blocks_m"]
    x = torch.randn(16, n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    ref = O.linear_forward_rht(x.float().numpy(), W_dec * art["Wscale"], su, sv, bn, bm, n, m)
    xd = x.to(DEV)
    for M in (1, 4, 16):
        y = e8_forward(ext, xd[:M], art, m, n, torch.bfloat16)
        assert rel(y, ref[:M]) < TOL, (M, rel(y, ref[:M]))
        assert torch.equal(y, e8_forward(ext, xd[:M], art, m, n, torch.bfloat16))
    # gates: gather-matmul on RHT-domain activations against x @ W_dec.T, fused layer against W_hat
    xr = (torch.randn(16, n, generator=torch.Generator().manual_seed(7)) * 0.5).to(torch.float16)
    pref = xr.float().numpy() @ W_dec.T * art["Wscale"]
    cb = e8_table_f16()
    for M in (1, 4, 16):
        q1, q2, _, _ = e8_prepared(ext, cb, art["Qidxs"], art["Qidxs2"])
        out = ext.glq_dequant_matmul_cuda(xr[:M].to(DEV), q1, cb, float(art["Wscale"]), q2, cb, 1 / 3.0)
        assert sqnr(pref[:M], out.float().cpu().numpy()) > 40.0, (M, sqnr(pref[:M], out.float().cpu().numpy()))
    W_hat = to_weight_domain(W_dec * art["Wscale"], su, sv, bm, bn)
    xh = x.to(torch.float16)
    y = e8_forward(ext, xh[:4].to(DEV), art, m, n, torch.float16)
    r = xh[:4].float().numpy() @ W_hat.T
    assert sqnr(r, y.float().cpu().numpy()) > 35.0, sqnr(r, y.float().cpu().numpy())
    # two E8 stages at x3 keep about 20 dB against the unquantized layer
    assert sqnr(xh[:4].float().numpy() @ W.T, y.float().cpu().numpy()) > 18.0


# ------------------------------------------------------------------ configs[3]: 256 / 1024 / 4096 tokens
def _sample_rows(M):
    """Rows of every position class of a 128-token tile (first, last, middle, tile edges) and of
    the first, a middle and the last tile."""
    base = [0, 1, 15, 16, 63, 64, 65, 126, 127]
    rows = sorted({r + off for off in (0, (M // 256) * 128, M - 128) for r in base if 0 <= r + off < M})
    return np.array(rows)


@pytest.mark.parametrize("m,n", [(14336, 4096), (4096, 14336)])
def test_trellis_prefill_quantized_layer_up_to_4096_tokens(ext, m, n, monkeypatch):
    say("quantized trellis prefill", m, n)
    monkeypatch.setattr(ext, "TRELLIS_BATCH_MAX", 1 << 30)     # every size on the packed stream
    _, art, W_dec = trellis_layer(ext, m, n)
    su, sv = art["SU"].astype(np.float32), art["SV"].astype(np.float32)
    args = trellis_args(art, m, n)
    x = torch.randn(4096, n, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    xd = x.to(DEV)
    Ws = (W_dec * art["Wscale"]).astype(np.float32)
    ys = {}
    for M in (24, 64, 256, 1024, 4096):                       # 24, 64: the small-tile kernel
        rows = _sample_rows(M)
        ref = O.linear_forward_rht(x[rows].float().numpy(), Ws, su, sv, art["blocks_n"], art["blocks_m"], n, m)
        y = ext.glq_fused_linear_trellis_3inst_cuda(xd[:M], *args, out_dtype=torch.bfloat16)
        assert y.shape == (M, m)
        assert rel(y[torch.from_numpy(rows).to(DEV)], ref) < TOL, (M, rel(y[torch.from_numpy(rows).to(DEV)], ref))
        assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_cuda(xd[:M], *args, out_dtype=torch.bfloat16))
        ys[M] = y
    # every row of the 4096-token call against the 1024-token call (other route or other K split)
    assert rel(ys[4096][:1024], ys[1024].float().cpu().numpy()) < 6e-3
    assert rel(ys[1024][:256], ys[256].float().cpu().numpy()) < 6e-3
    assert rel(ys[256][:64], ys[64].float().cpu().numpy()) < 6e-3
    assert rel(ys[64][:24], ys[24].float().cpu().numpy()) < 6e-3
    # the reference's quality gate at the full prefill size
    W_hat = to_weight_domain(Ws, su, sv, art["blocks_m"], art["blocks_n"])
    rows = _sample_rows(4096)
    r = x[rows].float().numpy() @ W_hat.T
    assert sqnr(r, ys[4096][torch.from_numpy(rows).to(DEV)].float().cpu().numpy()) > 35.0
    # the route the library takes by itself above 2048 tokens (dequantize + library GEMM): same result
    monkeypatch.setattr(ext, "TRELLIS_BATCH_MAX", 2048)
    yl = ext.glq_fused_linear_trellis_3inst_cuda(xd, *args, out_dtype=torch.bfloat16)
    assert rel(yl, ys[4096].float().cpu().numpy()) < 6e-3
    assert sqnr(r, yl[torch.from_numpy(rows).to(DEV)].float().cpu().numpy()) > 35.0


@pytest.mark.parametrize("m,n", [(14336, 4096), (4096, 14336)])
def test_e8_prefill_quantized_layer_up_to_4096_tokens(ext, m, n, monkeypatch):
    say("quantized e8 prefill", m, n)
    monkeypatch.setattr(ext, "E8_BATCH_MAX", 1 << 30)          # every size on the compressed indices
    _, art, W_dec = e8_layer(ext, m, n)
    su, sv = art["SU"].astype(np.float32), art["SV"].astype(np.float32)
    x = torch.randn(4096, n, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    xd = x.to(DEV)
    Ws = (W_dec * art["Wscale"]).astype(np.float32)
    ys = {}
    for M in (24, 64, 256, 1024, 4096):                       # up to 256: the small-tile kernel
        rows = _sample_rows(M)
        ref = O.linear_forward_rht(x[rows].float().numpy(), Ws, su, sv, art["blocks_n"], art["blocks_m"], n, m)
        y = e8_forward(ext, xd[:M], art, m, n, torch.bfloat16)
        assert y.shape == (M, m)
        assert rel(y[torch.from_numpy(rows).to(DEV)], ref) < TOL, (M, rel(y[torch.from_numpy(rows).to(DEV)], ref))
        assert torch.equal(y, e8_forward(ext, xd[:M], art, m, n, torch.bfloat16))
        ys[M] = y
    assert rel(ys[4096][:1024], ys[1024].float().cpu().numpy()) < 6e-3
    assert rel(ys[1024][:256], ys[256].float().cpu().numpy()) < 6e-3
    W_hat = to_weight_domain(Ws, su, sv, art["blocks_m"], art["blocks_n"])
    rows = _sample_rows(4096)
    r = x[rows].float().numpy() @ W_hat.T
    assert sqnr(r, ys[4096][torch.from_numpy(rows).to(DEV)].float().cpu().numpy()) > 35.0
    # the tile kernel on the indices themselves (no folded streams): the same operands and fp32 sums, where the
    # folded form hands fp16 sums to the output transform from 257 tokens on (the matmul entry, fp32 on both,
    # is bit-identical: test_gpu_e8_fold.py)
    monkeypatch.setattr(ext, "E8_FOLD", False)
    assert rel(e8_forward(ext, xd, art, m, n, torch.bfloat16), ys[4096].float().cpu().numpy()) < 2e-3
    monkeypatch.setattr(ext, "E8_FOLD", True)
    # the library route, the default above 4096 tokens (above 1024 without folded streams)
    monkeypatch.setattr(ext, "E8_BATCH_MAX", 1024)
    monkeypatch.setattr(ext, "E8_FOLD_BATCH_MAX", 1024)
    yl = e8_forward(ext, xd, art, m, n, torch.bfloat16)
    assert rel(yl, ys[4096].float().cpu().numpy()) < 6e-3
    assert sqnr(r, yl[torch.from_numpy(rows).to(DEV)].float().cpu().numpy()) > 35.0
