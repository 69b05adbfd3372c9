"""Trellis-3INST kernels against the oracle (needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, rel, say, t

pytestmark = pytest.mark.gpu

TOL = 1e-2          # relative Frobenius bound on layer outputs (bf16/fp16 I/O, fp32 accumulate)


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_decompress_bit_exact_on_reference_vectors(ext, golden, K):
    g = golden("trellis_storage")
    say("decompress golden K", K)
    W = ext.glq_decompress_trellis_3inst_cuda(t(g[f"K{K}_packed"]), 64, 128, allow_r1=(K == 1))
    assert W.dtype == torch.float16 and W.shape == (64, 128)
    assert np.array_equal(W.cpu().numpy().view(np.uint16), g[f"K{K}_decoded"].view(np.uint16))


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("m,n", [(64, 128), (128, 256), (256, 512), (96, 192)])
def test_decompress_bit_exact_random_bits(ext, m, n, K):
    say("decompress random", m, n, K)
    p = O.random_packed(m, n, K, seed=m + K)
    W = ext.glq_decompress_trellis_3inst_cuda(t(p), m, n)
    assert np.array_equal(W.float().cpu().numpy(), O.decode_layer(p, m, n))


def test_decompress_full_size_strips(ext):
    """2048 x 11008 at 4 bpw (SmolLM3 down_proj): first and last 32-row strips bit-exact;
    every other strip checked through the value histogram of 3INST (all outputs must be
    members of the 65536-entry LUT)."""
    m, n, K = 2048, 11008, 4
    say("decompress full size", m, n, K)
    p = O.random_packed(m, n, K, seed=5)
    W = ext.glq_decompress_trellis_3inst_cuda(t(p), m, n).cpu().numpy()
    per_strip = 2 * (n // 16)
    for mp in (0, m // 32 - 1):
        strip = p[mp * per_strip:(mp + 1) * per_strip]
        assert np.array_equal(W[32 * mp:32 * mp + 32].astype(np.float32), O.decode_layer(strip, 32, n))
    lut = np.unique(O.lut_3inst().view(np.uint16))
    assert np.isin(W.view(np.uint16), lut).all()


def test_r1_refused_unless_residual(ext):
    p = t(O.random_packed(64, 128, 1, 0))
    with pytest.raises(RuntimeError, match="bits/weight"):
        ext.glq_decompress_trellis_3inst_cuda(p, 64, 128)
    x = torch.zeros(128, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="bits/weight"):
        ext.glq_decode_matvec_trellis_3inst_cuda(x, p, 64, 128)
    with pytest.raises(RuntimeError, match="bits/weight"):
        ext.glq_decompress_trellis_3inst_cuda(t(np.zeros((32, 80), np.int16)), 64, 128)
    with pytest.raises(RuntimeError, match="rows"):
        ext.glq_decompress_trellis_3inst_cuda(t(O.random_packed(64, 128, 2, 0)), 64, 256)
    with pytest.raises(RuntimeError, match="% 32"):
        ext.glq_decompress_trellis_3inst_cuda(t(O.random_packed(48, 128, 2, 0)), 48, 128)


@pytest.mark.parametrize("K", [2, 3, 4])
@pytest.mark.parametrize("m,n", [(256, 512), (512, 2048), (64, 128)])
def test_gemv_matches_oracle_and_is_deterministic(ext, m, n, K):
    say("gemv", m, n, K)
    p = O.random_packed(m, n, K, seed=m + 1)
    W = O.decode_layer(p, m, n)
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(n) * 0.5).astype(np.float16)
    ref = x.astype(np.float32) @ W.T * np.float32(0.0137)
    pt, xt = t(p), t(x)
    out = ext.glq_decode_matvec_trellis_3inst_cuda(xt, pt, m, n, 0.0137)
    assert out.shape == (m,) and out.dtype == torch.float32
    assert rel(out, ref) < 2e-3, rel(out, ref)
    again = ext.glq_decode_matvec_trellis_3inst_cuda(xt, pt, m, n, 0.0137)
    assert torch.equal(out, again)


@pytest.mark.parametrize("K2", [1, 2, 4])
def test_gemv_accumulate_stage2(ext, K2):
    m, n = 128, 256
    say("gemv accum", K2)
    p1, p2 = O.random_packed(m, n, 4, 1), O.random_packed(m, n, K2, 2)
    x = (np.random.default_rng(3).standard_normal(n)).astype(np.float16)
    W = O.decode_layer_nstage([p1, p2], [1.0, 0.3], m, n)
    ref = x.astype(np.float32) @ W.T * np.float32(0.5)
    out = ext.glq_decode_matvec_trellis_3inst_cuda(t(x), t(p1), m, n, 0.5)
    ext.glq_decode_matvec_trellis_3inst_cuda(t(x), t(p2), m, n, 0.5 * 0.3, out=out, accum=True)
    assert rel(out, ref) < 2e-3
    with pytest.raises(RuntimeError, match="accumulate"):
        ext.glq_decode_matvec_trellis_3inst_cuda(t(x), t(p2), m, n, 1.0, accum=True)


@pytest.mark.parametrize("B", [1, 2, 4, 7, 8, 9, 16])
def test_matmul_batched_rows_equal_gemv(ext, B):
    m, n, K = 256, 512, 4
    say("matmul", B)
    p = O.random_packed(m, n, K, seed=21)
    W = O.decode_layer(p, m, n)
    x = (np.random.default_rng(B).standard_normal((B, n)) * 0.5).astype(np.float16)
    pt, xt = t(p), t(x)
    out = ext.glq_decode_matmul_trellis_3inst_cuda(xt, pt, m, n, 1.0)
    assert out.shape == (B, m)
    assert rel(out, x.astype(np.float32) @ W.T) < 2e-3
    for b in range(B):
        gv = ext.glq_decode_matvec_trellis_3inst_cuda(xt[b].contiguous(), pt, m, n, 1.0)
        assert torch.equal(out[b], gv), f"row {b} differs from the GEMV"
    assert torch.equal(out, ext.glq_decode_matmul_trellis_3inst_cuda(xt, pt, m, n, 1.0))


@pytest.mark.parametrize("m,n,B,K", [(64, 4096, 17, 4), (96, 4096, 33, 2), (128, 1024, 64, 3), (96, 192, 65, 4),
                                     (320, 1024, 130, 2), (256, 512, 257, 3), (64, 2048, 128, 4)])
def test_matmul_large_batch_tiles(ext, m, n, B, K):
    """From 17 tokens on: the 128-token tiles (one wave per 64 rows, K split only to fill the
    chip): odd m/32, ragged token tiles, direct and accumulating outputs."""
    say("matmul tiles", m, n, B, K)
    p1, p2 = O.random_packed(m, n, K, seed=3), O.random_packed(m, n, 1, seed=4)
    W1, W2 = O.decode_layer(p1, m, n), O.decode_layer(p2, m, n)
    x = (np.random.default_rng(B).standard_normal((B, n)) * 0.5).astype(np.float16)
    xt = t(x)
    out = ext.glq_decode_matmul_trellis_3inst_cuda(xt, t(p1), m, n, 0.25)
    ref1 = x.astype(np.float32) @ W1.T * np.float32(0.25)
    assert out.shape == (B, m) and rel(out, ref1) < 2e-3, rel(out, ref1)
    assert torch.equal(out, ext.glq_decode_matmul_trellis_3inst_cuda(xt, t(p1), m, n, 0.25))
    ext.glq_decode_matmul_trellis_3inst_cuda(xt, t(p2), m, n, 0.125, out=out, accum=True)
    ref = ref1 + x.astype(np.float32) @ W2.T * np.float32(0.125)
    assert rel(out, ref) < 2e-3, rel(out, ref)
    # rows agree with the small-batch kernel up to rounding: the tiles add a weight's two
    # fp16 halves before the multiply (as the dequantizer does), the small-batch kernel after
    rows = ext.glq_decode_matmul_trellis_3inst_cuda(xt[:3].contiguous(), t(p1), m, n, 0.25)
    first = ext.glq_decode_matmul_trellis_3inst_cuda(xt, t(p1), m, n, 0.25)[:3]
    assert rel(first, rows) < 1e-3


def _layer_args(art, m, n, dtype):
    from glq_amd import hadamard as H
    bn, bm = art["blocks_n"], art["blocks_m"]
    return dict(
        sv=t(art["SV"].astype(np.float16)), su=t(art["SU"].astype(np.float16)),
        packed=t(art["trellis_packed"]),
        packed2=t(art["trellis_packed2"]) if "trellis_packed2" in art else None,
        bn=torch.tensor(bn, dtype=torch.int64), bm=torch.tensor(bm, dtype=torch.int64),
        bn_meta=H.pack_block_meta(bn).to(DEV), bm_meta=H.pack_block_meta(bm).to(DEV),
        wscale=float(art["Wscale"]), inv2=float(art.get("inv_resid_scale2", 0.0)))


@pytest.mark.parametrize("tag", ["k2", "k4", "k4k2"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_linear_on_reference_layers(ext, golden, tag, dtype):
    g = golden("trellis_layer")
    say("fused golden", tag, dtype)
    W = g[f"{tag}_W"]
    m, n = W.shape
    art = {k: g[f"{tag}_{k}"] for k in ("trellis_packed", "SU", "SV", "Wscale")}
    art["blocks_m"], art["blocks_n"] = list(g[f"{tag}_blocks_m"]), list(g[f"{tag}_blocks_n"])
    if tag == "k4k2":
        art["trellis_packed2"] = g[f"{tag}_trellis_packed2"]
        art["inv_resid_scale2"] = g[f"{tag}_inv_resid_scale2"]
    a = _layer_args(art, m, n, dtype)
    x = torch.from_numpy(g[f"{tag}_x"]).to(dtype)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    if a["packed2"] is None:
        y = ext.glq_fused_linear_trellis_3inst_cuda(
            x.to(DEV), a["sv"], a["su"], a["packed"], a["bn"], a["bm"], a["bn_meta"], a["bm_meta"],
            a["wscale"], n, m, n, m, out_dtype=dtype)
    else:
        y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
            x.to(DEV), a["sv"], a["su"], a["packed"], a["packed2"], a["bn"], a["bm"], a["bn_meta"],
            a["bm_meta"], a["wscale"], a["inv2"], n, m, n, m, out_dtype=dtype)
    assert y.dtype == dtype and y.shape == (x.shape[0], m)
    assert rel(y, ref) < TOL, rel(y, ref)
    assert rel(y, g[f"{tag}_y"]) < TOL            # the reference's own CPU output (fp32 input)


def test_fused_refuses_half_configured_stage2(ext, golden):
    g = golden("trellis_layer")
    art = {k: g[f"k4k2_{k}"] for k in ("trellis_packed", "trellis_packed2", "SU", "SV", "Wscale")}
    art["blocks_m"], art["blocks_n"] = list(g["k4k2_blocks_m"]), list(g["k4k2_blocks_n"])
    a = _layer_args(art, 64, 128, torch.float16)
    x = torch.zeros(1, 128, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="half-configured"):
        ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
            x, a["sv"], a["su"], a["packed"], a["packed2"], a["bn"], a["bm"], a["bn_meta"],
            a["bm_meta"], a["wscale"], 0.0, 128, 64, 128, 64)


@pytest.mark.parametrize("m,n", [(2048, 2048), (512, 2048), (11008, 2048), (2048, 11008)])
def test_fused_linear_smollm3_shapes(ext, m, n):
    """Config-2 shapes, 4 bpw, bf16 activations, batch 1: random code bits (every bit
    pattern is a valid stream) with seeded signs; checked against the oracle through two
    sampled 32-row strips of the RHT-domain product and through linearity of the layer."""
    from glq_amd import hadamard as H
    say("fused smollm3", m, n)
    K = 4
    p = O.random_packed(m, n, K, seed=m % 97)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    wscale = 0.02 * O.trellis_opt_scale()
    rng = np.random.default_rng(1)
    x = torch.from_numpy(rng.standard_normal((1, n)).astype(np.float32)).to(torch.bfloat16)
    args = (t(sv.astype(np.float16)), t(su.astype(np.float16)), t(p),
            torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV),
            H.pack_block_meta(bm).to(DEV), wscale, n, m, n, m)
    y = ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), *args, out_dtype=torch.bfloat16)
    # RHT-domain product from the same entry family, stopped before the output transform
    yr = torch.zeros(1, m, dtype=torch.float32, device=DEV)
    ext.glq_fused_linear_trellis_3inst_yrht_cuda(x.to(DEV), args[0], args[2], args[3], args[5],
                                                 wscale, n, n, m, yr, 0)
    x_rht = O.block_diag_fht(x.float().numpy() * sv[None], bn)
    per_strip = 2 * (n // 16)
    for mp in (0, m // 64, m // 32 - 1):
        Wn = O.decode_layer(p[mp * per_strip:(mp + 1) * per_strip], 32, n)
        ref = x_rht @ Wn.T * np.float32(wscale)
        assert rel(yr[:, 32 * mp:32 * mp + 32], ref) < 5e-3, (mp, rel(yr[:, 32 * mp:32 * mp + 32], ref))
    # output transform of the full row, applied by the oracle to the kernel's y_rht
    y_ref = (O.block_diag_fht(yr.cpu().numpy(), bm) * su[None])[:, :m]
    assert rel(y, y_ref) < TOL
    # determinism, and linearity of the whole layer (scaling by 2 is exact up to fp16
    # subnormals of the transformed activations)
    assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), *args, out_dtype=torch.bfloat16))
    y2 = ext.glq_fused_linear_trellis_3inst_cuda((x * 2).to(DEV), *args, out_dtype=torch.bfloat16)
    assert rel(y2, y.float() * 2) < 1e-3


@pytest.mark.parametrize("outs,n,B,dtype", [((2048, 512, 512), 2048, 1, torch.bfloat16),
                                            ((11008, 11008), 2048, 1, torch.bfloat16),
                                            ((96, 320, 64, 2048), 960, 3, torch.float16),
                                            ((14336, 14336), 4096, 2, torch.bfloat16),
                                            ((6144, 6144, 1024), 4096, 4, torch.float16),
                                            ((2048, 512, 512), 2048, 5, torch.bfloat16),
                                            ((11008, 11008), 2048, 16, torch.float16),
                                            ((96, 320, 64, 2048), 960, 9, torch.bfloat16),
                                            ((2048, 512, 512), 2048, 17, torch.bfloat16),
                                            ((11008, 11008), 2048, 40, torch.float16),
                                            ((4096, 512), 8192, 64, torch.bfloat16),
                                            ((96, 320, 64, 2048), 960, 33, torch.bfloat16)])
def test_grouped_layers_match_per_layer_calls(ext, outs, n, B, dtype):
    """Fused q/k/v and gate/up: several separately quantized layers on one x in two launches
    equal the per-layer fused linears up to the rounding of a different K split.  The two large
    groups at 2-4 tokens take the separate input transform (one per distinct sign vector: the
    last case gives its first two layers the same one)."""
    from glq_amd import hadamard as H
    say("group", outs, n, B)
    bn = O.block_decompose(n)
    bnt, bnm = torch.tensor(bn), H.pack_block_meta(bn).to(DEV)
    rng = np.random.default_rng(len(outs))
    x = torch.from_numpy(rng.standard_normal((B, n)).astype(np.float32)).to(dtype).to(DEV)
    shards, singles = [], []
    for i, m in enumerate(outs):
        p = t(O.random_packed(m, n, 4, seed=10 + i))
        su, sv = O.rht_signs(m, n, 100 + i)
        su, sv = t(su.astype(np.float16)), t(sv.astype(np.float16))
        if i == 1 and len(outs) == 3 and outs[0] == outs[1]:
            sv = shards[0][0]                                  # same tensor: one transform serves both
        wscale = 0.02 + 0.001 * i
        bm = O.block_decompose(m)
        shards.append((sv, su, p, wscale, m, m))
        singles.append(ext.glq_fused_linear_trellis_3inst_cuda(
            x, sv, su, p, bnt, torch.tensor(bm), bnm, H.pack_block_meta(bm).to(DEV), wscale, n, m, n, m,
            out_dtype=dtype))
    y = ext.glq_fused_linear_trellis_3inst_group(x, shards, bnt, bnm, n, n, out_dtype=dtype)
    assert y.shape == (B, sum(outs)) and y.dtype == dtype
    off = 0
    for m, ref in zip(outs, singles):
        assert rel(y[:, off:off + m], ref.float().cpu().numpy()) < 4e-3, (m, rel(y[:, off:off + m], ref.float().cpu().numpy()))
        off += m
    assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_group(x, shards, bnt, bnm, n, n, out_dtype=dtype))
    with pytest.raises(RuntimeError, match="x must be"):
        ext.glq_fused_linear_trellis_3inst_group(x.float(), shards, bnt, bnm, n, n, out_dtype=dtype)


def test_yrht_shards_equal_sequential(ext):
    """Fused q/k/v: three shards write their RHT-domain rows into one buffer and one
    shard-batched output transform finishes them; equals the per-shard fused op."""
    from glq_amd import hadamard as H
    n = 256
    shards = [(128, 4), (64, 4), (64, 2)]
    say("yrht shards")
    total = sum(m for m, _ in shards)
    x = torch.randn(3, n, dtype=torch.float16, device=DEV)
    bn = O.block_decompose(n)
    bn_t, bn_meta = torch.tensor(bn), H.pack_block_meta(bn).to(DEV)
    y_rht = torch.zeros(3, total, dtype=torch.float32, device=DEV)
    su_all, seq, col = [], [], 0
    for i, (m, K) in enumerate(shards):
        p = t(O.random_packed(m, n, K, seed=i))
        su, sv = O.rht_signs(m, n, 100 + i)
        su_t, sv_t = t(su.astype(np.float16)), t(sv.astype(np.float16))
        bm = O.block_decompose(m)
        seq.append(ext.glq_fused_linear_trellis_3inst_cuda(
            x, sv_t, su_t, p, bn_t, torch.tensor(bm), bn_meta, H.pack_block_meta(bm).to(DEV),
            0.03, n, m, n, m))
        ext.glq_fused_linear_trellis_3inst_yrht_cuda(x, sv_t, p, bn_t, bn_meta, 0.03, n, n, m, y_rht, col)
        su_all.append(su_t)
        col += m
    meta = H.pack_shard_meta([O.block_decompose(m) for m, _ in shards]).to(DEV)
    y = torch.empty(3, total, dtype=torch.float16, device=DEV)
    ext.glq_output_rht_shards_cuda(y_rht, torch.cat(su_all), y, total, meta, 128)
    assert torch.equal(y, torch.cat(seq, dim=1))


def test_fusein_gemv_matches_unfused_pipeline(ext):
    from glq_amd import hadamard as H
    m, n, inf = 64, 2048, 2000
    say("fusein")
    p = t(O.random_packed(m, n, 3, seed=51))
    x_raw = (torch.randn(inf, device=DEV) * 0.5).to(torch.float16)
    sv = torch.where(torch.rand(n, device=DEV) < 0.5, -1.0, 1.0).to(torch.float16)
    x_rht = torch.empty(1, n, dtype=torch.float32, device=DEV)
    ext.glq_input_rht_cuda(x_raw.unsqueeze(0), sv, x_rht, inf, inf, 1.0 / np.sqrt(n), n, 11)
    ref = ext.glq_decode_matvec_trellis_3inst_cuda(x_rht[0].half(), p, m, n, 0.01371)
    out = ext.glq_decode_matvec_trellis_3inst_fusein_cuda(x_raw, sv, p, m, n, inf, 0.01371)
    # the fused kernel builds its slice of the transform in a different summation order
    assert rel(out, ref) < 1e-3, rel(out, ref)
    assert torch.equal(out, ext.glq_decode_matvec_trellis_3inst_fusein_cuda(x_raw, sv, p, m, n, inf, 0.01371))
