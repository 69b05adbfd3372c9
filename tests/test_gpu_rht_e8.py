"""RHT kernels and the E8 shell path against the oracle (needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t, e8_prepared

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e


@pytest.mark.parametrize("n,inf", [(16, 16), (64, 50), (2048, 2048), (2048, 2000), (16384, 16384),
                                   (32768, 30000)])
def test_input_rht_pow2(ext, n, inf):
    say("input_rht", n, inf)
    rng = np.random.default_rng(n)
    x = rng.standard_normal((3, inf)).astype(np.float16)
    sv = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    out = torch.empty(3, n, dtype=torch.float32, device=DEV)
    ext.glq_input_rht_cuda(t(x), t(sv), out, inf, inf, 1.0 / np.sqrt(n), n, int(np.log2(n)))
    xp = np.zeros((3, n), np.float32)
    xp[:, :inf] = x
    ref = O.fht(xp * sv.astype(np.float32)[None])
    assert np.allclose(out.cpu().numpy(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("B", [2, 70])       # few tokens: 1024-point slices; many: whole blocks
@pytest.mark.parametrize("n,inf,dtype", [(960, 960, torch.float16), (11008, 11008, torch.bfloat16),
                                         (14336, 14000, torch.bfloat16), (160, 160, torch.float16),
                                         (49152, 49152, torch.float16)])
def test_input_output_rht_blockdiag(ext, n, inf, dtype, B):
    from glq_amd import hadamard as H
    say("blockdiag rht", n, inf, dtype, B)
    blocks = O.block_decompose(n)
    x = torch.randn(B, inf).to(dtype)
    rng = np.random.default_rng(n)
    sv = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    out = torch.empty(B, n, dtype=torch.float32, device=DEV)
    ext.glq_input_rht_blockdiag_cuda(x.to(DEV), t(sv), out, inf, n, torch.tensor(blocks),
                                     H.pack_block_meta(blocks).to(DEV))
    xp = np.zeros((B, n), np.float32)
    xp[:, :inf] = x.float().numpy()
    ref = O.block_diag_fht(xp * sv.astype(np.float32)[None], blocks)
    assert np.allclose(out.cpu().numpy(), ref, rtol=1e-5, atol=2e-5)
    # output side: FHT * su, unpad, cast
    y = torch.empty(B, inf, dtype=dtype, device=DEV)
    ext.glq_output_rht_blockdiag_cuda(out, t(sv), y, inf, n, torch.tensor(blocks),
                                      H.pack_block_meta(blocks).to(DEV))
    yref = (O.block_diag_fht(ref, blocks) * sv.astype(np.float32)[None])[:, :inf]
    assert rel(y, yref) < 5e-3
    if inf == n:                                     # H(H(x sv)) sv == x
        assert rel(y, x.float().numpy()) < 5e-3


def test_rht_refusals(ext):
    x = torch.zeros(1, 96, dtype=torch.float16, device=DEV)
    sv = torch.ones(96, dtype=torch.float16, device=DEV)
    out = torch.empty(1, 96, dtype=torch.float32, device=DEV)
    with pytest.raises(RuntimeError, match="power of two"):
        ext.glq_input_rht_blockdiag_cuda(x, sv, out, 96, 96, torch.tensor([96]), None)
    with pytest.raises(RuntimeError, match="sum"):
        from glq_amd import hadamard as H
        ext.glq_input_rht_blockdiag_cuda(x, sv, out, 96, 96, torch.tensor([64, 16]),
                                         H.pack_block_meta([64, 16]).to(DEV))


# ------------------------------------------------------------------- E8 shell
def _rand_idx(rng, m, nb):
    return rng.integers(0, 65536, size=(m, nb)).astype(np.uint16).view(np.int16)


@pytest.mark.parametrize("m,n", [(32, 64), (96, 160), (960, 960), (100, 72)])
@pytest.mark.parametrize("stages", [1, 2, 4])
def test_e8_dequant_matmul_matches_oracle(ext, m, n, stages):
    say("e8 matmul", m, n, stages)
    rng = np.random.default_rng(m + stages)
    cb = e8_table_f16()
    q = [_rand_idx(rng, m, n // 8) for _ in range(4)]
    q[0][0, 0] = 0
    q[0][0, 1] = -1                                   # index 65535
    sc = [0.0, 0.0, 0.0]
    for s in range(1, stages):
        sc[s - 1] = [1 / 3.0, 1 / 9.0, 1 / 27.0][s - 1]
    B = 3
    x = (rng.standard_normal((B, n)) * 0.5).astype(np.float16)
    W = O.e8_dequant(q[0], q[1], sc[0], q[2], sc[1], q[3], sc[2])
    ref = x.astype(np.float32) @ W.T * np.float32(0.021)
    out = ext.glq_dequant_matmul_cuda(t(x), t(q[0]), cb, 0.021, t(q[1]), cb, sc[0], None, t(q[2]), cb,
                                      sc[1], t(q[3]), cb, sc[2])
    assert out.shape == (B, m) and out.dtype == torch.float32
    assert rel(out, ref) < 1e-3, rel(out, ref)
    out2 = ext.glq_dequant_matmul_cuda(t(x), t(q[0]), cb, 0.021, t(q[1]), cb, sc[0], None, t(q[2]), cb,
                                       sc[1], t(q[3]), cb, sc[2])
    assert torch.equal(out, out2)
    gv = ext.glq_dequant_matvec_cuda(t(x[1]), t(q[0]), cb, 0.021, t(q[1]), cb, sc[0])
    if stages <= 2:
        assert torch.equal(gv, out[1])


@pytest.mark.parametrize("m,n,B", [(96, 160, 1), (960, 960, 8), (2048, 2048, 5), (2048, 2048, 40)])
def test_e8_packed_table_variants(ext, m, n, B):
    """The single-stage entries that take the reference's 4-bit `codebook_packed` buffer
    (glq/inference_kernel.py:1047-1054) give what the fp16-table entries give, bit for bit,
    and match the oracle; a word with a code above 12 is refused."""
    say("e8 packed table", m, n, B)
    rng = np.random.default_rng(m + B)
    q = _rand_idx(rng, m, n // 8)
    q[0, 0], q[0, 1] = 0, -1
    x = (rng.standard_normal((B, n)) * 0.5).astype(np.float16)
    cbp = t(O.e8_nibbles().view(np.int32))             # == the reference's codebook_packed
    out = ext.glq_dequant_matmul_packed_cuda(t(x), t(q), cbp, 0.021)
    ref = x.astype(np.float32) @ O.e8_dequant(q).T * np.float32(0.021)
    assert out.shape == (B, m) and out.dtype == torch.float32
    assert rel(out, ref) < 1e-3, rel(out, ref)
    assert torch.equal(out, ext.glq_dequant_matmul_cuda(t(x), t(q), e8_table_f16(), 0.021))
    gv = ext.glq_dequant_matvec_packed_cuda(t(x[0]), t(q), cbp, 0.021)
    assert gv.shape == (m,) and torch.equal(gv, ext.glq_dequant_matvec_cuda(t(x[0]), t(q), e8_table_f16(), 0.021))
    from glq_amd import custom_ops
    custom_ops.register()
    assert torch.equal(torch.ops.glq.dequant_matmul_packed(t(x), t(q), cbp, 0.021), out)
    assert torch.equal(torch.ops.glq.dequant_matvec_packed(t(x[0]), t(q), cbp, 0.021), gv)
    bad = cbp.clone()
    bad[7] = 0x0000000D
    with pytest.raises(RuntimeError, match="code above 12"):
        ext.glq_dequant_matmul_packed_cuda(t(x), t(q), bad, 0.021)
    with pytest.raises(RuntimeError, match="65536"):
        ext.glq_dequant_matmul_packed_cuda(t(x), t(q), cbp[:256].contiguous(), 0.021)


def test_large_transform_op_names(ext):
    """`input_rht_triton` / `output_rht_triton` are the names the vLLM call sites use above
    16384 points (glq_vllm/linear_method.py:470-473, 506-518); same kernels, same results."""
    from glq_amd import custom_ops
    custom_ops.register()
    n, feat, B = 32768, 30000, 2
    say("large transform op names", n)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((B, feat)).astype(np.float16)
    sgn = (rng.integers(0, 2, n) * 2 - 1).astype(np.float16)
    a = torch.empty(B, n, dtype=torch.float32, device=DEV)
    b = torch.empty_like(a)
    r = float(1.0 / np.sqrt(n))
    torch.ops.glq.input_rht(t(x), t(sgn), a, feat, feat, r, n, 15)
    torch.ops.glq.input_rht_triton(t(x), t(sgn), b, feat, feat, r, n, 15)
    assert torch.equal(a, b)
    xp = np.zeros((B, n), np.float32)
    xp[:, :feat] = x.astype(np.float32)
    ref = O.fht(xp * sgn.astype(np.float32)[None, :])
    assert rel(a, ref) < 1e-5, rel(a, ref)
    ya = torch.empty(B, feat, dtype=torch.float16, device=DEV)
    yb = torch.empty_like(ya)
    torch.ops.glq.output_rht(a, t(sgn), ya, feat, n, 15, r)
    torch.ops.glq.output_rht_triton(a, t(sgn), yb, feat, n, 15, r)
    assert torch.equal(ya, yb)
    back = (O.fht(ref) * sgn.astype(np.float32)[None, :])[:, :feat]
    assert rel(ya, back) < 2e-3, rel(ya, back)


@pytest.mark.parametrize("m,n,B,stages", [(2048, 2048, 1, 1), (2048, 2048, 3, 2), (2100, 2048, 16, 2),
                                          (1024, 4160, 1, 4), (4096, 1024, 9, 3), (512, 8192, 4, 2),
                                          (2048, 2048, 40, 2), (1024, 4160, 33, 4), (2100, 2048, 17, 1)])
def test_e8_large_layers_lds_table(ext, m, n, B, stages):
    """Layers of 4M weights and more: the table prefix sits in LDS, the tail comes from L2.
    Up to 16 tokens the products run on MFMA straight from the indices; above, the tile kernel
    decodes them once per 128-row x 512-token tile (widths that are multiples of 256; others are
    dequantized once for a library GEMM).  Half of the indices are drawn from
    the low shells, half uniformly, and the extremes are planted."""
    say("e8 large", m, n, B, stages)
    rng = np.random.default_rng(m + n + B)
    cb = e8_table_f16()
    q = []
    for s in range(4):
        lo = rng.integers(0, 30000, size=(m, n // 8))
        hi = rng.integers(0, 65536, size=(m, n // 8))
        q.append(np.where(rng.random((m, n // 8)) < 0.5, lo, hi).astype(np.uint16).view(np.int16))
    q[0][0, 0] = 0
    q[0][0, 1] = -1
    q[0][m - 1, n // 8 - 1] = -1
    sc = [0.0, 0.0, 0.0]
    for s in range(1, stages):
        sc[s - 1] = [1 / 3.0, 1 / 9.0, 1 / 27.0][s - 1]
    x = (rng.standard_normal((B, n)) * 0.5).astype(np.float16)
    W = O.e8_dequant(q[0], q[1], sc[0], q[2], sc[1], q[3], sc[2])
    ref = x.astype(np.float32) @ W.T * np.float32(0.021)
    d = e8_prepared(ext, cb, *q[:stages])                         # the load-time step: folded streams where they serve
    d += [t(q[s]) for s in range(stages, 4)]                      # absent stages (scale 0) are never read
    args = (d[0], cb, 0.021, d[1], cb, sc[0], None, d[2], cb, sc[1], d[3], cb, sc[2])
    out = ext.glq_dequant_matmul_cuda(t(x), *args)
    assert out.shape == (B, m) and rel(out, ref) < 1e-3, rel(out, ref)
    assert torch.equal(out, ext.glq_dequant_matmul_cuda(t(x), *args))


def test_e8_large_layer_small_secondary_table(ext):
    rng = np.random.default_rng(5)
    m, n = 2048, 2048
    cb = e8_table_f16()
    cb2 = cb[:256].contiguous()
    q1 = _rand_idx(rng, m, n // 8)
    q2 = rng.integers(0, 256, size=(m, n // 8)).astype(np.int16)
    x = rng.standard_normal((2, n)).astype(np.float16)
    W = O.e8_dequant(q1, q2, 0.5)
    d1, d2, _, _ = e8_prepared(ext, cb, q1, q2, cb2=cb2)
    out = ext.glq_dequant_matmul_cuda(t(x), d1, cb, 1.0, d2, cb2, 0.5)
    assert rel(out, x.astype(np.float32) @ W.T) < 1e-3
    x = rng.standard_normal((24, n)).astype(np.float16)          # many tokens: tile kernel, second table from L2
    out = ext.glq_dequant_matmul_cuda(t(x), d1, cb, 1.0, d2, cb2, 0.5)
    assert rel(out, x.astype(np.float32) @ W.T) < 1e-3


@pytest.mark.parametrize("m,n,stages", [(100, 512, 1), (300, 768, 2), (128, 1024, 3), (200, 256, 4)])
def test_e8_many_token_tile_kernel_edges(ext, m, n, stages):
    """The kernel that keeps E8 layers compressed above 16 tokens: token counts on both sides of
    its 128 / 256 / 512-token tiles, row counts that end inside a 16-row fragment, 1-4 stages,
    against the oracle; rows of a larger call equal the rows of a smaller one up to the K split."""
    say("e8 tile edges", m, n, stages)
    rng = np.random.default_rng(m + stages)
    cb = e8_table_f16()
    q = [_rand_idx(rng, m, n // 8) for _ in range(4)]
    q[0][0, 0], q[0][0, 1], q[0][m - 1, n // 8 - 1] = 0, -1, -1
    sc = [0.0, 0.0, 0.0]
    for s in range(1, stages):
        sc[s - 1] = [1 / 3.0, 1 / 9.0, 1 / 27.0][s - 1]
    W = O.e8_dequant(q[0], q[1], sc[0], q[2], sc[1], q[3], sc[2])
    args = (t(q[0]), cb, 0.021, t(q[1]), cb, sc[0], None, t(q[2]), cb, sc[1], t(q[3]), cb, sc[2])
    xs = (rng.standard_normal((600, n)) * 0.5).astype(np.float16)
    ref = xs.astype(np.float32) @ W.T * np.float32(0.021)
    outs = {}
    for B in (17, 128, 129, 256, 257, 513, 600):
        out = ext.glq_dequant_matmul_cuda(t(xs[:B]), *args)
        assert out.shape == (B, m)
        # fp16 operands combined stage by stage: each stage adds one fp16 rounding of the weight
        assert rel(out, ref[:B]) < 1.5e-3, (B, rel(out, ref[:B]))
        assert torch.equal(out, ext.glq_dequant_matmul_cuda(t(xs[:B]), *args))
        outs[B] = out
    assert rel(outs[600][:129], outs[129].cpu().numpy()) < 1e-5
    assert rel(outs[257][:17], outs[17].cpu().numpy()) < 1e-5


def test_e8_small_secondary_table(ext):
    """3 bpw recipe: the second stage indexes the first 256 rows."""
    rng = np.random.default_rng(0)
    m, n = 64, 128
    cb = e8_table_f16()
    cb2 = cb[:256].contiguous()
    q1 = _rand_idx(rng, m, n // 8)
    q2 = rng.integers(0, 256, size=(m, n // 8)).astype(np.int16)
    x = rng.standard_normal((1, n)).astype(np.float16)
    W = O.e8_dequant(q1, q2, 0.5)
    out = ext.glq_dequant_matmul_cuda(t(x), t(q1), cb, 1.0, t(q2), cb2, 0.5)
    assert rel(out, x.astype(np.float32) @ W.T) < 1e-3


def test_e8_rejects_foreign_table(ext):
    bad = torch.randn(65536, 8, device=DEV).half()
    q = torch.zeros(32, 8, dtype=torch.int16, device=DEV)
    x = torch.zeros(1, 64, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="half-integer grid"):
        ext.glq_dequant_matmul_cuda(x, q, bad, 1.0)
    with pytest.raises(RuntimeError, match="65536 entries"):   # a first-stage table must be whole
        ext.glq_dequant_matmul_cuda(x, q, e8_table_f16()[:256].contiguous(), 1.0)


@pytest.mark.parametrize("tag,bpw,bd", [("bd2", 2, True), ("bd4", 4, True), ("p2", 2, False),
                                        ("p4", 4, False)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_e8_fused_linear_on_reference_layers(ext, golden, tag, bpw, bd, dtype):
    from glq_amd import hadamard as H
    g = golden("e8_layer")
    say("e8 fused golden", tag, dtype)
    m, n = g[f"{tag}_W"].shape
    bm, bn = list(g[f"{tag}_blocks_m"]), list(g[f"{tag}_blocks_n"])
    m_pad, n_pad = sum(bm), sum(bn)
    art = {"Qidxs": g[f"{tag}_Qidxs"], "SU": g[f"{tag}_SU"], "SV": g[f"{tag}_SV"],
           "Wscale": g[f"{tag}_Wscale"], "blocks_m": bm, "blocks_n": bn}
    q2, irs = None, 0.0
    if bpw == 4:
        art["Qidxs2"], art["inv_resid_scale"] = g[f"{tag}_Qidxs2"], g[f"{tag}_inv_resid_scale"]
        q2, irs = t(art["Qidxs2"]), float(art["inv_resid_scale"])
    x = torch.from_numpy(g[f"{tag}_x"]).to(dtype)
    ref = O.e8_linear_forward(x.float().numpy(), art, n, m)
    cb = e8_table_f16()
    common = (x.to(DEV), t(art["SV"]), t(art["SU"]), t(art["Qidxs"]), cb, float(art["Wscale"]), n, m,
              n_pad, m_pad)
    if bd:
        y = ext.glq_fused_linear_block_diag_cuda(
            *common, torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV),
            H.pack_block_meta(bm).to(DEV), q2, cb if q2 is not None else None, irs, out_dtype=dtype)
    else:
        y = ext.glq_fused_linear_cuda(*common, int(np.log2(n_pad)), int(np.log2(m_pad)), q2,
                                      cb if q2 is not None else None, irs, out_dtype=dtype)
    assert y.shape == (x.shape[0], m) and y.dtype == dtype
    assert rel(y, ref) < TOL, rel(y, ref)
    assert rel(y, g[f"{tag}_y"]) < TOL


@pytest.mark.parametrize("B", [1, 8])
def test_e8_config1_layer(ext, B):
    """960x960 at 2 bpw, weights N(0, 0.02) seed 0, quantised by RHT + nearest-E8,
    fp16 activations N(0,1), batch 1 and 8."""
    from glq_amd import hadamard as H
    say("e8 config1", B)
    torch.manual_seed(0)
    Wt = (torch.randn(960, 960) * 0.02).numpy()
    art, _ = O.e8_quantize_layer(Wt, bpw=2, seed=42)
    assert art["blocks_n"] == [512, 256, 128, 64]
    x = torch.randn(B, 960).to(torch.float16)
    ref = O.e8_linear_forward(x.float().numpy(), art, 960, 960)
    bn = bm = art["blocks_n"]
    y = ext.glq_fused_linear_block_diag_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(art["Qidxs"]), e8_table_f16(), float(art["Wscale"]),
        960, 960, 960, 960, torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV),
        H.pack_block_meta(bm).to(DEV))
    assert rel(y, ref) < TOL, rel(y, ref)
    # and against the unquantised layer: 2 bpw E8 keeps ~9 dB
    dense = x.float().numpy() @ Wt.T
    assert rel(y, dense) < 0.5


@pytest.mark.parametrize("xdt,odt", [(torch.bfloat16, torch.float16), (torch.float16, torch.float32),
                                     (torch.float32, torch.float16)])
def test_many_token_transforms_with_ragged_rows(ext, xdt, odt):
    """Whole-block 16-byte kernels (more than 64 tokens): rows that end inside an 8-element
    run on the input side, out_features that end inside one on the output side, fp32 /
    16-bit inputs and outputs, and equality with the few-token kernels row by row."""
    import ctypes as C
    from glq_amd import _lib, hadamard as H
    say("wide rht", xdt, odt)
    lib = _lib.load()
    B, n, inf, stride = 70, 2688, 2685, 2696                # blocks [2048, 512, 128]
    blocks = O.block_decompose(n)
    meta = H.pack_block_meta(blocks).to(DEV)
    xw = torch.randn(B, stride).to(xdt).to(DEV)
    rng = np.random.default_rng(7)
    sv = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    out = torch.empty(B, n, dtype=odt, device=DEV)
    arr = (C.c_int64 * len(blocks))(*blocks)
    dt = {torch.float16: _lib.GLQH_F16, torch.bfloat16: _lib.GLQH_BF16, torch.float32: _lib.GLQH_F32}
    svt = t(sv)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.glqh_input_rht(C.c_void_p(xw.data_ptr()), dt[xdt], stride, C.c_void_p(svt.data_ptr()),
                                  C.c_void_p(out.data_ptr()), dt[odt], B, inf, n, C.c_void_p(meta.data_ptr()),
                                  arr, len(blocks), 0.0, stream))
    xp = np.zeros((B, n), np.float32)
    xp[:, :inf] = xw[:, :inf].float().cpu().numpy()
    ref = O.block_diag_fht(xp * sv.astype(np.float32)[None], blocks)
    tol = 2e-5 if odt == torch.float32 else 2e-3
    assert np.allclose(out.float().cpu().numpy(), ref, rtol=tol, atol=tol)
    few = torch.empty(3, n, dtype=odt, device=DEV)
    _lib.check(lib.glqh_input_rht(C.c_void_p(xw.data_ptr()), dt[xdt], stride, C.c_void_p(svt.data_ptr()),
                                  C.c_void_p(few.data_ptr()), dt[odt], 3, inf, n, C.c_void_p(meta.data_ptr()),
                                  arr, len(blocks), 0.0, stream))
    assert torch.allclose(out[:3].float(), few.float(), rtol=tol, atol=tol)   # sliced vs whole 2048-point block
    # output side: out_features ends inside a run; y rows padded to a 16-byte multiple
    outf, ystride = 2683, 2688
    yr = torch.randn(B, n, device=DEV)
    su = np.where(rng.random(n) < 0.5, -1.0, 1.0).astype(np.float16)
    sut = t(su)
    y = torch.zeros(B, ystride, dtype=xdt, device=DEV)
    _lib.check(lib.glqh_output_rht(C.c_void_p(yr.data_ptr()), n, C.c_void_p(sut.data_ptr()), C.c_void_p(y.data_ptr()),
                                   dt[xdt], ystride, B, outf, n, C.c_void_p(meta.data_ptr()), arr, len(blocks),
                                   0.0, stream))
    ref = (O.block_diag_fht(yr.cpu().numpy(), blocks) * su.astype(np.float32)[None])[:, :outf]
    tol = 2e-5 if xdt == torch.float32 else 1e-2
    assert np.allclose(y[:, :outf].float().cpu().numpy(), ref, rtol=tol, atol=tol)
    assert torch.count_nonzero(y[:, outf:]) == 0
    y3 = torch.zeros(3, ystride, dtype=xdt, device=DEV)
    _lib.check(lib.glqh_output_rht(C.c_void_p(yr.data_ptr()), n, C.c_void_p(sut.data_ptr()), C.c_void_p(y3.data_ptr()),
                                   dt[xdt], ystride, 3, outf, n, C.c_void_p(meta.data_ptr()), arr, len(blocks),
                                   0.0, stream))
    # the few-token kernels cut the 2048-point block into two slices: other summation order
    assert torch.allclose(y[:3].float(), y3.float(), rtol=4e-3, atol=4e-3)
