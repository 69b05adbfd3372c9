"""Folded form of the E8 index streams (glqh_e8_fold_table / glqh_e8_fold_indices and the
small-batch kernel that reads it): the fold is checked against a numpy restatement of its
definition on the real table, and a product on the folded streams must give the same bits as the
product on the indices themselves wherever both run the same K plan (same K slots, same order of
summation, same decoded values) and agree to 1e-5 where the folded form sums K inside the
workgroup; against the oracle the usual bound holds (relative Frobenius error <= 1e-2)."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import DEV, e8_table_f16, rel, say, t
from oracle import glq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e


def _unfold(halves, fmap):
    """(n, 8) values from the half-codeword table and the map (first | second << 16)"""
    return np.concatenate([halves[fmap & 0xFFFF], halves[fmap >> 16]], axis=1).astype(np.float32)


def test_fold_of_the_shell_table(ext):
    say("e8 fold table")
    packed = ext._packed_table(e8_table_f16())
    halves, fmap = ext._fold_table(packed)
    hv, fm = halves.cpu().numpy(), fmap.cpu().numpy().view(np.uint32)
    table = O.e8_table()
    # the 65536 codewords are built from 1286 distinct halves (a property of the table itself: the
    # same count from the oracle's fp32 table)
    n_half = len(np.unique(np.concatenate([table[:, :4], table[:, 4:]]), axis=0))
    assert n_half == 1286 and hv.shape == (n_half, 4)
    assert ((fm & 0xFFFF) < n_half).all() and ((fm >> 16) < n_half).all()
    assert np.array_equal(_unfold(hv, fm), table)
    # numbered in order of first appearance, the first half of an entry before its second
    order = np.stack([fm & 0xFFFF, fm >> 16], axis=1).reshape(-1)
    _, first = np.unique(order, return_index=True)
    assert np.array_equal(order[np.sort(first)], np.arange(n_half))


def test_fold_of_an_index_stream_and_a_short_table(ext):
    say("e8 fold indices")
    small = e8_table_f16()[:256].contiguous()                 # the 3 bpw recipe's secondary table
    packed = ext._packed_table(small)
    rng = np.random.default_rng(0)
    q = rng.integers(0, 65536, size=(64, 40)).astype(np.uint16)          # indices past the table clamp to its last row
    qd = t(q.view(np.int16))
    lo16, hi8 = ext._fold_stream(qd, packed)
    hv, fm = ext._fold_table(packed)
    hv, fm = hv.cpu().numpy(), fm.cpu().numpy().view(np.uint32)
    assert np.array_equal(_unfold(hv, fm), O.e8_table()[:256])
    # tile order: 16 rows x 32 indices per tile, entry 8 * (16 g + i) + e = row i, index 8 g + e of the tile;
    # 40 columns are padded to 64 with half number 0
    want = np.zeros((64, 64), np.uint32)
    want[:, :40] = fm[np.minimum(q, 255)]
    tiles = want.reshape(4, 16, 2, 4, 8).transpose(0, 2, 3, 1, 4).reshape(-1)       # [row tile][col tile][g][i][e]
    first, second = tiles & 0xFFFF, tiles >> 16
    assert lo16.numel() == 4 * 2 * 512 == ext._lib.load().glqh_e8_folded_count(64, 40)
    assert np.array_equal(lo16.cpu().numpy().view(np.uint16), (first | (second & 31) << 11).astype(np.uint16))
    assert np.array_equal(hi8.cpu().numpy(), (second >> 5).astype(np.uint8))
    # the same tensors again come from the cache; a changed index tensor is folded again
    assert ext._fold_stream(qd, packed)[0] is lo16
    qd[0, 0] = 5
    lo2, _ = ext._fold_stream(qd, packed)
    assert lo2 is not lo16 and int(lo2.view(torch.int16)[0]) & 0x7FF == int(fm[5] & 0xFFFF)


def test_folded_copies_go_with_their_index_tensor(ext):
    say("e8 fold cache lifetime")
    import gc
    packed = ext._packed_table(e8_table_f16())
    qd = t(np.zeros((32, 64), np.int16))
    ext._fold_stream(qd, packed)
    ptr = qd.data_ptr()
    assert ext._FOLD_STREAMS.holds(qd)
    view = qd.view(64, 32)                                     # the storage lives on in a view
    del qd
    gc.collect()
    assert any(k[0] == ptr for k in ext._FOLD_STREAMS._d)
    del view
    gc.collect()
    assert not any(k[0] == ptr for k in ext._FOLD_STREAMS._d)


def _indices(m, n, stages, seed):
    rng = np.random.default_rng(seed)
    lo = rng.integers(0, 30000, size=(stages, m, n // 8))
    hi = rng.integers(0, 65536, size=(stages, m, n // 8))
    return np.where(rng.random((stages, m, n // 8)) < 0.6, lo, hi).astype(np.uint16).view(np.int16)


@pytest.mark.parametrize("m,n,B", [(4096, 2048, 1), (2048, 4096, 3), (1024, 8192, 16), (4096, 14336, 1)])
@pytest.mark.parametrize("stages", [1, 2, 3, 4])
def test_products_on_folded_streams_equal_products_on_indices(ext, m, n, B, stages):
    say("e8 folded matmul", m, n, B, stages)
    lib = ext._lib.load()
    assert lib.glqh_e8_fold_eligible(m, n, B) == 1
    q = [t(a) for a in _indices(m, n, stages, m + stages)]
    cb = e8_table_f16()
    cb2 = cb[:256].contiguous() if stages in (2, 3) else cb   # two, three stages: the short secondary table
    if stages in (2, 3):
        q[1] = t((_indices(m, n, 1, 7)[0].view(np.uint16) & 255).view(np.int16))
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).half().to(DEV)
    args = dict(qidxs2=q[1] if stages > 1 else None, codebook2=cb2, inv_resid_scale=1 / 3.0 if stages > 1 else 0.0,
                qidxs3=q[2] if stages > 2 else None, inv_resid_scale2=1 / 9.0 if stages > 2 else 0.0,
                qidxs4=q[3] if stages > 3 else None, inv_resid_scale3=1 / 27.0 if stages > 3 else 0.0)
    ext.E8_FOLD = True
    try:
        held = ext.e8_prepare(q[0], cb, args["qidxs2"], cb2, args["qidxs3"], args["qidxs4"])
        assert held == 3 * stages * lib.glqh_e8_folded_count(m, n // 8) and ext._FOLD_STREAMS.holds(q[0])
        y_fold = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)
        ext.E8_FOLD = False
        y_idx = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)
    finally:
        ext.E8_FOLD = True
    # same K slots and order of summation, same decoded values: the same bits -- except when
    # 16-row tiles fill the chip once: there the folded form keeps all of K inside a workgroup (sixteen K
    # parts summed in LDS, finished sums written by the kernel, no reduction launch), and at 5..16 tokens on rows
    # of up to 1536 blocks (four K parts per workgroup instead of none): another order
    props = torch.cuda.get_device_properties(0)
    if ((m + 15) // 16 <= props.multi_processor_count and 512 <= n // 8 <= (512 if B > 4 else 2048)) or \
            (B > 4 and n // 8 <= 1536):
        assert rel(y_fold, y_idx) < 1e-5
    else:
        assert torch.equal(y_fold, y_idx)
    if m * n <= 1 << 23:                                       # and both are the oracle's product
        tabs = [O.e8_table(), O.e8_table()[:256] if stages in (2, 3) else O.e8_table(), O.e8_table(), O.e8_table()]
        W = sum(tabs[s][q[s].cpu().numpy().view(np.uint16).astype(np.int64)].reshape(m, n) * (3.0 ** -s)
                for s in range(stages)).astype(np.float32) * np.float32(0.02)
        assert rel(y_fold, x.float().cpu().numpy() @ W.T) < TOL


@pytest.mark.parametrize("m,n,B", [(1000, 2048, 17), (2048, 1024, 40), (520, 4096, 64), (1024, 2048, 100), (4096, 1024, 130),
                                   (2048, 4096, 300), (1000, 1024, 300), (1536, 2560, 520)])
@pytest.mark.parametrize("stages", [1, 2, 3, 4])
def test_many_token_products_on_folded_streams_equal_products_on_indices(ext, m, n, B, stages):
    """Above 16 tokens the tile kernel reads the folded streams too: same tiles, same K slots, same fp16
    operands (half codewords out of LDS instead of expanded table words), hence the same bits."""
    say("e8 folded tile matmul", m, n, B, stages)
    lib = ext._lib.load()
    assert lib.glqh_e8_fold_eligible(m, n, B) == 1
    q = [t(a) for a in _indices(m, n, stages, m + stages + B)]
    cb = e8_table_f16()
    cb2 = cb[:256].contiguous() if stages in (2, 3) else cb   # two, three stages: the short secondary table
    if stages in (2, 3):
        q[1] = t((_indices(m, n, 1, 7)[0].view(np.uint16) & 255).view(np.int16))
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).half().to(DEV)
    args = dict(qidxs2=q[1] if stages > 1 else None, codebook2=cb2, inv_resid_scale=1 / 3.0 if stages > 1 else 0.0,
                qidxs3=q[2] if stages > 2 else None, inv_resid_scale2=1 / 9.0 if stages > 2 else 0.0,
                qidxs4=q[3] if stages > 3 else None, inv_resid_scale3=1 / 27.0 if stages > 3 else 0.0)
    ext.E8_FOLD = True
    try:
        held = ext.e8_prepare(q[0], cb, args["qidxs2"], cb2, args["qidxs3"], args["qidxs4"])
        assert held == 3 * stages * lib.glqh_e8_folded_count(m, n // 8) and ext._FOLD_STREAMS.holds(q[0])
        y_fold = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)
        ext.E8_FOLD = False
        y_idx = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)
    finally:
        ext.E8_FOLD = True
    assert torch.equal(y_fold, y_idx)
    if m * n <= 1 << 23:
        tabs = [O.e8_table(), O.e8_table()[:256] if stages in (2, 3) else O.e8_table(), O.e8_table(), O.e8_table()]
        W = sum(tabs[s][q[s].cpu().numpy().view(np.uint16).astype(np.int64)].reshape(m, n) * (3.0 ** -s)
                for s in range(stages)).astype(np.float32) * np.float32(0.02)
        assert rel(y_fold, x.float().cpu().numpy() @ W.T) < TOL


def test_fused_linear_on_folded_streams_and_under_capture(ext):
    """The forward path only looks the folded streams up.  A layer that was never prepared runs on its
    indices -- also under capture, with a warning -- and makes nothing; after `e8_prepare` a captured
    first call reads the folded streams and equals the eager folded result bit for bit."""
    say("e8 folded fused linear + graph")
    import warnings
    from glq_amd import hadamard as H
    m, n = 4096, 3072                                          # block-diagonal input side
    q = [t(a) for a in _indices(m, n, 2, 3)]
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    cb = e8_table_f16()
    ext._packed_table(cb)                                      # the table itself is known (another layer used it)
    args = (t(sv.astype(np.float16)), t(su.astype(np.float16)), q[0], cb, 0.02, n, m, n, m, torch.tensor(bn),
            torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), q[1], cb, 1 / 3.0)
    x = torch.randn(2, n, generator=torch.Generator().manual_seed(5)).bfloat16().to(DEV)
    n_before = len(ext._FOLD_STREAMS)
    with pytest.warns(RuntimeWarning, match="was not prepared"):
        y_idx = ext.glq_fused_linear_block_diag_cuda(x, *args, out_dtype=torch.bfloat16)
    q_new = [a.clone() for a in q]                             # first seen under capture
    g = torch.cuda.CUDAGraph()
    with pytest.warns(RuntimeWarning, match="under stream capture"):
        with torch.cuda.graph(g):
            y_cap = ext.glq_fused_linear_block_diag_cuda(x, *args[:2], q_new[0], *args[3:13], q_new[1], *args[14:],
                                                         out_dtype=torch.bfloat16)
    assert len(ext._FOLD_STREAMS) == n_before                  # nothing was made on the way
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(y_cap, y_idx)
    # load-time step, then a captured FIRST call: it runs the folded kernel
    bytes_before = ext.e8_fold_bytes()
    held = ext.e8_prepare(q[0], cb, q[1], cb)
    assert held == 2 * 3 * ext._lib.load().glqh_e8_folded_count(m, n // 8) == ext.e8_fold_bytes() - bytes_before
    g2 = torch.cuda.CUDAGraph()
    with warnings.catch_warnings():
        warnings.simplefilter("error")                         # no "not prepared" warning any more
        with torch.cuda.graph(g2):
            y2 = ext.glq_fused_linear_block_diag_cuda(x, *args, out_dtype=torch.bfloat16)
        y_fold = ext.glq_fused_linear_block_diag_cuda(x, *args, out_dtype=torch.bfloat16)
    for _ in range(2):
        g2.replay()
        torch.cuda.synchronize()
        assert torch.equal(y2, y_fold)
    assert torch.equal(y_fold, y_idx)                          # this shape keeps the K plan: the same bits as on the indices
    art = {"Qidxs": q[0].cpu().numpy(), "Qidxs2": q[1].cpu().numpy(), "inv_resid_scale": np.float32(1 / 3.0),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": bm, "blocks_n": bn}
    assert rel(y_fold, O.e8_linear_forward(x.float().cpu().numpy(), art, n, m)) < TOL


@pytest.mark.parametrize("m,n,B", [(1536, 1024, 300), (1536, 1024, 700), (1000, 2048, 520), (1004, 1024, 300), (1002, 1024, 300),
                                   (4096, 512, 1100)])
@pytest.mark.parametrize("stages", [1, 2, 4])
def test_fused_linear_at_many_tokens_on_folded_streams(ext, m, n, B, stages):
    """From 257 tokens on the folded form hands its sums to the output transform as fp16, times Wscale, when
    the rows of the sums and of y start on 16 bytes (m a multiple of 8), and as fp32 otherwise; both are the
    oracle's linear, also with activations large enough to take unscaled sums past the fp16 range."""
    say("e8 folded fused linear, many tokens", m, n, B, stages)
    from glq_amd import hadamard as H
    q = [t(a) for a in _indices(m, n, stages, 3 * m + stages + B)]
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    cb = e8_table_f16()
    inv = [1 / 3.0, 1 / 9.0, 1 / 27.0]
    extra = []
    for s in range(1, 4):
        extra += [q[s] if s < stages else None, cb if s < stages else None, inv[s - 1] if s < stages else 0.0]
    qs = q + [None] * (4 - stages)
    assert ext.e8_prepare(qs[0], cb, qs[1], cb, qs[2], qs[3]) > 0
    args = (t(sv.astype(np.float16)), t(su.astype(np.float16)), q[0], cb, 0.02, n, m, n, m, torch.tensor(bn),
            torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), *extra)
    W = sum(O.e8_table()[q[s].cpu().numpy().view(np.uint16).astype(np.int64)].reshape(m, n) * (3.0 ** -s)
            for s in range(stages)).astype(np.float32) * np.float32(0.02)
    for amp in (1.0, 600.0):
        x = (torch.randn(B, n, generator=torch.Generator().manual_seed(B)) * amp).bfloat16().to(DEV)
        y = ext.glq_fused_linear_block_diag_cuda(x, *args, out_dtype=torch.bfloat16)
        assert torch.isfinite(y).all()
        want = O.linear_forward_rht(x.float().cpu().numpy(), W, su.astype(np.float32), sv.astype(np.float32), bn, bm, n, m)
        assert rel(y, want) < TOL


def test_fresh_views_of_the_indices_hit_the_one_fold(ext):
    """A caller that passes a new view object of the same index memory on every call (a shard of a
    stacked tensor, `.view()`) finds the one folded copy: nothing is folded again, nothing dropped."""
    say("e8 fold: fresh views")
    m, n = 2048, 4096
    stacked = t(_indices(2 * m, n, 1, 12)[0])                  # two layers stacked row-wise
    cb = e8_table_f16()
    shard = lambda: stacked[m:]                                # noqa: E731  (a new tensor object per call)
    assert ext.e8_prepare(shard(), cb) > 0
    n_entries = len(ext._FOLD_STREAMS)
    x = torch.randn(1, n, generator=torch.Generator().manual_seed(1)).half().to(DEV)
    import warnings
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        y1 = ext.glq_dequant_matmul_cuda(x, shard(), cb, 0.02)
        y2 = ext.glq_dequant_matmul_cuda(x, stacked.view(2, m, n // 8)[1], cb, 0.02)
    assert len(ext._FOLD_STREAMS) == n_entries and torch.equal(y1, y2)
    ext.E8_FOLD = False
    try:
        assert rel(y1, ext.glq_dequant_matmul_cuda(x, shard(), cb, 0.02)) < 1e-5
    finally:
        ext.E8_FOLD = True
    assert ext.e8_prepare(shard(), cb) > 0 and len(ext._FOLD_STREAMS) == n_entries    # again: a lookup
    # the bound on the copies: a layer prepared beyond it stays on its indices
    other = t(_indices(m, n, 1, 13)[0])
    ext.E8_FOLD_MAX_BYTES = ext.e8_fold_bytes() + 1024
    try:
        assert ext.e8_prepare(other, cb) == 0 and not ext._FOLD_STREAMS.holds(other)
    finally:
        ext.E8_FOLD_MAX_BYTES = 0
    ext.e8_release(stacked[m:])
    assert not ext._FOLD_STREAMS.holds(stacked[m:])


@pytest.mark.parametrize("m,n,B", [(960, 960, 24), (1024, 2080, 70), (520, 4128, 300), (2048, 1056, 17)])
@pytest.mark.parametrize("stages", [1, 2, 4])
def test_many_token_products_on_widths_that_are_not_whole_tile_groups(ext, m, n, B, stages):
    """Rows of any multiple of 32 columns run the tile kernel on folded streams (the folded tiles end in the
    zero codeword, the blocked activations in zero columns); on the indices themselves such widths go to the
    dequantize + library route.  Against the oracle's product and against that route."""
    say("e8 folded tile matmul, ragged width", m, n, B, stages)
    lib = ext._lib.load()
    assert n % 256 != 0 and lib.glqh_e8_fold_eligible(m, n, B) == 1
    q = [t(a) for a in _indices(m, n, stages, m + n + stages)]
    cb = e8_table_f16()
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).half().to(DEV)
    args = dict(qidxs2=q[1] if stages > 1 else None, codebook2=cb, inv_resid_scale=1 / 3.0 if stages > 1 else 0.0,
                qidxs3=q[2] if stages > 2 else None, inv_resid_scale2=1 / 9.0 if stages > 2 else 0.0,
                qidxs4=q[3] if stages > 3 else None, inv_resid_scale3=1 / 27.0 if stages > 3 else 0.0)
    assert ext.e8_prepare(q[0], cb, args["qidxs2"], cb, args["qidxs3"], args["qidxs4"]) > 0
    y_fold = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)
    assert torch.equal(y_fold, ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args))
    ext.E8_FOLD = False
    try:
        y_lib = ext.glq_dequant_matmul_cuda(x, q[0], cb, 0.02, **args)      # dequantize + library GEMM
    finally:
        ext.E8_FOLD = True
    assert rel(y_fold, y_lib) < 2e-3
    W = sum(O.e8_table()[q[s].cpu().numpy().view(np.uint16).astype(np.int64)].reshape(m, n) * (3.0 ** -s)
            for s in range(stages)).astype(np.float32) * np.float32(0.02)
    assert rel(y_fold, x.float().cpu().numpy() @ W.T) < TOL
    # the fused linear (transform writes the blocked layout, zero columns appended) on the same layer
    from glq_amd import hadamard as H
    su, sv = O.rht_signs(m, n, 7)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    xb = torch.randn(B, n, generator=torch.Generator().manual_seed(1)).bfloat16().to(DEV)
    y = ext.glq_fused_linear_block_diag_cuda(
        xb, t(sv.astype(np.float16)), t(su.astype(np.float16)), q[0], cb, 0.02, n, m, n, m, torch.tensor(bn),
        torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), args["qidxs2"], cb,
        args["inv_resid_scale"], args["qidxs3"], cb, args["inv_resid_scale2"], args["qidxs4"], cb,
        args["inv_resid_scale3"], out_dtype=torch.bfloat16)
    ref = O.linear_forward_rht(xb.float().cpu().numpy(), W, su.astype(np.float32), sv.astype(np.float32), bn, bm, n, m)
    assert rel(y, ref) < TOL, rel(y, ref)


def test_c_abi_refusals(ext):
    say("e8 fold refusals")
    lib = ext._lib.load()
    packed = ext._packed_table(e8_table_f16())
    fmap = torch.empty(65536, dtype=torch.int32, device=DEV)
    n = C.c_int64(0)
    small = torch.empty((16, 4), dtype=torch.float16, device=DEV)
    rc = lib.glqh_e8_fold_table(packed.data_ptr(), 65536, small.data_ptr(), 16, fmap.data_ptr(), C.addressof(n), None)
    assert rc != 0 and b"room for 16" in lib.glqh_last_error() and n.value == 1286
    assert lib.glqh_e8_fold_eligible(960, 960, 1) == 0       # a small layer: the gather kernel serves it
    assert lib.glqh_e8_fold_eligible(4096, 14336, 17) == 1   # the tile kernel reads them too ...
    assert lib.glqh_e8_fold_eligible(4096, 14336 + 32, 17) == 1  # ... on rows of any multiple of 32 columns
    assert lib.glqh_e8_fold_eligible(4096, 14336 + 8, 17) == 0
