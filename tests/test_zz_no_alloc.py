"""The entry point that allocates nothing (glqh_fused_linear_trellis_3inst_noalloc) against the
entry point it is a variant of (glqh_fused_linear_trellis_3inst with a caller workspace), both
through the C ABI with raw ctypes: bit-identical outputs on two calls in a row, the second on a
smaller input, so that what the first call left in the shared scratch array is in the way."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from gpu_util import DEV, rel, say, t

pytestmark = pytest.mark.gpu


def _vp(x):
    return C.c_void_p(x.data_ptr()) if x is not None else C.c_void_p(0)


def _call(lib, noalloc, x, art, n, m, y):
    from glq_amd import _lib, hadamard as H
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    abn, abm = (C.c_int64 * len(bn))(*bn), (C.c_int64 * len(bm))(*bm)
    mn, mm = H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV)
    p1, p2 = art["p1"], art.get("p2")
    B = x.shape[0]
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = [_vp(x), _lib.GLQH_BF16, x.shape[1], B, _vp(art["sv"]), _vp(art["su"]),
            _vp(p1), p1.shape[0], p1.shape[1],
            _vp(p2), p2.shape[0] if p2 is not None else 0, p2.shape[1] if p2 is not None else 0,
            abn, len(bn), abm, len(bm), _vp(mn), _vp(mm),
            art["wscale"], art["inv_rs2"] if p2 is not None else 0.0, n, m, n, m,
            _vp(y), _lib.GLQH_BF16, m, C.c_void_p(0), 0]
    if noalloc:
        _lib.check(lib.glqh_fused_linear_trellis_3inst_noalloc(*head, stream))
    else:
        nb = lib.glqh_fused_linear_trellis_workspace_bytes(B, n, m)
        ws = torch.empty(nb, dtype=torch.uint8, device=DEV)
        _lib.check(lib.glqh_fused_linear_trellis_3inst(*head, _vp(ws), nb, stream))
    torch.cuda.synchronize()


def _layer(m, n, seed, two_stage):
    su, sv = O.rht_signs(m, n, 42 + seed)
    art = {"p1": t(O.random_packed(m, n, 4, seed)), "su": t(su.astype(np.float16)),
           "sv": t(sv.astype(np.float16)), "wscale": 0.017, "inv_rs2": 0.27}
    host = {"trellis_packed": art["p1"].cpu().numpy(), "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
            "Wscale": np.float32(0.017), "blocks_m": O.block_decompose(m), "blocks_n": O.block_decompose(n)}
    if two_stage:
        art["p2"] = t(O.random_packed(m, n, 2, seed + 100))
        host["trellis_packed2"] = art["p2"].cpu().numpy()
        host["inv_resid_scale2"] = np.float32(0.27)
    return art, host


def test_noalloc_entry_equals_workspace_entry_twice_in_a_row():
    from glq_amd import _lib
    lib = _lib.load()
    assert lib.glqh_noalloc_scratch_bytes() == 8 << 20
    # first call: a 2048 x 11008 two-stage layer at 3 tokens (block-diagonal both sides);
    # second call: a smaller single-stage layer at 1 token (fused-input route, other K plan)
    cases = [(2048, 11008, 3, True, 1), (512, 2048, 1, False, 2), (96, 192, 5, True, 3)]
    for m, n, B, two, seed in cases:
        say("noalloc", m, n, B, two)
        art, host = _layer(m, n, seed, two)
        x = torch.randn(B, n).to(torch.bfloat16).to(DEV)
        y_ws = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
        y_na = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
        _call(lib, False, x, art, n, m, y_ws)
        _call(lib, True, x, art, n, m, y_na)
        assert torch.equal(y_ws, y_na), (m, n, B)
        if m * n <= 1 << 21:                                   # the oracle's forward in seconds
            ref = O.trellis_linear_forward(x.float().cpu().numpy(), host, n, m)
            assert rel(y_na, ref) < 1e-2
    # repeat the first (large) case after the small ones: same bits again
    m, n, B, two, seed = cases[0]
    art, _ = _layer(m, n, seed, two)
    x = torch.randn(B, n).to(torch.bfloat16).to(DEV)
    y_ws = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
    y_na = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
    _call(lib, True, x, art, n, m, y_na)
    _call(lib, False, x, art, n, m, y_ws)
    assert torch.equal(y_ws, y_na)


def test_noalloc_entry_under_capture_allocates_nothing():
    """Captured after glqh_init() alone (no earlier call of the entry): replays on new activations
    equal the workspace entry bit for bit, and the device's free memory is the same before and
    after the calls (hipMemGetInfo through torch; the outputs are allocated beforehand)."""
    from glq_amd import _lib
    lib = _lib.load()
    assert lib.glqh_init() == 0
    m, n, B = 2048, 2048, 2
    art, _ = _layer(m, n, 21, True)
    xs = [torch.randn(B, n).to(torch.bfloat16).to(DEV) for _ in range(3)]
    static_x, y_na = xs[0].clone(), torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
    y_ws = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
    from glq_amd import hadamard as H
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    abn, abm = (C.c_int64 * len(bn))(*bn), (C.c_int64 * len(bm))(*bm)
    mn, mm = H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV)
    p1, p2 = art["p1"], art["p2"]

    def launch():
        _lib.check(lib.glqh_fused_linear_trellis_3inst_noalloc(
            _vp(static_x), _lib.GLQH_BF16, n, B, _vp(art["sv"]), _vp(art["su"]), _vp(p1), p1.shape[0], p1.shape[1],
            _vp(p2), p2.shape[0], p2.shape[1], abn, len(bn), abm, len(bm), _vp(mn), _vp(mm), art["wscale"],
            art["inv_rs2"], n, m, n, m, _vp(y_na), _lib.GLQH_BF16, m, C.c_void_p(0), 0,
            C.c_void_p(torch.cuda.current_stream().cuda_stream)))

    say("noalloc under capture")
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            launch()
    torch.cuda.current_stream().wait_stream(s)
    for x in xs[1:] + xs[:1]:
        _call(lib, False, x, art, n, m, y_ws)                  # eager work between the replays
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_na, y_ws)
    # an eager call between two readings of the device's free memory, nothing else in between
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    launch()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert torch.equal(y_na, y_ws)


def test_noalloc_entry_refuses_what_does_not_fit():
    from glq_amd import _lib
    lib = _lib.load()
    m, n, B = 14336, 4096, 64
    assert lib.glqh_fused_linear_trellis_workspace_bytes(B, n, m) > lib.glqh_noalloc_scratch_bytes()
    art, _ = _layer(64, 128, 9, False)                         # pointers are never touched: refused on sizes
    x = torch.zeros(B, n, dtype=torch.bfloat16, device=DEV)
    y = torch.zeros(B, m, dtype=torch.bfloat16, device=DEV)
    fake = dict(art)
    with pytest.raises(RuntimeError, match="bytes of scratch"):
        _call_sizes_only(lib, x, fake, n, m, y)


def _call_sizes_only(lib, x, art, n, m, y):
    """The refusal happens before any pointer is used; packed_rows is given as the layer's true
    count so that only the scratch size can be the reason."""
    from glq_amd import _lib, hadamard as H
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    abn, abm = (C.c_int64 * len(bn))(*bn), (C.c_int64 * len(bm))(*bm)
    mn, mm = H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.glqh_fused_linear_trellis_3inst_noalloc(
        _vp(x), _lib.GLQH_BF16, n, x.shape[0], _vp(art["sv"]), _vp(art["su"]), _vp(art["p1"]),
        (m // 16) * (n // 16), 64, C.c_void_p(0), 0, 0, abn, len(bn), abm, len(bm), _vp(mn), _vp(mm),
        0.017, 0.0, n, m, n, m, _vp(y), _lib.GLQH_BF16, m, C.c_void_p(0), 0, stream))
