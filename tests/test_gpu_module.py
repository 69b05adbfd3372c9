"""E8RHTLinear module, torch.ops.glq, dense many-token route and graph replay (MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.mark.parametrize("tag", ["k2", "k4", "k4k2"])
def test_trellis_module_loads_reference_checkpoint(golden, tag):
    from glq_amd.quantized_linear import E8RHTLinear
    g = golden("trellis_layer")
    say("module trellis", tag)
    m, n = g[f"{tag}_W"].shape
    keys = ["trellis_packed", "SU", "SV", "Wscale"] + (
        ["trellis_packed2", "inv_resid_scale2"] if tag == "k4k2" else [])
    sd = {k: torch.from_numpy(np.asarray(g[f"{tag}_{k}"])) for k in keys}
    layer = E8RHTLinear(n, m, codebook_type="trellis")
    layer.load_state_dict(sd)
    layer.to(DEV)
    x = torch.from_numpy(g[f"{tag}_x"])
    for dtype in (torch.float16, torch.bfloat16):
        y = layer(x.to(DEV, dtype))
        assert y.dtype == dtype and y.shape == (x.shape[0], m)
        assert rel(y, g[f"{tag}_y"]) < TOL
    y3 = layer(x.to(DEV, torch.bfloat16).reshape(1, 5, n))
    assert y3.shape == (1, 5, m)


@pytest.mark.parametrize("tag,bpw,bd", [("bd2", 2, True), ("bd4", 4, True), ("p2", 2, False),
                                        ("p4", 4, False)])
def test_shell_module_loads_reference_checkpoint(golden, tag, bpw, bd):
    from glq_amd.quantized_linear import E8RHTLinear
    g = golden("e8_layer")
    say("module shell", tag)
    m, n = g[f"{tag}_W"].shape
    keys = ["Qidxs", "SU", "SV", "Wscale"] + (["Qidxs2", "inv_resid_scale"] if bpw == 4 else [])
    sd = {k: torch.from_numpy(np.asarray(g[f"{tag}_{k}"])) for k in keys}
    layer = E8RHTLinear(n, m, block_diagonal=bd)
    layer.load_state_dict(sd)
    layer.to(DEV)
    cb = e8_table_f16()
    layer.set_codebook(cb, cb if bpw == 4 else None)
    x = torch.from_numpy(g[f"{tag}_x"]).to(DEV, torch.bfloat16)
    y = layer(x)
    assert y.dtype == torch.bfloat16 and y.shape == (3, m)
    assert rel(y, g[f"{tag}_y"]) < TOL
    assert torch.equal(y, layer(x))


@pytest.mark.parametrize("kind", ["trellis", "shell"])
def test_module_with_no_tokens_and_with_more_than_one_call_holds(golden, kind):
    """An empty batch gives an empty result (as the reference's torch path does), and a batch
    beyond what one launch grid indexes is served in pieces with the same rows as a short call."""
    from glq_amd.quantized_linear import E8RHTLinear
    say("module empty / long batch", kind)
    if kind == "trellis":
        g, tag = golden("trellis_layer"), "k4"
        keys = ["trellis_packed", "SU", "SV", "Wscale"]
        m, n = g[f"{tag}_W"].shape
        layer = E8RHTLinear(n, m, codebook_type="trellis")
    else:
        g, tag = golden("e8_layer"), "bd2"
        keys = ["Qidxs", "SU", "SV", "Wscale"]
        m, n = g[f"{tag}_W"].shape
        layer = E8RHTLinear(n, m, block_diagonal=True)
    layer.load_state_dict({k: torch.from_numpy(np.asarray(g[f"{tag}_{k}"])) for k in keys})
    layer.to(DEV)
    if kind == "shell":
        layer.set_codebook(e8_table_f16())
    y0 = layer(torch.empty(0, n, dtype=torch.bfloat16, device=DEV))
    assert y0.shape == (0, m) and y0.dtype == torch.bfloat16
    assert layer(torch.empty(2, 0, n, dtype=torch.float16, device=DEV)).shape == (2, 0, m)
    B = 32768 + 700
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(3)).to(DEV, torch.bfloat16)
    y = layer(x)
    assert y.shape == (B, m)
    for lo in (0, 32768 - 300, B - 600):                   # rows either side of the split
        assert rel(y[lo:lo + 600], layer(x[lo:lo + 600]).float()) < 5e-3
    assert rel(y[-3:], x[-3:].float().cpu().numpy() @ g[f"{tag}_W_hat"].T) < TOL


def test_ops_namespace_runs_the_hip_path():
    from glq_amd import custom_ops, hadamard as H
    custom_ops.register()
    m, n = 128, 256
    p = t(O.random_packed(m, n, 4, 3))
    su, sv = O.rht_signs(m, n, 7)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    x = torch.randn(2, n, device=DEV).half()
    from glq_amd import ext
    args = (x, t(sv.astype(np.float16)), t(su.astype(np.float16)), p, torch.tensor(bn), torch.tensor(bm),
            H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.02, n, m, n, m)
    assert torch.equal(torch.ops.glq.fused_linear_trellis_3inst(*args),
                       ext.glq_fused_linear_trellis_3inst_cuda(*args))


@pytest.mark.parametrize("route", ["mfma", "dense"])
@pytest.mark.parametrize("B", [17, 33, 64, 65, 200, 600])
def test_trellis_many_tokens(B, route, monkeypatch):
    """More than 16 tokens: the tile kernels over the compressed stream, and the
    dequantize-then-GEMM route the reference takes (GLQ_TRELLIS_BATCH_MAX; by default above
    8192 tokens)."""
    from glq_amd import ext, hadamard as H
    monkeypatch.setattr(ext, "TRELLIS_BATCH_MAX", 16 if route == "dense" else 1 << 30)
    m, n = 256, 512
    say("trellis many tokens", B, route)
    p1, p2 = O.random_packed(m, n, 4, 1), O.random_packed(m, n, 2, 2)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": p1, "trellis_packed2": p2, "inv_resid_scale2": np.float32(0.3),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(B, n).to(torch.bfloat16)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.02, 0.3, n, m, n, m,
        out_dtype=torch.bfloat16)
    assert y.shape == (B, m) and rel(y, ref) < TOL
    # rows agree with the compressed small-batch route
    y8 = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x[:8].to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.02, 0.3, n, m, n, m,
        out_dtype=torch.bfloat16)
    assert rel(y[:8], y8.float()) < 5e-3


@pytest.mark.parametrize("B", [17, 24, 32, 40])
def test_trellis_two_stage_tile_kernel_at_few_tokens(B):
    """From 17 tokens on the tile kernels run; they do not pre-scale the second
    stage's sums, so a two-stage layer with canonical output blocks must not be finished as plain K slots."""
    from glq_amd import ext, hadamard as H
    m, n = 256, 4096
    say("trellis two-stage tile route", B)
    p1, p2 = O.random_packed(m, n, 4, 1), O.random_packed(m, n, 2, 2)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": p1, "trellis_packed2": p2, "inv_resid_scale2": np.float32(0.3),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).to(torch.bfloat16)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.02, 0.3, n, m, n, m,
        out_dtype=torch.bfloat16)
    assert y.shape == (B, m) and rel(y, ref) < TOL
    # single stage through the same route
    art1 = {k: v for k, v in art.items() if k not in ("trellis_packed2", "inv_resid_scale2")}
    ref1 = O.trellis_linear_forward(x.float().numpy(), art1, n, m)
    y1 = ext.glq_fused_linear_trellis_3inst_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.02, n, m, n, m, out_dtype=torch.bfloat16)
    assert rel(y1, ref1) < TOL


@pytest.mark.parametrize("m,n", [(256, 512), (2048, 2048), (2080, 1152)])
@pytest.mark.parametrize("K2", [1, 2, 3, 4])
@pytest.mark.parametrize("B", [1, 3, 6])
def test_trellis_two_stage_few_tokens(m, n, K2, B):
    """Two-stage layers at a few tokens: up to four tokens both stages fold the input transform
    into their launch (small and large layers take the two decode forms; a 1-bit second stage
    and more tokens take the separate transform).  Against the oracle, against the stages
    computed one at a time, and through the y_rht entry."""
    from glq_amd import ext, hadamard as H
    say("trellis two stages", m, n, K2, B)
    p1, p2 = O.random_packed(m, n, 4, 1), O.random_packed(m, n, K2, 2)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": p1, "trellis_packed2": p2, "inv_resid_scale2": np.float32(0.3),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).to(torch.bfloat16)
    args = (torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV))
    y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), *args, 0.02, 0.3, n, m, n, m,
        out_dtype=torch.bfloat16)
    if m * n <= 1 << 20:
        ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
        assert y.shape == (B, m) and rel(y, ref) < TOL, rel(y, ref)
    assert torch.equal(y, ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), *args, 0.02, 0.3, n, m, n, m,
        out_dtype=torch.bfloat16))
    # the same sum from single-stage calls (fp32 out): y1 + 0.3 * y2, linear in the weights
    y1 = ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), *args, 0.02,
                                                 n, m, n, m, out_dtype=torch.bfloat16).float()
    yr = torch.zeros(B, m, dtype=torch.float32, device=DEV)
    ext.glq_fused_linear_trellis_3inst_yrht_rvq2_cuda(x.to(DEV), t(art["SV"]), t(p1), t(p2), args[0], args[2],
                                                      0.02, 0.3, n, n, m, yr, 0)
    yo = torch.empty(B, m, dtype=torch.bfloat16, device=DEV)
    ext.glq_output_rht_blockdiag_cuda(yr, t(art["SU"]), yo, m, m, args[1], args[3])
    assert rel(yo, y.float()) < 5e-3, rel(yo, y.float())
    if K2 >= 2:
        y2 = ext.glq_fused_linear_trellis_3inst_cuda(x.to(DEV), t(art["SV"]), t(art["SU"]), t(p2), *args, 0.02 * 0.3,
                                                     n, m, n, m, out_dtype=torch.bfloat16).float()
        assert rel(y1 + y2, y.float()) < 1e-2, rel(y1 + y2, y.float())


@pytest.mark.parametrize("K1,K2", [(2, 2), (3, 1), (3, 3), (2, 4)])
@pytest.mark.parametrize("B", [1, 2, 4])
def test_trellis_two_stage_other_rates(K1, K2, B):
    """First stages of 2 and 3 bits per weight through the same routes (one layer large enough
    for the MFMA form of the folded transform), against the oracle."""
    from glq_amd import ext, hadamard as H
    m, n = 2048, 512
    say("trellis two stages, rates", K1, K2, B)
    p1, p2 = O.random_packed(m, n, K1, 5), O.random_packed(m, n, K2, 6)
    su, sv = O.rht_signs(m, n, 7)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"trellis_packed": p1, "trellis_packed2": p2, "inv_resid_scale2": np.float32(0.25),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.03),
           "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(K1 * 10 + K2)).to(torch.bfloat16)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    y = ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(p1), t(p2), torch.tensor(bn), torch.tensor(bm),
        H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), 0.03, 0.25, n, m, n, m,
        out_dtype=torch.bfloat16)
    assert y.shape == (B, m) and rel(y, ref) < TOL, rel(y, ref)


def test_e8_dense_route_many_tokens():
    from glq_amd import ext, hadamard as H
    m, n, B = 96, 160, 40
    rng = np.random.default_rng(0)
    q1 = rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16)
    q2 = rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16)
    su, sv = O.rht_signs(m, n, 42)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    art = {"Qidxs": q1, "Qidxs2": q2, "inv_resid_scale": np.float32(1 / 3.0), "SU": su.astype(np.float16),
           "SV": sv.astype(np.float16), "Wscale": np.float32(0.02), "blocks_m": bm, "blocks_n": bn}
    x = torch.randn(B, n).to(torch.float16)
    ref = O.e8_linear_forward(x.float().numpy(), art, n, m)
    cb = e8_table_f16()
    y = ext.glq_fused_linear_block_diag_cuda(
        x.to(DEV), t(art["SV"]), t(art["SU"]), t(q1), cb, 0.02, n, m, n, m, torch.tensor(bn),
        torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV), t(q2), cb, 1 / 3.0)
    assert rel(y, ref) < TOL
    xr = torch.randn(B, n, device=DEV).half()
    W = O.e8_dequant(q1, q2, 1 / 3.0)
    out = ext.glq_dequant_matmul_cuda(xr, t(q1), cb, 0.5, t(q2), cb, 1 / 3.0)
    assert rel(out, xr.float().cpu().numpy() @ W.T * 0.5) < 2e-3


def test_graph_capture_and_replay_is_bit_exact():
    """A decode step is replayed from a HIP graph: every replay, with eager work and
    synchronisation in between, must equal the eager result bit for bit."""
    from glq_amd.quantized_linear import E8RHTLinear
    m, n = 512, 2048
    layer = E8RHTLinear(n, m, codebook_type="trellis")
    su, sv = O.rht_signs(m, n, 1)
    layer.load_state_dict({"trellis_packed": torch.from_numpy(O.random_packed(m, n, 4, 9)),
                           "SU": torch.from_numpy(su).half(), "SV": torch.from_numpy(sv).half(),
                           "Wscale": torch.tensor(0.02)})
    layer.to(DEV)
    xs = torch.randn(1, n, device=DEV).to(torch.bfloat16)
    eager = layer(xs).clone()
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            y = layer(xs)
    torch.cuda.synchronize()
    for i in range(4):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {i}"
        other = layer(torch.randn(1, n, device=DEV).to(torch.bfloat16))      # eager work in between
        torch.cuda.synchronize()
        assert other.shape == (1, m)
    xs.copy_(torch.randn(1, n, device=DEV).to(torch.bfloat16))               # new input, same graph
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, layer(xs))


@pytest.mark.parametrize("B", [24, 48, 200])
def test_graph_capture_of_a_batched_step_on_the_tile_kernels(B):
    """17 tokens and more run the tile kernels (small-tile kernels up to 64 tokens, E8 on its folded streams):
    captured after a warm-up call, every replay equals the eager result bit for bit."""
    from glq_amd import ext, hadamard as H
    m, n = 512, 2048
    p = t(O.random_packed(m, n, 4, 11))
    su, sv = O.rht_signs(m, n, 3)
    bn, bm = O.block_decompose(n), O.block_decompose(m)
    meta = (torch.tensor(bn), torch.tensor(bm), H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV))
    svt, sut = t(sv.astype(np.float16)), t(su.astype(np.float16))
    rng = np.random.default_rng(B)
    q1, q2 = (t(rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16)) for _ in range(2))
    cb = e8_table_f16()
    assert ext.e8_prepare(q1, cb, q2, cb) > 0                  # the load-time step: folded streams exist before capture
    xs = torch.randn(B, n, device=DEV).to(torch.bfloat16)

    def step():
        return (ext.glq_fused_linear_trellis_3inst_cuda(xs, svt, sut, p, *meta, 0.02, n, m, n, m, out_dtype=torch.bfloat16),
                ext.glq_fused_linear_block_diag_cuda(xs, svt, sut, q1, cb, 0.02, n, m, n, m, *meta, q2, cb, 1 / 3.0,
                                                     out_dtype=torch.bfloat16))
    eager = [y.clone() for y in step()]
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            ys = step()
    torch.cuda.synchronize()
    for i in range(3):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ys[0], eager[0]) and torch.equal(ys[1], eager[1]), f"replay {i}"
        step()                                                # eager work in between
        torch.cuda.synchronize()
    xs.copy_(torch.randn(B, n, device=DEV).to(torch.bfloat16))  # new input, same graph
    g.replay()
    torch.cuda.synchronize()
    again = step()
    assert torch.equal(ys[0], again[0]) and torch.equal(ys[1], again[1])


def _two_stage_module(m, n, seed):
    from glq_amd.quantized_linear import E8RHTLinear
    p1, p2 = O.random_packed(m, n, 4, seed), O.random_packed(m, n, 2, seed + 1)
    su, sv = O.rht_signs(m, n, 42)
    art = {"trellis_packed": p1, "trellis_packed2": p2, "inv_resid_scale2": np.float32(0.3),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16), "Wscale": np.float32(0.02),
           "blocks_m": O.block_decompose(m), "blocks_n": O.block_decompose(n)}
    lin = E8RHTLinear(n, m, codebook_type="trellis")
    lin.load_state_dict({"trellis_packed": torch.from_numpy(p1), "trellis_packed2": torch.from_numpy(p2),
                         "SU": torch.from_numpy(art["SU"]), "SV": torch.from_numpy(art["SV"]),
                         "Wscale": torch.tensor(0.02), "inv_resid_scale2": torch.tensor(0.3)}, strict=False)
    return lin.to(DEV), art


@pytest.mark.parametrize("B", [1, 5, 70])
def test_reference_switches_fused_trellis_and_trellis_dense(B, monkeypatch):
    """GLQ_FUSED_TRELLIS=0 (three separate ops) and GLQ_TRELLIS_DENSE (dequantize + library GEMM),
    the reference's A/B switches (glq/quantized_linear.py:23-30, glq/csrc/glq_trellis.cu:1023-1029):
    both against the oracle, tolerance 1e-2 relative Frobenius."""
    from glq_amd import ext, quantized_linear as QL
    m, n = 512, 1024
    say("trellis switches", B)
    lin, art = _two_stage_module(m, n, 11)
    x = torch.randn(B, n).to(torch.bfloat16)
    ref = O.trellis_linear_forward(x.float().numpy(), art, n, m)
    y0 = lin(x.to(DEV))
    assert rel(y0, ref) < TOL
    monkeypatch.setattr(QL, "_GLQ_FUSED_TRELLIS_ENABLED", False)
    y1 = lin(x.to(DEV))
    assert y1.shape == y0.shape and y1.dtype == y0.dtype and rel(y1, ref) < TOL
    monkeypatch.setattr(QL, "_GLQ_FUSED_TRELLIS_ENABLED", True)
    monkeypatch.setattr(ext, "TRELLIS_DENSE", True)
    y2 = lin(x.to(DEV))
    assert rel(y2, ref) < TOL


def test_reference_switch_fuse_input_off_in_a_fresh_process(tmp_path):
    """GLQ_TRELLIS_FUSE_INPUT=0 (glq/csrc/glq_trellis.cu:1270-1274) is read once by the library, so
    the run with it set is a process of its own: same layer, same input, one token and three,
    single call and grouped call; its outputs agree with this process's within 1e-2."""
    import os
    import subprocess
    import sys
    from glq_amd import ext, hadamard as H
    m, n = 2048, 2048
    say("fuse-input switch, child process")
    script = r'''
import sys, numpy as np, torch
sys.path.insert(0, %r)
from oracle import glq_oracle as O
from glq_amd import ext, hadamard as H
m, n = 2048, 2048
dev = "cuda"
p = torch.from_numpy(O.random_packed(m, n, 4, 3)).to(dev)
su, sv = O.rht_signs(m, n, 42)
su, sv = torch.from_numpy(su.astype(np.float16)).to(dev), torch.from_numpy(sv.astype(np.float16)).to(dev)
bn = O.block_decompose(n)
outs = {}
for B in (1, 3):
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).to(torch.bfloat16).to(dev)
    outs["single%%d" %% B] = ext.glq_fused_linear_trellis_3inst_cuda(
        x, sv, su, p, torch.tensor(bn), torch.tensor(bn), H.pack_block_meta(bn).to(dev),
        H.pack_block_meta(bn).to(dev), 0.02, n, m, n, m, out_dtype=torch.float32).cpu().numpy()
    outs["group%%d" %% B] = ext.glq_fused_linear_trellis_3inst_group(
        x, [(sv, su, p, 0.02, m, m)] * 2, torch.tensor(bn), H.pack_block_meta(bn).to(dev), n, n,
        out_dtype=torch.float32)[:, m:].cpu().numpy()
np.savez(sys.argv[1], **outs)
''' % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    files = {}
    for tag, env in (("on", {}), ("off", {"GLQ_TRELLIS_FUSE_INPUT": "0"})):
        files[tag] = str(tmp_path / f"{tag}.npz")
        r = subprocess.run([sys.executable, "-c", script, files[tag]], env={**os.environ, **env},
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
    a, b = np.load(files["on"]), np.load(files["off"])
    for k in a.files:
        assert np.isfinite(b[k]).all() and rel(a[k], b[k]) < TOL, k
    # and both are the oracle's result
    x = torch.randn(1, n, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    su, sv = O.rht_signs(m, n, 42)
    W = O.decode_layer(O.random_packed(m, n, 4, 3), m, n, fast=True) * np.float32(0.02)
    bn = O.block_decompose(n)
    ref = O.linear_forward_rht(x.float().numpy(), W, su.astype(np.float32), sv.astype(np.float32), bn, bn, n, m)
    assert rel(b["single1"], ref) < TOL and rel(a["single1"], ref) < TOL
