"""The serving-side call sequence of a merged trellis linear (glq_vllm/linear_method.py:643-741)
through the registered `torch.ops.glq.*` ops: every shard against the oracle, the shard-batched
output transform against the per-shard route, and the whole sequence captured in a HIP graph and
replayed on new activations (needs an MI355X)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, rel, say, t

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module", autouse=True)
def ops():
    from glq_amd import custom_ops
    custom_ops.register()
    return torch.ops.glq


def _shard_art(m, n, K, K2, seed):
    su, sv = O.rht_signs(m, n, 200 + seed)
    art = {"trellis_packed": O.random_packed(m, n, K, seed), "SU": su.astype(np.float16),
           "SV": sv.astype(np.float16), "Wscale": np.float32(0.02 + 0.003 * seed),
           "blocks_m": O.block_decompose(m), "blocks_n": O.block_decompose(n)}
    if K2:
        art["trellis_packed2"] = O.random_packed(m, n, K2, 50 + seed)
        art["inv_resid_scale2"] = np.float32(0.21 + 0.01 * seed)
    return art


def _merged(n, shards, bpw):
    """shards: [(m, K, K2)] -> (MergedTrellisLinear after its load-time step, per-shard artifacts)."""
    from glq_amd.linear_method import GLQShards, MergedTrellisLinear
    arts = [_shard_art(m, n, K, K2, i) for i, (m, K, K2) in enumerate(shards)]
    layer = MergedTrellisLinear(n, [m for m, _, _ in shards], bpw=bpw)
    layer.trellis_packed = GLQShards(torch.from_numpy(a["trellis_packed"]) for a in arts)
    layer.trellis_packed2 = GLQShards(torch.from_numpy(a["trellis_packed2"]) if "trellis_packed2" in a
                                      else torch.zeros(0, dtype=torch.int16) for a in arts)
    layer.SU = GLQShards(torch.from_numpy(a["SU"]) for a in arts)
    layer.SV = GLQShards(torch.from_numpy(a["SV"]) for a in arts)
    layer.Wscale = GLQShards(torch.tensor(float(a["Wscale"])) for a in arts)
    layer.inv_resid_scale2 = GLQShards(torch.tensor(float(a.get("inv_resid_scale2", 0.0))) for a in arts)
    layer.process_weights_after_loading(DEV)
    return layer, arts


def _oracle(x16, arts, n):
    xs = x16.float().cpu().numpy()
    return np.concatenate([O.trellis_linear_forward(xs, a, n, a["SU"].shape[0]) for a in arts], axis=1)


@pytest.mark.parametrize("bpw,shards", [(4, [(256, 4, 0), (64, 4, 0), (64, 4, 0)]),       # fused q/k/v
                                        (6, [(352, 4, 2), (352, 4, 2)]),                  # gate/up, 4+2 bits
                                        (5, [(2048, 4, 1), (512, 4, 1), (512, 4, 1)])])   # SmolLM3 q/k/v rows, 4+1
@pytest.mark.parametrize("B", [1, 3, 40])
def test_s4b_sequence_through_registered_ops_matches_oracle(ops, bpw, shards, B, monkeypatch):
    """`fused_linear_trellis_3inst_yrht[_rvq2]` per shard into one (B, total_m) buffer + one
    `output_rht_shards`, each called as `torch.ops.glq.<op>`: every shard's columns within 1e-2 of
    the oracle's fp32 CPU forward of that shard; equal to the per-shard fused op's result up to the
    fp16 rounding of its output; bit-identical when repeated."""
    n = 512 if shards[0][0] < 2048 else 2048
    say("s4b ops", bpw, shards, B)
    layer, arts = _merged(n, shards, bpw)
    assert layer._glq_s4b is not None and layer._glq_s4b["has_s2"] == (bpw > 4)
    x = torch.randn(B, n, generator=torch.Generator().manual_seed(B)).to(DEV, torch.float16)
    ref = _oracle(x, arts, n)
    # the sequence written out with the registered ops, as the reference's apply does
    total = sum(m for m, _, _ in shards)
    y_rht = torch.empty(B, total, dtype=torch.float32, device=DEV)
    col = 0
    for i, meta in enumerate(layer._glq_trellis_meta):
        if meta["has_s2"]:
            ops.fused_linear_trellis_3inst_yrht_rvq2(
                x, layer.SV.get_shard(i), layer.trellis_packed.get_shard(i), layer.trellis_packed2.get_shard(i),
                meta["_bn"], meta["_bnm"], meta["wscale"], meta["inv_rs2"], n, n, meta["m_pad"], y_rht, col)
        else:
            ops.fused_linear_trellis_3inst_yrht(
                x, layer.SV.get_shard(i), layer.trellis_packed.get_shard(i), meta["_bn"], meta["_bnm"],
                meta["wscale"], n, n, meta["m_pad"], y_rht, col)
        col += meta["m_pad"]
    y = torch.empty(B, total, dtype=torch.float16, device=DEV)
    ops.output_rht_shards(y_rht, layer._glq_s4b["su_cat"], y, total, layer._glq_s4b["shard_meta"],
                          layer._glq_s4b["max_bs"])
    col = 0
    for (m, _, _), a in zip(shards, arts):
        e = rel(y[:, col:col + m], ref[:, col:col + m])
        assert e < TOL, (m, e)
        col += m
    # the layer object's apply() is that sequence (with GLQ_MERGED_GROUPED=0 at every token count)
    from glq_amd import linear_method as LM
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", False)
    ya = layer.apply(x)
    assert ya.dtype == x.dtype and torch.equal(ya, y)
    assert torch.equal(layer.apply(x), ya)
    # and the transform-domain rows of a shard are what the oracle's transform-domain product gives
    a0 = arts[0]
    m0 = shards[0][0]
    Wn = O.decode_layer_nstage([a0["trellis_packed"]] + ([a0["trellis_packed2"]] if "trellis_packed2" in a0 else []),
                               [1.0] + ([float(a0["inv_resid_scale2"])] if "trellis_packed2" in a0 else []), m0, n)
    xr = O.block_diag_fht(x.float().cpu().numpy() * a0["SV"].astype(np.float32)[None], a0["blocks_n"])
    assert rel(y_rht[:, :m0], (xr @ Wn.T) * np.float32(a0["Wscale"])) < TOL


def test_batched_output_transform_switch_and_unloaded_shard(ops, monkeypatch):
    """GLQ_TRELLIS_BATCH_OUT_RHT=0: one fused op per shard, concatenated -- against the oracle and
    against the shard-batched route (same decode, another launch for the output transform: equal to
    fp16 rounding).  A shard that was never loaded gives exact-zero columns on both routes."""
    from glq_amd import linear_method as LM
    say("s4b switch")
    n, shards = 512, [(256, 4, 0), (64, 4, 0), (64, 4, 0)]
    layer, arts = _merged(n, shards, 4)
    x = torch.randn(4, n, generator=torch.Generator().manual_seed(3)).to(DEV, torch.bfloat16)
    ref = _oracle(x, arts, n)
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", False)      # the reference's sequence, not the grouped call
    y_batched = layer.apply(x)
    monkeypatch.setattr(LM, "_GLQ_BATCH_OUT_RHT", False)
    y_per_shard = layer.apply(x)
    assert y_per_shard.dtype == torch.bfloat16
    assert rel(y_per_shard, ref) < TOL and rel(y_batched, ref) < TOL
    assert rel(y_per_shard, y_batched.float().cpu().numpy()) < 4e-3
    # an unloaded k shard (KV-shared layers): zeros, the other columns unchanged
    layer.trellis_packed._shard_data[1] = torch.zeros(0, dtype=torch.int16, device=DEV)
    layer.process_weights_after_loading(DEV)
    for flag in (True, False):
        monkeypatch.setattr(LM, "_GLQ_BATCH_OUT_RHT", flag)
        y0 = layer.apply(x)
        assert float(y0[:, 256:320].abs().max()) == 0.0
        want = y_batched if flag else y_per_shard
        assert torch.equal(y0[:, :256], want[:, :256]) and torch.equal(y0[:, 320:], want[:, 320:])


def test_load_time_invariants(ops):
    """What the checkpoint carries must match the recipe (glq_vllm/linear_method.py:1372-1396)."""
    from glq_amd.linear_method import MergedTrellisLinear, trellis_rvq_recipe
    say("s4b invariants")
    assert [trellis_rvq_recipe(b) for b in (2, 4, 5, 6, 8)] == [[2], [4], [4, 1], [4, 2], [4, 4]]
    with pytest.raises(ValueError):
        trellis_rvq_recipe(9)
    n, shards = 512, [(64, 4, 2), (64, 4, 2)]
    layer, _ = _merged(n, shards, 6)
    layer.glq_bpw = 4
    with pytest.raises(RuntimeError, match="no stage for"):
        layer.process_weights_after_loading(DEV)
    layer.glq_bpw = 6
    layer.inv_resid_scale2._shard_data[1] = torch.tensor(0.0)
    with pytest.raises(RuntimeError, match="half-written"):
        layer.process_weights_after_loading(DEV)
    layer.trellis_packed2._shard_data[1] = torch.zeros(0, dtype=torch.int16)
    with pytest.raises(RuntimeError, match="trellis_packed2 is missing"):
        layer.process_weights_after_loading(DEV)
    fresh = MergedTrellisLinear(n, [64])
    with pytest.raises(RuntimeError, match="process_weights_after_loading"):
        fresh.apply(torch.zeros(1, n, device=DEV, dtype=torch.float16))


@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("bpw,shards", [(4, [(2048, 4, 0), (512, 4, 0), (512, 4, 0)]), (6, [(352, 4, 2), (352, 4, 2)])])
def test_s4b_sequence_captured_in_a_graph_replays_on_new_activations(ops, bpw, shards, grouped, monkeypatch):
    """The whole apply() -- yrht ops, the shared buffer, output_rht_shards, the cast; or the library's grouped
    call, the default at this token count -- captured once; replays with new contents in the static input equal
    the eager result bit for bit, replay after replay, with eager work in between."""
    from glq_amd import linear_method as LM
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", grouped)
    n = 2048 if shards[0][0] == 2048 else 512
    say("s4b graph", bpw, grouped)
    layer, arts = _merged(n, shards, bpw)
    gen = torch.Generator().manual_seed(11)
    xs = [torch.randn(2, n, generator=gen).to(DEV, torch.bfloat16) for _ in range(4)]
    static_x = xs[0].clone()
    layer.apply(static_x)                                    # warm-up outside capture
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            static_y = layer.apply(static_x)
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    for x in xs[1:] + xs[:1]:
        eager = layer.apply(x)
        torch.cuda.synchronize()
        static_x.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_y, eager)
        assert rel(static_y, _oracle(x, arts, n)) < TOL


@pytest.mark.parametrize("B", [2, 7, 16, 30, 64, 100])
def test_merged_linear_through_the_grouped_call(ops, monkeypatch, B):
    """Single-stage merged shards through the library's grouped call, the default (one decode launch at
    1-4 tokens, one per shard at 5-64, one launch of the many-token kernel above 64) against the oracle and against
    the reference's sequence of registered ops; two-stage shards take their own grouped call or that sequence."""
    from glq_amd import linear_method as LM
    say("merged linear, grouped call", B)
    n = 512
    layer, arts = _merged(n, [(256, 4, 0), (64, 4, 0), (64, 4, 0)], 4)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(B)) * 0.5).to(torch.bfloat16).to(DEV)
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", False)
    y_ref = layer.apply(x)
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", True)
    assert layer._grouped_ok(B)
    y = layer.apply(x)
    assert y.dtype == x.dtype and y.shape == y_ref.shape
    assert rel(y, _oracle(x, arts, n)) < TOL
    assert rel(y, y_ref.float().cpu().numpy()) < 6e-3
    two, _ = _merged(n, [(352, 4, 2), (352, 4, 2)], 6)
    assert not two._grouped_ok(B)


@pytest.mark.parametrize("n,shards,bpw", [(512, [(352, 4, 2), (352, 4, 2)], 6), (2048, [(2048, 4, 1), (512, 4, 1), (512, 4, 1)], 5),
                                          (576, [(1184, 4, 4), (1184, 4, 4)], 8)])
@pytest.mark.parametrize("B", [1, 2, 9, 16, 17, 40, 64])
def test_merged_two_stage_linear_through_the_grouped_call(ops, monkeypatch, n, shards, bpw, B):
    """One token of merged stacked shards (5, 6, 8 bpw = 4 + 1, 2, 4) through the library's grouped
    two-stage call (one token: one decode launch for both streams of every shard; 2-64: one per shard; one
    finishing launch) against the oracle and against the reference's sequence of registered ops; more tokens keep
    that sequence."""
    from glq_amd import linear_method as LM
    say("merged two-stage linear, grouped call", n, bpw, B)
    layer, arts = _merged(n, shards, bpw)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(n + B)) * 0.5).to(torch.bfloat16).to(DEV)
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", False)
    y_ref = layer.apply(x)
    monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", True)
    assert layer._grouped_rvq2_ok(B) and not layer._grouped_rvq2_ok(65) and not layer._grouped_ok(B)
    y = layer.apply(x)
    assert y.dtype == x.dtype and y.shape == y_ref.shape
    assert rel(y, _oracle(x, arts, n)) < TOL
    assert rel(y, y_ref.float().cpu().numpy()) < 6e-3
    assert torch.equal(y, layer.apply(x))
    mixed, _ = _merged(512, [(352, 4, 2), (352, 4, 1)], 6)
    assert not mixed._grouped_rvq2_ok(B)


@pytest.mark.parametrize("B", [65, 200])
def test_merged_stacked_shards_at_many_tokens_run_as_whole_linears(ops, monkeypatch, B):
    """Above 64 tokens, shards the grouped call does not take (here 4+2-bit gate/up and a mixed pair) run as
    whole fused linears, concatenated: against the oracle and against the reference's shard-batched sequence."""
    from glq_amd import linear_method as LM
    say("merged stacked shards, many tokens", B)
    for n, shards, bpw in ((512, [(352, 4, 2), (352, 4, 2)], 6), (512, [(256, 4, 2), (96, 4, 1)], 6)):
        layer, arts = _merged(n, shards, bpw)
        x = (torch.randn(B, n, generator=torch.Generator().manual_seed(B)) * 0.5).to(torch.bfloat16).to(DEV)
        monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", False)
        y_ref = layer.apply(x)
        monkeypatch.setattr(LM, "_GLQ_MERGED_GROUPED", True)
        assert not layer._grouped_ok(B) and not layer._grouped_rvq2_ok(B)
        y = layer.apply(x)
        assert y.dtype == x.dtype and y.shape == y_ref.shape
        assert rel(y, _oracle(x, arts, n)) < TOL
        assert rel(y, y_ref.float().cpu().numpy()) < 6e-3
        assert torch.equal(y, layer.apply(x))


def _shell_indices(m, n, stages, seed):
    rng = np.random.default_rng(seed)
    lo = rng.integers(0, 30000, size=(stages, m, n // 8))
    hi = rng.integers(0, 65536, size=(stages, m, n // 8))
    return np.where(rng.random((stages, m, n // 8)) < 0.6, lo, hi).astype(np.uint16).view(np.int16)


@pytest.mark.parametrize("B", [1, 5, 70, 300])
def test_merged_shell_linear(ops, B):
    """E8-shell shards behind one activation (glq_vllm/linear_method.py:1490-1522 with `_glq_apply_shard` per
    shard): block-diagonal shards of one, two and four stages and a legacy shard padded to powers of two, each
    column range against the oracle's forward of that shard; the load-time step folds the index streams, so a
    captured first call equals the eager one."""
    from glq_amd import ext
    from glq_amd.linear_method import GLQShards, MergedShellLinear, process_weights_after_loading
    from tests.gpu_util import e8_table_f16
    say("merged shell linear", B)
    n, cb = 512, e8_table_f16()
    table = O.e8_table()
    inv = [1 / 3.0, 1 / 9.0, 1 / 27.0]

    def build(shards, n_in, legacy=False):
        layer = MergedShellLinear(n_in, [m for m, _ in shards], cb)
        arts = []
        for i, (m, stages) in enumerate(shards):
            m_pad, n_pad = (1 << (m - 1).bit_length(), 1 << (n_in - 1).bit_length()) if legacy else (m, n_in)
            q = _shell_indices(m_pad, n_pad, stages, 10 * i + stages)
            su, sv = O.rht_signs(m_pad, n_pad, 300 + i)
            W = sum(table[q[s].view(np.uint16).astype(np.int64)].reshape(m_pad, n_pad) * np.float32(inv[s - 1] if s else 1.0)
                    for s in range(stages)).astype(np.float32) * np.float32(0.02 + 0.001 * i)
            arts.append(dict(q=q, su=su, sv=sv, W=W, m=m, m_pad=m_pad, n_pad=n_pad, stages=stages, ws=0.02 + 0.001 * i))
        empty = torch.zeros(0, dtype=torch.int16)
        for s, name in enumerate(("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4")):
            setattr(layer, name, GLQShards(torch.from_numpy(a["q"][s].copy()) if s < a["stages"] else empty for a in arts))
        layer.SU = GLQShards(torch.from_numpy(a["su"].astype(np.float16)) for a in arts)
        layer.SV = GLQShards(torch.from_numpy(a["sv"].astype(np.float16)) for a in arts)
        layer.Wscale = GLQShards(torch.tensor(a["ws"], dtype=torch.float32) for a in arts)
        for s, name in enumerate(("inv_resid_scale", "inv_resid_scale2", "inv_resid_scale3")):
            setattr(layer, name, GLQShards(torch.tensor(inv[s] if s + 2 <= a["stages"] else 0.0, dtype=torch.float32)
                                           for a in arts))
        process_weights_after_loading(layer, DEV)
        return layer, arts

    def check(layer, arts, n_in, x):
        y = layer.apply(x)
        assert y.dtype == x.dtype and y.shape == (x.shape[0], sum(a["m"] for a in arts))
        col = 0
        for a in arts:
            legacy = a["m_pad"] != a["m"] or a["n_pad"] != n_in
            bn = [a["n_pad"]] if legacy else O.block_decompose(a["n_pad"])
            bm = [a["m_pad"]] if legacy else O.block_decompose(a["m_pad"])
            want = O.linear_forward_rht(np.pad(x.float().cpu().numpy(), ((0, 0), (0, a["n_pad"] - n_in))), a["W"],
                                        a["su"].astype(np.float32), a["sv"].astype(np.float32), bn, bm, a["n_pad"], a["m"])
            e = rel(y[:, col:col + a["m"]], want)
            assert e < TOL, (a["m"], a["stages"], e)
            col += a["m"]
        return y

    layer, arts = build([(256, 2), (64, 1), (96, 4)], n)
    assert all(m["bd_meta"] is not None for m in layer._glq_shard_meta)
    assert [m["n_stages"] for m in layer._glq_shard_meta] == [2, 1, 4]
    assert ext._FOLD_STREAMS.holds(layer.Qidxs.get_shard(0))     # folded at load time
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(B)) * 0.5).to(torch.bfloat16).to(DEV)
    y = check(layer, arts, n, x)
    assert torch.equal(y, layer.apply(x))
    if B == 1:                                                   # a captured first call of a fresh layer
        fresh, _ = build([(256, 2), (64, 1), (96, 4)], n)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            yc = fresh.apply(x)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(yc, y)
    legacy, larts = build([(200, 2)], 300, legacy=True)          # buffers of 256 x 512
    assert legacy._glq_shard_meta[0]["bd_meta"] is None and legacy._glq_shard_meta[0]["m_pad"] == 256
    xl = (torch.randn(B, 300, generator=torch.Generator().manual_seed(B + 1)) * 0.5).half().to(DEV)
    check(legacy, larts, 300, xl)
    bad, _ = build([(64, 1)], n)
    bad.inv_resid_scale._shard_data[0] = torch.tensor(0.3)
    with pytest.raises(RuntimeError, match="half-configured"):
        bad.process_weights_after_loading(DEV)


@pytest.mark.parametrize("B", [1, 3, 100])
def test_more_shards_than_a_grouped_call_takes(ops, B):
    """Five merged shards: the grouped call takes at most four layers, so the default falls back to the
    reference's sequence (whole fused linears from 64 tokens on); against the oracle."""
    say("merged linear, five shards", B)
    n = 512
    layer, arts = _merged(n, [(64, 4, 0)] * 5, 4)
    assert not layer._grouped_ok(B)
    x = (torch.randn(B, n, generator=torch.Generator().manual_seed(B)) * 0.5).to(torch.bfloat16).to(DEV)
    y = layer.apply(x)
    assert y.shape == (B, 320) and rel(y, _oracle(x, arts, n)) < TOL


def test_merged_linears_without_tokens_and_with_more_than_a_launch_takes(ops):
    """An empty batch gives an empty result without a launch; more tokens than one call takes (32768, as in
    E8RHTLinear.forward) are served in pieces: rows of the long call equal the rows of a short one."""
    from glq_amd.linear_method import MergedShellLinear
    from tests.gpu_util import e8_table_f16
    say("merged linears, 0 and 70000 tokens")
    n = 512
    layer, _ = _merged(n, [(256, 4, 0), (64, 4, 0), (64, 4, 0)], 4)
    two, _ = _merged(n, [(352, 4, 2), (352, 4, 2)], 6)
    shell = MergedShellLinear(n, [128, 64], e8_table_f16())
    from glq_amd.linear_method import GLQShards
    shell.Qidxs = GLQShards(torch.from_numpy(_shell_indices(m, n, 1, m)[0].copy()) for m in (128, 64))
    shell.Wscale = GLQShards(torch.tensor(0.02) for _ in range(2))
    shell.process_weights_after_loading(DEV)
    for L, width in ((layer, 384), (two, 704), (shell, 192)):
        y0 = L.apply(torch.zeros(0, n, dtype=torch.bfloat16, device=DEV))
        assert y0.shape == (0, width) and y0.dtype == torch.bfloat16
        assert L.apply(torch.zeros(2, 0, n, dtype=torch.float16, device=DEV)).shape == (2, 0, width)
        x = (torch.randn(70000, n, generator=torch.Generator().manual_seed(1)) * 0.5).to(torch.bfloat16).to(DEV)
        y = L.apply(x)
        assert y.shape == (70000, width) and bool(torch.isfinite(y.float()).all())
        for lo in (0, 32763, 65535, 69990):
            assert rel(y[lo:lo + 10], L.apply(x[lo:lo + 10]).float().cpu().numpy()) < 6e-3
