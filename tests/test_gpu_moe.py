"""Routed-expert step of a mixture-of-experts layer on stacked trellis-3INST experts
(glq_fused_moe_trellis_3inst_cuda, glq/csrc/glq_cuda.cu:5030-5250) against the oracle's
moe_trellis_forward.  Floating point: relative Frobenius error <= 1e-2, the reference's own bar
for the fused linears (tests/test_trellis_parity.py)."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, rel, say, t
from oracle import glq_oracle as O

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def ext():
    from glq_amd import ext as e
    return e


class Experts:
    """E experts of one layer: w13 (hidden -> gate | up) and w2 (intermediate -> hidden), every
    expert with its own code bits, output signs and scale; the input signs are shared."""

    def __init__(self, E, hidden, inter, K=4, K2=0, seed=0):
        self.E, self.hidden, self.inter = E, hidden, inter
        self.arts = {"w13": [], "w2": []}
        for name, m, n in (("w13", 2 * inter, hidden), ("w2", hidden, inter)):
            _, sv = O.rht_signs(m, n, 7 + seed)
            for e in range(E):
                su, _ = O.rht_signs(m, n, 100 * seed + 10 * e + (name == "w2"))
                art = {"trellis_packed": O.random_packed(m, n, K, 1000 * seed + 2 * e + (name == "w2")),
                       "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
                       "Wscale": np.float32((0.04 + 0.01 * e) * O.trellis_opt_scale()),
                       "blocks_m": O.block_decompose(m), "blocks_n": O.block_decompose(n)}
                if K2:
                    art["trellis_packed2"] = O.random_packed(m, n, K2, 5000 + 2 * e + (name == "w2"))
                    art["inv_resid_scale2"] = np.float32(0.2 + 0.03 * e)
                self.arts[name].append(art)
        self.dense13 = O.moe_dense_experts(self.arts["w13"], 2 * inter, hidden)
        self.dense2 = O.moe_dense_experts(self.arts["w2"], hidden, inter)

    def device_args(self, act):
        from glq_amd import hadamard as H
        out = []
        metas = []
        for name, m, n in (("w13", 2 * self.inter, self.hidden), ("w2", self.hidden, self.inter)):
            a = self.arts[name]
            packed = t(np.stack([x["trellis_packed"] for x in a]))
            if "trellis_packed2" in a[0]:
                packed2 = t(np.stack([x["trellis_packed2"] for x in a]))
                inv2 = t(np.array([x["inv_resid_scale2"] for x in a], np.float32))
            else:                                          # the placeholder the reference registers
                packed2 = torch.zeros(self.E, 1, 1, dtype=torch.int16, device=DEV)
                inv2 = torch.zeros(self.E, dtype=torch.float32, device=DEV)
            out += [packed, packed2, t(np.stack([x["SU"] for x in a])), t(a[0]["SV"]),
                    t(np.array([x["Wscale"] for x in a], np.float32)), inv2]
            bn, bm = a[0]["blocks_n"], a[0]["blocks_m"]
            metas.append((torch.tensor(bn, dtype=torch.int64), torch.tensor(bm, dtype=torch.int64),
                          H.pack_block_meta(bn).to(DEV), H.pack_block_meta(bm).to(DEV)))
        out += [self.hidden, self.inter, 2 * self.inter, self.hidden, 2 * self.inter, self.inter, self.hidden]
        out += list(metas[0]) + list(metas[1]) + [act]
        return out

    def oracle(self, x, ids, w, act):
        return O.moe_trellis_forward(x, ids, w, self.arts["w13"], self.arts["w2"], self.hidden, self.inter,
                                     act, self.dense13, self.dense2)


_cache = {}


def experts(E, hidden, inter, K=4, K2=0, seed=0):
    key = (E, hidden, inter, K, K2, seed)
    if key not in _cache:
        _cache[key] = Experts(*key)
    return _cache[key]


def routing(T, K, E, seed):
    rng = np.random.default_rng(seed)
    ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int64)
    w = rng.random((T, K)).astype(np.float32)
    w /= w.sum(1, keepdims=True)
    return ids, w


@pytest.mark.parametrize("hidden,inter", [(256, 128), (320, 192)])
@pytest.mark.parametrize("T,K", [(1, 1), (1, 4), (3, 2), (9, 4)])
@pytest.mark.parametrize("act", [0, 1, 2])
def test_routed_experts_match_oracle(ext, hidden, inter, T, K, act):
    say("moe", hidden, inter, T, K, act)
    ex = experts(6, hidden, inter)
    ids, w = routing(T, K, 6, T * 10 + K)
    x = torch.from_numpy(np.random.default_rng(T).standard_normal((T, hidden)).astype(np.float32)).half()
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *ex.device_args(act))
    assert y.shape == (T, hidden) and y.dtype == torch.float16
    ref = ex.oracle(x.float().numpy(), ids, w, act)
    assert rel(y, ref) < TOL, rel(y, ref)
    # fixed order of summation: the same call gives the same bits
    assert torch.equal(y, ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *ex.device_args(act)))


@pytest.mark.parametrize("K1,K2", [(4, 2), (3, 1), (2, 2)])
def test_two_stage_experts_and_bf16_input(ext, K1, K2):
    say("moe two-stage", K1, K2)
    ex = experts(4, 320, 192, K1, K2, seed=1)
    ids, w = routing(5, 2, 4, 3)
    x = torch.from_numpy(np.random.default_rng(2).standard_normal((5, 320)).astype(np.float32)).bfloat16()
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *ex.device_args(0))
    assert y.dtype == torch.bfloat16
    ref = ex.oracle(x.float().numpy(), ids, w, 0)
    assert rel(y, ref) < TOL, rel(y, ref)


def test_out_of_range_experts_contribute_nothing(ext):
    say("moe pad slots")
    ex = experts(6, 256, 128)
    x = torch.from_numpy(np.random.default_rng(5).standard_normal((3, 256)).astype(np.float32)).half()
    ids = np.array([[1, -1, 4], [6, 2, 0], [-1, 99, -7]], np.int64)
    w = np.full((3, 3), 1 / 3, np.float32)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *ex.device_args(0))
    ref = ex.oracle(x.float().numpy(), ids, w, 0)
    assert rel(y[:2], ref[:2]) < TOL
    assert torch.count_nonzero(y[2]) == 0 and not ref[2].any()
    # int32 routing tensors (what a router's topk returns after a cast) are accepted as well
    y32 = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids.astype(np.int32)), t(w), *ex.device_args(0))
    assert torch.equal(y, y32)


def test_single_choice_equals_the_fused_linears(ext):
    """One expert with weight 1 is down(act(gate) * up): the same library's fused trellis linear,
    called per projection with that expert's tensors, gives the operands."""
    say("moe vs linears")
    ex = experts(6, 320, 192)
    e = 3
    x = torch.from_numpy(np.random.default_rng(8).standard_normal((2, 320)).astype(np.float32)).half().to(DEV)
    a = ex.device_args(0)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x, t(np.full((2, 1), e, np.int64)), t(np.ones((2, 1), np.float32)), *a)
    bn13, bm13, bn13m, bm13m, bn2, bm2, bn2m, bm2m = a[19:27]
    h = ext.glq_fused_linear_trellis_3inst_cuda(x, a[3], a[2][e], a[0][e], bn13, bm13, bn13m, bm13m,
                                                float(a[4][e]), 320, 384, 320, 384, out_dtype=torch.float16)
    act = (torch.nn.functional.silu(h[:, :192].float()) * h[:, 192:].float()).half()
    y2 = ext.glq_fused_linear_trellis_3inst_cuda(act, a[9], a[8][e], a[6][e], bn2, bm2, bn2m, bm2m,
                                                 float(a[10][e]), 192, 320, 192, 320, out_dtype=torch.float16)
    assert rel(y, y2) < 2e-3, rel(y, y2)


@pytest.mark.parametrize("T", [4, 700])
def test_registered_op_and_graph_replay(ext, T):
    """T = 700: 1400 slots on 6 experts, the tile kernel's form, whose token tiles are listed on the device
    from the routing of each replay."""
    say("moe op + graph", T)
    from glq_amd import custom_ops
    custom_ops.register()
    ex = experts(6, 256, 128)
    ids, w = routing(T, 2, 6, 11)
    x = torch.from_numpy(np.random.default_rng(9).standard_normal((T, 256)).astype(np.float32)).half().to(DEV)
    a = ex.device_args(0)
    ids_d, w_d = t(ids), t(w)
    eager = ext.glq_fused_moe_trellis_3inst_cuda(x, ids_d, w_d, *a)
    y = torch.ops.glq.fused_moe_trellis_3inst(x, ids_d, w_d, *a)
    assert torch.equal(y, eager)
    # the routing is read on the device: a captured call follows new routing tensors' contents
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        ext.glq_fused_moe_trellis_3inst_cuda(x, ids_d, w_d, *a)
    torch.cuda.current_stream().wait_stream(s)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = ext.glq_fused_moe_trellis_3inst_cuda(x, ids_d, w_d, *a)
    for rep in range(3):
        ids2, w2 = routing(T, 2, 6, 20 + rep)
        if rep == 1:                                           # skewed: expert 2 is every token's first choice
            ids2[:, 1] = np.where(ids2[:, 1] == 2, ids2[:, 0], ids2[:, 1])
            ids2[:, 0] = 2
        ids_d.copy_(t(ids2)); w_d.copy_(t(w2))
        want = ext.glq_fused_moe_trellis_3inst_cuda(x, ids_d, w_d, *a)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        assert rel(out, ex.oracle(x.float().cpu().numpy(), ids2, w2, 0)) < TOL


def test_empty_batch(ext):
    say("moe empty batch")
    ex = experts(6, 256, 128)
    x = torch.zeros(0, 256, dtype=torch.float16, device=DEV)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x, torch.zeros(0, 2, dtype=torch.int64, device=DEV),
                                             torch.zeros(0, 2, device=DEV), *ex.device_args(0))
    assert y.shape == (0, 256) and y.dtype == torch.float16


def test_refusals(ext):
    say("moe refusals")
    ex = experts(6, 256, 128)
    a = ex.device_args(0)
    x = torch.zeros(2, 256, dtype=torch.float16, device=DEV)
    ids, w = t(np.zeros((2, 1), np.int64)), t(np.ones((2, 1), np.float32))
    with pytest.raises(RuntimeError, match="gated"):
        ext.glq_fused_moe_trellis_3inst_cuda(x, ids, w, *a[:-1], 3)
    with pytest.raises(RuntimeError, match="hidden"):
        ext.glq_fused_moe_trellis_3inst_cuda(x[:, :128].contiguous(), ids, w, *a)
    with pytest.raises(RuntimeError, match="top_k"):
        ext.glq_fused_moe_trellis_3inst_cuda(x, ids[:1], w, *a)
    b = list(a)
    b[13] = 64                                             # intermediate size that does not match w13
    with pytest.raises(RuntimeError, match="intermediate"):
        ext.glq_fused_moe_trellis_3inst_cuda(x, ids, w, *b)


@pytest.mark.parametrize("hidden,inter,T,K,K2", [(256, 128, 16, 4, 0), (320, 192, 40, 2, 0), (320, 192, 33, 3, 2),
                                                 (256, 128, 24, 4, 0), (256, 128, 90, 2, 0), (256, 128, 80, 3, 1),
                                                 (256, 128, 200, 3, 0), (320, 192, 300, 2, 2), (256, 128, 530, 2, 0),
                                                 (256, 128, 1100, 4, 0), (320, 192, 600, 2, 2)])
def test_many_slots_grouped_by_expert(ext, hidden, inter, T, K, K2):
    """From max(16, 3/4 of the experts) slots on the rows are grouped by expert.  Skewed routing: every token's first choice is
    expert 2 (more than two tiles of 16 rows for it), expert 5 gets nothing, some ids are out of range.  From an
    average of 12 rows per expert on, a pass over an expert's stream takes up to 64 of its rows: the cases give
    expert 2 one pass of 16 (T = 16), of 32 (24), of 64 (33, 40), 64 + 32 (90) and 64 + 16 (80) rows.  From 48 rows
    per expert on average the sorted slots go through the tile kernel in runs of up to 256 positions of one
    expert: expert 2 has one run of 199 (T = 200), two of 160 and 139 (300), three of 192, 192 and 145 (530), the
    other experts one partial run each.  T = 1100: 4400 slots, whose routing table is made by two launches over
    three segments of the slots, and runs of up to 512 positions.  T = 600 with two-stage experts: 1200 slots, from
    1024 on one launch between the projections and one after them, here on the sums of both stages."""
    say("moe grouped", hidden, inter, T, K, K2)
    ex = experts(6, hidden, inter, 4, K2, seed=2)
    rng = np.random.default_rng(T)
    ids = np.stack([np.concatenate([[2], rng.permutation([0, 1, 3, 4])[:K - 1]]) for _ in range(T)]).astype(np.int64)
    ids[3, K - 1] = -1
    ids[T - 1, 0] = 6
    w = rng.random((T, K)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((T, hidden)).astype(np.float32)).bfloat16()
    a = ex.device_args(1)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *a)
    ref = ex.oracle(x.float().numpy(), ids, w, 1)
    assert rel(y, ref) < TOL, rel(y, ref)
    worst = max(rel(y[i], ref[i]) for i in range(T))
    assert worst < 3 * TOL, worst                            # no single token is off
    assert torch.equal(y, ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *a))


@pytest.mark.parametrize("hidden,inter", [(256, 4096), (8192, 128)])
def test_rows_with_a_block_of_8192_points(ext, hidden, inter):
    """The first projection's row (2 x 4096 = one block of 8192 points) or the second's (hidden 8192) takes sixteen
    elements per thread in the launches between and after the projections; 600 tokens x 2 choices over 3 experts
    (tile kernel, fused launches)."""
    say("moe large blocks", hidden, inter)
    ex = experts(3, hidden, inter, seed=5)
    T, K = 600, 2
    rng = np.random.default_rng(1)
    ids = np.stack([rng.permutation(3)[:K] for _ in range(T)]).astype(np.int64)
    ids[7, 1] = -1
    w = rng.random((T, K)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((T, hidden)).astype(np.float32)).bfloat16()
    a = ex.device_args(0)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *a)
    ref = ex.oracle(x.float().numpy(), ids, w, 0)
    assert rel(y, ref) < TOL, rel(y, ref)
    assert torch.equal(y, ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *a))


def test_large_activations_stay_finite_in_the_tile_form(ext):
    """Squared-ReLU experts on activations of a few units: the second projection's unscaled sums pass the fp16
    range while the result does not; the tile form's fp16 sums carry the expert's scale, so it stays finite and
    inside the bound (1500 tokens x 5 choices over 22 experts, two-stage experts, runs of up to 512 positions)."""
    say("moe large activations")
    ex = experts(22, 448, 320, 4, 1, seed=9)
    rng = np.random.default_rng(3)
    T, K = 1500, 5
    ids = np.stack([rng.permutation(22)[:K] for _ in range(T)]).astype(np.int64)
    w = rng.random((T, K)).astype(np.float32)
    x = torch.from_numpy(rng.standard_normal((T, 448)).astype(np.float32)).bfloat16()
    ref = ex.oracle(x.float().numpy(), ids, w, 2)
    assert bool(np.isfinite(ref).all())
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *ex.device_args(2))
    assert bool(torch.isfinite(y.float()).all())
    assert rel(y, ref) < TOL, rel(y, ref)


@pytest.mark.parametrize("group_min,wide_min,tile_min,tile_ntw,fuse,pc_steps", [
    ("1", "1", "0", "", "1", ""), ("1", "1000000", "0", "", "0", ""), ("1000000", "12", "0", "", "1", ""),
    ("1", "12", "1", "", "1", ""), ("1", "12", "1", "1", "0", ""), ("1", "12", "1", "4", "1", ""),
    ("1000000", "12", "0", "", "0", ""), ("1", "12", "1", "", "1", "1"), ("1", "12", "1", "1", "0", "1"),
    ("1", "12", "1", "4", "1", "1")])
def test_both_forms_on_every_case_in_a_fresh_process(group_min, wide_min, tile_min, tile_ntw, fuse, pc_steps):
    """GLQ_MOE_GROUP_MIN (read once by the library) moves the slot count from which rows are grouped by
    expert: with 1 every case of this file runs in the grouped form, with 1000000 in the per-slot form,
    each against the oracle, in a process of its own.  GLQ_MOE_WIDE_MIN_ROWS moves the average number of rows
    per expert from which the grouped form takes up to 64 rows per pass: 1 = always, 1000000 = never.
    GLQ_MOE_TILE_MIN_ROWS the average from which the tile kernel takes the grouped rows: 0 = never, 1 = always,
    then with runs of up to 256 positions, or 128 / 512 with GLQ_MOE_TILE_NTW = 1 / 4.  GLQ_MOE_FUSE=0 keeps the
    launches between and after the two decode launches separate (output transform, activation, input
    transform; output transform, weighted sum) where one launch each is the default.  GLQ_TT_PC_STEPS=1: runs of
    up to 256 positions with four decoding and four multiplying waves whatever the length of the rows (by
    default from 8 steps of 64 columns on)."""
    import os
    import subprocess
    import sys
    say("moe forms, child process", group_min, wide_min, tile_min, tile_ntw, fuse, pc_steps)
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-m", "gpu",
                        "-k", "not fresh_process", "--timeout", "300", "--timeout-method", "thread",
                        "-p", "no:cacheprovider"],
                       env={**os.environ, "GLQ_MOE_GROUP_MIN": group_min, "GLQ_MOE_WIDE_MIN_ROWS": wide_min,
                            "GLQ_MOE_TILE_MIN_ROWS": tile_min, "GLQ_MOE_FUSE": fuse, **({"GLQ_MOE_TILE_NTW": tile_ntw} if tile_ntw else {}),
                            **({"GLQ_TT_PC_STEPS": pc_steps} if pc_steps else {})},
                       capture_output=True, text=True, timeout=900,
                       cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-1000:])


@pytest.mark.parametrize("T", [1, 4, 40, 140])
def test_qwen3_moe_expert_shapes(ext, T):
    """Expert shapes of a Qwen3-MoE layer (hidden 2048, intermediate 768, top-8), 16 of the experts,
    4 bpw, bf16 activations: every chosen expert decoded whole by the oracle.  One and four tokens run slot by
    slot, 40 tokens grouped by expert (20 rows each on average), 140 tokens through the tile kernel (70 rows
    each, runs of up to 128 positions, 1120 slots: with the fused launches around the second projection)."""
    say("moe qwen3 shapes", T)
    ex = experts(16, 2048, 768, seed=3)
    ids, w = routing(T, 8, 16, T)
    x = torch.from_numpy(np.random.default_rng(T).standard_normal((T, 2048)).astype(np.float32)).bfloat16()
    a = ex.device_args(0)
    y = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(w), *a)
    ref = ex.oracle(x.float().numpy(), ids, w, 0)
    assert rel(y, ref) < TOL, rel(y, ref)
    # the routing weights enter linearly, after every rounding but the last
    y2 = ext.glq_fused_moe_trellis_3inst_cuda(x.to(DEV), t(ids), t(2 * w), *a)
    assert rel(y2, 2 * y.float()) < 1e-2
