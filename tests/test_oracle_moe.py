"""The oracle's routed-expert forward (mixture of experts on trellis weights), pinned without a
golden vector: the reference tests only the op's schema (tests/test_glq_vllm.py:595-640), so the
function is checked as a composition of pinned parts and through the invariants the operation has."""
import math

import numpy as np

from oracle import glq_oracle as O

HID, INTER, E = 128, 64, 4


def _experts(seed, two_stage=False):
    w13, w2 = [], []
    for e in range(E):
        for arts, m, n in ((w13, 2 * INTER, HID), (w2, HID, INTER)):
            su, sv = O.rht_signs(m, n, 100 + seed)               # the experts share SV, SU differs
            su_e, _ = O.rht_signs(m, n, 1000 * seed + e)
            art = {"trellis_packed": O.random_packed(m, n, 4, 10 * seed + e + (0 if m == HID else 50)),
                   "SU": su_e.astype(np.float16), "SV": sv.astype(np.float16),
                   "Wscale": np.float32(0.05 + 0.01 * e), "blocks_m": O.block_decompose(m),
                   "blocks_n": O.block_decompose(n)}
            if two_stage:
                art["trellis_packed2"] = O.random_packed(m, n, 2, 77 + e)
                art["inv_resid_scale2"] = np.float32(0.25 + 0.05 * e)
            arts.append(art)
    return w13, w2


def test_activation_known_values():
    h = np.array([[1.0, -1.0, 2.0, 0.0, 3.0, 5.0, 7.0, 11.0]], np.float32)        # gate | up, intermediate 4
    silu = O.gated_activation(h, 4, 0)[0]
    assert np.allclose(silu, [1 / (1 + math.exp(-1)) * 3, -1 / (1 + math.e) * 5, 2 / (1 + math.exp(-2)) * 7, 0], atol=1e-6)
    gelu = O.gated_activation(h, 4, 1)[0]
    g1 = 0.5 * (1 + math.tanh(0.7978845608028654 * (1 + 0.044715)))
    assert abs(gelu[0] - g1 * 3) < 1e-6 and abs(g1 - 0.841192) < 1e-5 and gelu[3] == 0
    relu2 = O.gated_activation(h, 4, 2)[0]
    assert list(relu2) == [3.0, 0.0, 28.0, 0.0]


def test_single_choice_is_the_composition_of_two_linears():
    for act in (0, 1, 2):
        w13, w2 = _experts(1)
        x = np.random.default_rng(act).standard_normal((2, HID)).astype(np.float32)
        ids = np.array([[2], [0]])
        got = O.moe_trellis_forward(x, ids, np.ones((2, 1), np.float32), w13, w2, HID, INTER, act)
        for t in range(2):
            e = int(ids[t, 0])
            h = O.trellis_linear_forward(x[t:t + 1], w13[e], HID, 2 * INTER).astype(np.float16).astype(np.float64)[0]
            a = np.empty(INTER)
            for i in range(INTER):                                # the activation written out with math.*
                g, up = h[i], h[INTER + i]
                if act == 0:
                    v = g / (1 + math.exp(-g))
                elif act == 1:
                    v = 0.5 * g * (1 + math.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))
                else:
                    v = max(g, 0.0) ** 2
                a[i] = v * up
            a = a.astype(np.float16).astype(np.float32)[None]
            y = O.trellis_linear_forward(a, w2[e], INTER, HID).astype(np.float16).astype(np.float32)
            assert O.rel_fro(got[t], y[0]) < 2e-3, (act, t)


def test_linear_in_the_routing_weights_and_order_free():
    w13, w2 = _experts(2, two_stage=True)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((3, HID)).astype(np.float32)
    ids = np.array([[0, 3, 1], [2, 2, 0], [1, 0, 3]])
    w = rng.random((3, 3)).astype(np.float32)
    base = O.moe_trellis_forward(x, ids, w, w13, w2, HID, INTER, 0)
    assert O.rel_fro(O.moe_trellis_forward(x, ids, 2 * w, w13, w2, HID, INTER, 0), 2 * base) < 1e-3
    perm = [2, 0, 1]
    assert O.rel_fro(O.moe_trellis_forward(x, ids[:, perm], w[:, perm], w13, w2, HID, INTER, 0), base) < 1e-3
    # a sum over choices is the sum of the single-choice results
    parts = sum(O.moe_trellis_forward(x, ids[:, j:j + 1], w[:, j:j + 1], w13, w2, HID, INTER, 0) for j in range(3))
    assert O.rel_fro(parts, base) < 2e-3


def test_out_of_range_experts_contribute_nothing():
    w13, w2 = _experts(3)
    x = np.random.default_rng(1).standard_normal((2, HID)).astype(np.float32)
    w = np.array([[0.5, 0.25], [1.0, 0.5]], np.float32)
    a = O.moe_trellis_forward(x, np.array([[1, -1], [E, 2]]), w, w13, w2, HID, INTER, 2)
    b = O.moe_trellis_forward(x, np.array([[1], [2]]), w[[0, 1], [0, 1]][:, None], w13, w2, HID, INTER, 2)
    assert np.array_equal(a, b)
