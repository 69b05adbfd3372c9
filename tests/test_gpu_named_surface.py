"""The module-level names of the reference's Python kernels (glq.inference_kernel,
glq.hadamard, glq.codebook_kernel, glq.trellis_step_kernel) on the HIP library, against
the oracle (needs an MI355X)."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, e8_table_f16, rel, say, t

pytestmark = pytest.mark.gpu


def _gpu_viterbi(X, K, lut, overlap=None):
    """The control flow of bitshift_codebook.viterbi (glq/trellis.py:253-296) with every
    add-compare-select step done by fused_update on the GPU; start costs, masks and the
    traceback in numpy."""
    from glq_amd.trellis_step_kernel import fused_update
    T, B = X.shape
    S, G = 1 << 16, 1 << (16 - K)
    lutf = lut.astype(np.float32)
    cb = SimpleNamespace(L=16, K=K, V=1, recons_state=t(lutf).reshape(1, 1, S))
    inf = np.float32(np.inf)
    cost = (lutf[None, :] - X[0][:, None]) ** 2
    if overlap is not None:
        mask = np.full((B, S), inf, dtype=np.float32)
        np.put_along_axis(mask, (overlap[:, None].astype(np.int64) << K) + np.arange(1 << K)[None, :], 0.0, axis=1)
        cost = np.minimum(cost + mask, inf)
    cost = t(cost.astype(np.float32))
    Xd = t(X.astype(np.float16))
    from_state = torch.empty(T, B, G, dtype=torch.int32, device=DEV)
    for i in range(1, T):
        cost = fused_update(cb, cost, Xd[i:i + 1], from_state[i])
    cost = cost.cpu().numpy()
    fs = from_state.cpu().numpy()
    if overlap is not None:
        mask = np.full((B, S), inf, dtype=np.float32)
        np.put_along_axis(mask, overlap[:, None].astype(np.int64) + (np.arange(1 << K)[None, :] << (16 - K)),
                          0.0, axis=1)
        cost = np.minimum(cost + mask, inf)
    final = np.empty((T, B), dtype=np.int64)
    final[T - 1] = cost.argmin(-1)
    for i in range(T - 1, 0, -1):
        final[i - 1] = np.take_along_axis(fs[i], (final[i] >> K)[:, None], axis=1)[:, 0]
    return final, cost


@pytest.mark.parametrize("K", [1, 2, 3, 4])
def test_fused_update_steps_reproduce_the_search(K):
    """255 single steps composed = the oracle's search (pinned on the reference's state
    sequences), free and with the tail-biting masks (+inf costs)."""
    say("fused_update", K)
    rng = np.random.default_rng(K)
    lut = O.lut_3inst()
    B = 3
    X = rng.standard_normal((256, B)).astype(np.float16).astype(np.float32)
    st, _ = _gpu_viterbi(X, K, lut)
    assert np.array_equal(st, O._viterbi(X, K, lut))
    overlap = st[128] >> K
    st2, _ = _gpu_viterbi(X, K, lut, overlap=overlap)
    assert np.array_equal(st2, O._viterbi(X, K, lut, overlap=overlap))


def test_fused_update_single_step_values_ties_and_nan():
    """One step against the formula of glq/trellis.py:238-250 written out in numpy: exact
    cost values, lowest k on exact ties, a NaN candidate wins, +inf rows stay +inf."""
    from glq_amd.trellis_step_kernel import fused_update
    say("fused_update single step")
    K, S = 2, 1 << 16
    G = S >> K
    rng = np.random.default_rng(7)
    lut = O.lut_3inst().astype(np.float32)
    cost = rng.standard_normal((2, S)).astype(np.float32) ** 2
    cost[0, 5] = cost[0, G + 5] = cost[0, 2 * G + 5] = cost[0, 3 * G + 5] = np.float32(0.25)   # four-way tie
    cost[0, 2 * G + 9] = np.float32(np.nan)
    cost[1, :] = np.float32(np.inf)
    cost[1, 3 * G + 77] = np.float32(1.5)
    x = np.array([0.375, -1.25], dtype=np.float16)
    c = cost.reshape(2, 1 << K, G)
    with np.errstate(invalid="ignore"):
        k = np.where(np.isnan(c).any(axis=1), np.isnan(c).argmax(axis=1), np.nan_to_num(c, nan=np.inf).argmin(axis=1))
    best = np.take_along_axis(c, k[:, None, :], axis=1)[:, 0, :]
    prev_ref = (np.arange(G)[None, :] + (k << (16 - K))).astype(np.int32)
    d = lut[None, :] - x.astype(np.float32)[:, None]
    ref = (d * d).astype(np.float32) + np.repeat(best, 1 << K, axis=1)
    cb = SimpleNamespace(L=16, K=K, V=1, recons_state=t(lut).reshape(1, 1, S))
    prev = torch.empty(2, G, dtype=torch.int32, device=DEV)
    out = fused_update(cb, t(cost), t(x).reshape(1, 2), prev)
    assert np.array_equal(prev.cpu().numpy(), prev_ref)
    assert prev_ref[0, 5] == 5 and prev_ref[0, 9] == 9 + 2 * G and prev_ref[1, 77] == 77 + 3 * G
    assert np.array_equal(out.cpu().numpy(), ref, equal_nan=True)
    with pytest.raises(KeyError):
        fused_update(SimpleNamespace(L=16, K=2, V=2, recons_state=cb.recons_state), t(cost), t(x), prev)


@pytest.mark.parametrize("shape", [(5, 512), (2, 3, 64), (2048,), (70, 4096), (1, 32768)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_fast_hadamard_transform(shape, dtype):
    from glq_amd.hadamard import fast_hadamard_transform
    say("fast_hadamard_transform", shape, dtype)
    rng = np.random.default_rng(shape[-1])
    x = rng.standard_normal(shape).astype(np.float32)
    xd = t(x, dtype)
    y = fast_hadamard_transform(xd)
    assert y.shape == xd.shape and y.dtype == dtype
    ref = O.fht(xd.float().cpu().numpy())
    assert rel(y, ref) < (1e-5 if dtype == torch.float32 else 1e-3)


def test_block_diagonal_fht_in_place():
    from glq_amd.hadamard import _block_decompose, block_diagonal_fht
    say("block_diagonal_fht")
    rng = np.random.default_rng(3)
    blocks = _block_decompose(2688)
    assert blocks == [2048, 512, 128]
    x = rng.standard_normal((4, 2688)).astype(np.float32)
    xd = t(x)
    y = block_diagonal_fht(xd, blocks)
    assert y.data_ptr() == xd.data_ptr()
    assert rel(xd, O.block_diag_fht(x, blocks)) < 1e-5
    with pytest.raises(RuntimeError, match="GPU only"):
        block_diagonal_fht(torch.zeros(1, 64), [64])


def test_codebook_nn_names():
    from glq_amd.codebook_kernel import triton_codebook_nn, triton_codebook_nn_decode
    say("triton_codebook_nn")
    rng = np.random.default_rng(11)
    cb = O.e8_table()
    X = rng.standard_normal((777, 8)).astype(np.float32)
    dec_ref, idx_ref = O.e8_quantize(X)
    cbd = e8_table_f16()
    norms = (cbd.float() ** 2).sum(-1)
    idx = triton_codebook_nn(t(X), cbd, norms)
    assert idx.dtype == torch.int64 and np.array_equal(idx.cpu().numpy(), idx_ref)
    out = torch.empty(777, dtype=torch.int32, device=DEV)
    assert triton_codebook_nn(t(X), cbd, norms, out=out) is out and np.array_equal(out.cpu().numpy(), idx_ref)
    dec, idx2 = triton_codebook_nn_decode(t(X), cbd, norms)
    assert dec.dtype == torch.float16 and np.array_equal(dec.float().cpu().numpy(), dec_ref)
    assert torch.equal(idx2, idx)
    assert np.array_equal(cb[idx_ref], dec_ref)


@pytest.mark.parametrize("B,stages,packed", [(1, 1, False), (1, 2, False), (4, 1, True), (4, 2, True),
                                             (3, 4, False), (1, 3, False)])
def test_glq_dequant_matmul_dispatch(B, stages, packed):
    """The routes of glq/inference_kernel.py:1038-1069 all give the oracle's product."""
    from glq_amd import inference_kernel as ik
    say("glq_dequant_matmul", B, stages, packed)
    assert ik.cuda_ext_status() == (True, None)
    assert ik.require_cuda_ext("glq_dequant_matmul_packed_cuda") is ik._glq_cuda
    with pytest.raises(RuntimeError, match="no 'glq_not_there'"):
        ik.require_cuda_ext("glq_not_there")
    m, n = 96, 160
    rng = np.random.default_rng(B * 10 + stages)
    q = [rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16) for _ in range(4)]
    sc = [1 / 3.0, 1 / 9.0, 1 / 27.0]
    x = (rng.standard_normal((B, n)) * 0.5).astype(np.float32)
    cb32 = t(O.e8_table())                                   # fp32 table, as the modules hold it
    cbp = t(O.e8_nibbles().view(np.int32)) if packed else None
    kw = {}
    if stages >= 2:
        kw.update(Qidxs2=t(q[1]), codebook2=cb32, inv_resid_scale=sc[0])
    if stages >= 3:
        kw.update(Qidxs3=t(q[2]), codebook3=cb32, inv_resid_scale2=sc[1])
    if stages >= 4:
        kw.update(Qidxs4=t(q[3]), codebook4=cb32, inv_resid_scale3=sc[2])
    y = ik.glq_dequant_matmul(t(x), t(q[0]), cb32, 0.021, codebook_packed=cbp, **kw)
    W = O.e8_dequant(q[0], q[1] if stages >= 2 else None, sc[0] if stages >= 2 else 0.0,
                     q[2] if stages >= 3 else None, sc[1] if stages >= 3 else 0.0,
                     q[3] if stages >= 4 else None, sc[2] if stages >= 4 else 0.0)
    ref = x.astype(np.float16).astype(np.float32) @ W.T * np.float32(0.021)
    assert y.shape == (B, m) and y.dtype == torch.float32
    assert rel(y, ref) < 1e-3, rel(y, ref)
    with pytest.raises(RuntimeError, match="GPU only"):
        ik.glq_dequant_matmul(torch.zeros(1, n), t(q[0]), cb32, 1.0)
