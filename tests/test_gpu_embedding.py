"""E8RHTEmbedding on the GPU against the oracle (through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import glq_oracle as O
from tests.gpu_util import DEV, rel, say, t

pytestmark = pytest.mark.gpu


def _make(vocab, dim, seed, two):
    rng = np.random.default_rng(seed)
    n_pad = O.next_pow2(dim)
    q1 = rng.integers(0, 65536, (vocab, n_pad // 8)).astype(np.uint16).view(np.int16)
    q2 = rng.integers(0, 65536, (vocab, n_pad // 8)).astype(np.uint16).view(np.int16) if two else None
    sv = rng.choice([-1.0, 1.0], n_pad).astype(np.float16)
    ws = rng.uniform(0.01, 0.05, vocab).astype(np.float32)
    inv = rng.uniform(0.2, 0.4, vocab).astype(np.float32) if two else None
    return n_pad, q1, q2, sv, ws, inv


@pytest.mark.parametrize("vocab,dim,two,scale,dtype", [
    (37, 64, False, 1.0, torch.float16),
    (300, 1000, True, 31.6, torch.bfloat16),
    (64, 2048, True, 1.0, torch.float32),
    (16, 8192, False, 2.0, torch.float16),
    (9, 8, True, 1.0, torch.float32),
])
def test_embedding_rows_match_oracle(vocab, dim, two, scale, dtype):
    from glq_amd import ext
    say(f"embedding vocab={vocab} dim={dim} two={two} {dtype}")
    n_pad, q1, q2, sv, ws, inv = _make(vocab, dim, vocab + dim, two)
    rng = np.random.default_rng(1)
    ids = rng.integers(0, vocab, (3, 7))
    ids[0, 0], ids[0, 1] = 0, vocab - 1
    want = O.e8_embedding_rows(ids, q1, sv.astype(np.float32), ws, q2, inv, embedding_dim=dim, embed_scale=scale)
    tab = t(O.e8_table())                                        # fp32 table, as the reference passes it
    got = ext.glq_embedding_dequant(t(ids), t(q1), t(sv), t(ws), tab, t(q2) if two else None,
                                    t(inv) if two else None, tab if two else None, n_pad, dim, scale, dtype)
    assert got.shape == (3, 7, dim) and got.dtype == dtype
    tol = {torch.float32: 1e-5, torch.float16: 1e-3, torch.bfloat16: 6e-3}[dtype]
    assert rel(got, want) < tol
    again = ext.glq_embedding_dequant(t(ids), t(q1), t(sv), t(ws), tab, t(q2) if two else None,
                                      t(inv) if two else None, tab if two else None, n_pad, dim, scale, dtype)
    assert torch.equal(got, again)


def test_embedding_module_and_op():
    from glq_amd import custom_ops
    from glq_amd.quantized_linear import E8RHTEmbedding
    custom_ops.register()
    vocab, dim = 50, 96
    n_pad, q1, q2, sv, ws, inv = _make(vocab, dim, 3, True)
    emb = E8RHTEmbedding(vocab, dim, embed_scale=float(np.sqrt(dim)))
    sd = {"Qidxs": torch.from_numpy(q1), "SV": torch.from_numpy(sv), "SU": torch.ones(1, dtype=torch.float16),
          "Wscale": torch.from_numpy(ws), "Qidxs2": torch.from_numpy(q2), "inv_resid_scale": torch.from_numpy(inv)}
    emb.load_state_dict(sd)
    emb = emb.to(DEV)
    tab = t(O.e8_table())
    emb.set_codebook(tab, tab)
    assert emb._n_stages == 2 and emb.n_pad == 128
    ids = torch.tensor([[1, 49, 0, 7]], device=DEV)
    want = O.e8_embedding_rows(ids.cpu().numpy(), q1, sv.astype(np.float32), ws, q2, inv, embedding_dim=dim,
                               embed_scale=float(np.sqrt(dim)))
    got = emb(ids)
    assert got.dtype == torch.float16 and rel(got, want) < 1e-3
    via_op = torch.ops.glq.embedding_dequant(ids, emb.Qidxs, emb.SV, emb.Wscale, tab, emb.Qidxs2,
                                             emb.inv_resid_scale, tab, 128, dim, float(np.sqrt(dim)), None)
    assert torch.equal(via_op, got)
    # a 2-bpw checkpoint (no residual keys) loads and runs single-stage
    emb1 = E8RHTEmbedding(vocab, dim)
    emb1.load_state_dict({k: v for k, v in sd.items() if k not in ("Qidxs2", "inv_resid_scale")})
    emb1 = emb1.to(DEV)
    emb1.set_codebook(tab, tab)
    assert emb1._n_stages == 1
    want1 = O.e8_embedding_rows(ids.cpu().numpy(), q1, sv.astype(np.float32), ws, embedding_dim=dim)
    assert rel(emb1(ids), want1) < 1e-3


def test_embedding_out_of_range_id_gives_zero_row_and_refusals():
    from glq_amd import ext
    n_pad, q1, q2, sv, ws, inv = _make(5, 16, 0, False)
    tab = t(O.e8_table())
    ids = torch.tensor([2, 5, -1], device=DEV)
    got = ext.glq_embedding_dequant(ids, t(q1), t(sv), t(ws), tab, n_pad=n_pad, embedding_dim=16)
    assert torch.count_nonzero(got[1:]) == 0 and torch.count_nonzero(got[0]) > 0
    with pytest.raises(RuntimeError, match="power of two"):
        ext.glq_embedding_dequant(ids, t(q1[:, :1].repeat(3, 1).reshape(5, 3)), t(np.ones(24, np.float16)), t(ws), tab)
    big = np.zeros((2, 2048), np.int16)
    with pytest.raises(RuntimeError, match="exceeds"):
        ext.glq_embedding_dequant(ids[:1], t(big), t(np.ones(16384, np.float16)), t(ws[:2]), tab)
