"""The SmolLM3-shaped decoder around the quantized linears: cache consistency and graph
replay on a small configuration (needs an MI355X)."""
import pytest
import torch

from tests.gpu_util import DEV, rel, say

pytestmark = pytest.mark.gpu


def _small():
    from glq_amd.decoder import DecoderConfig, TrellisDecoder
    cfg = DecoderConfig(hidden=256, layers=3, heads=2, kv_heads=1, head_dim=128, ffn=512, vocab=1000,
                        no_rope_interval=2, bits=4)
    return TrellisDecoder(cfg, device=DEV, seed=3, max_len=64)


def test_decode_step_matches_prefill_of_longer_prompt():
    say("decoder cache")
    dec = _small()
    ids = torch.randint(0, 1000, (20,), generator=torch.Generator().manual_seed(0)).to(DEV)
    full = dec.prefill(ids)                                   # logits after 20 tokens
    dec.prefill(ids[:19])
    dec.tok.copy_(ids[19:20])
    step = dec._step()                                        # 19 cached + 1 decoded
    assert rel(step, full.cpu().numpy()) < 3e-2
    assert int(dec.pos.item()) == 20


def test_graph_replay_equals_eager_decode():
    say("decoder graph")
    dec = _small()
    ids = torch.randint(0, 1000, (12,), generator=torch.Generator().manual_seed(1)).to(DEV)
    eager, _, _ = dec.generate(ids, 10, use_graph=False)
    graph, _, _ = dec.generate(ids, 10, use_graph=True)
    again, _, _ = dec.generate(ids, 10, use_graph=True)
    assert torch.equal(eager, graph) and torch.equal(graph, again)


def test_glue_ops_match_torch():
    """RMSNorm, rotary + cache append, single-query GQA attention and the SiLU gate against
    plain PyTorch fp32 references."""
    import torch.nn.functional as F
    from glq_amd import _lib, decoder as D
    say("decoder glue ops")
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=DEV).manual_seed(0)
    T, H, heads, kvh, hd, L = 5, 2048, 16, 4, 128, 96
    x = torch.randn(T, H, generator=g, device=DEV).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(H, generator=g, device=DEV)).to(torch.bfloat16)
    assert rel(D._rms_norm(x, w, 1e-6), D._rms_norm_torch(x, w, 1e-6).float().cpu().numpy()) < 4e-3

    q = torch.randn(T, heads, hd, generator=g, device=DEV).to(torch.bfloat16)
    k = torch.randn(T, kvh, hd, generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn(T, kvh, hd, generator=g, device=DEV).to(torch.bfloat16)
    pos = torch.tensor([7, 3, 11, 0, 90], device=DEV)
    inv = 1.0 / (2e6 ** (torch.arange(0, hd, 2, device=DEV, dtype=torch.float32) / hd))
    ang = torch.arange(L, device=DEV, dtype=torch.float32)[:, None] * inv[None]
    ang = torch.cat((ang, ang), -1)
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
    kc = torch.zeros(kvh, L, hd, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    qo = torch.empty_like(q)
    _lib.check(lib.glqh_rope_kv_store_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), pos.data_ptr(),
                                           cos.data_ptr(), sin.data_ptr(), qo.data_ptr(), kc.data_ptr(),
                                           vc.data_ptr(), T, heads, kvh, hd, L, 1, st))
    c, s = cos.float()[pos], sin.float()[pos]
    def rope(t):
        tf = t.float()
        rot = torch.cat((-tf[..., hd // 2:], tf[..., :hd // 2]), -1)
        return tf * c[:, None] + rot * s[:, None]
    assert rel(qo, rope(q).cpu().numpy()) < 4e-3
    assert rel(kc[:, pos].transpose(0, 1), rope(k).cpu().numpy()) < 4e-3
    assert torch.equal(vc[:, pos].transpose(0, 1), v)

    kc = torch.randn(kvh, L, hd, generator=g, device=DEV).to(torch.bfloat16)
    vc = torch.randn(kvh, L, hd, generator=g, device=DEV).to(torch.bfloat16)
    q1 = torch.randn(heads, hd, generator=g, device=DEV).to(torch.bfloat16)
    p1 = torch.tensor([40], device=DEV)
    out = torch.empty(heads, hd, dtype=torch.bfloat16, device=DEV)
    _lib.check(lib.glqh_attn_decode_bf16(q1.data_ptr(), kc.data_ptr(), vc.data_ptr(), p1.data_ptr(),
                                         out.data_ptr(), heads, kvh, hd, L, st))
    ref = F.scaled_dot_product_attention(q1.float()[None, :, None], kc.float()[None, :, :41],
                                         vc.float()[None, :, :41], enable_gqa=True)[0, :, 0]
    assert rel(out, ref.cpu().numpy()) < 5e-3

    d = torch.randn(T, H, generator=g, device=DEV).to(torch.bfloat16)
    xo, ho = D._add_rms_norm(x, d, w, 1e-6)
    assert torch.equal(xo, x + d)
    assert rel(ho, D._rms_norm_torch(x + d, w, 1e-6).float().cpu().numpy()) < 4e-3

    a = torch.randn(3, 11008, generator=g, device=DEV).to(torch.bfloat16)
    b = torch.randn(3, 11008, generator=g, device=DEV).to(torch.bfloat16)
    o = torch.empty_like(a)
    _lib.check(lib.glqh_silu_mul_bf16(a.data_ptr(), b.data_ptr(), o.data_ptr(), a.numel(), st))
    assert rel(o, (F.silu(a.float()) * b.float()).cpu().numpy()) < 4e-3


@pytest.mark.parametrize("hidden,ffn", [(2048, 11008), (256, 512), (2560, 768)])
def test_fused_output_epilogues_match_separate_launches(hidden, ffn):
    """o/down + residual add + RMSNorm and gate/up + SiLU gate finished inside the launch that
    transforms the linear's output, against the separate launches (same kernels before the
    output transform).  The gate is bit-identical; the norm path transforms whole blocks
    where the separate launch uses 1024-point slices, so it agrees to bf16 rounding."""
    from glq_amd import decoder as D
    say("fused epilogues", hidden, ffn)
    g = torch.Generator(device=DEV).manual_seed(hidden)
    down = D._Linear(hidden, ffn, 4, g, DEV)
    gate, up = D._Linear(ffn, hidden, 4, g, DEV), D._Linear(ffn, hidden, 4, g, DEV)
    a = torch.randn(1, ffn, generator=g, device=DEV).to(torch.bfloat16)
    x = torch.randn(1, hidden, generator=g, device=DEV).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(hidden, generator=g, device=DEV)).to(torch.bfloat16)
    x_ref, h_ref = D._add_rms_norm(x, down(a), w, 1e-6)
    x_out, h = D._linear_add_rms_norm(down, a, x, w, 1e-6)
    assert rel(x_out, x_ref.float().cpu().numpy()) < 4e-3 and rel(h, h_ref.float().cpu().numpy()) < 6e-3
    x2, h2 = D._linear_add_rms_norm(down, a, x, w, 1e-6)
    assert torch.equal(x_out, x2) and torch.equal(h, h2)

    hin = torch.randn(1, hidden, generator=g, device=DEV).to(torch.bfloat16)
    gu = D._group(hin, (gate, up))
    act_ref = torch.empty(1, ffn, dtype=torch.bfloat16, device=DEV)
    D.check(D._lib.load().glqh_silu_mul_bf16(gu[:, :ffn].data_ptr(), gu[:, ffn:].data_ptr(), act_ref.data_ptr(),
                                             ffn, D._stream()))
    act = D._gate_up_silu(gate, up, hin)
    assert torch.equal(act, act_ref)


def test_decoder_with_and_without_fused_epilogues():
    say("decoder fused vs separate")
    from glq_amd.decoder import DecoderConfig, TrellisDecoder
    cfg = DecoderConfig(hidden=256, layers=3, heads=2, kv_heads=1, head_dim=128, ffn=512, vocab=1000,
                        no_rope_interval=2, bits=4)
    ids = torch.randint(0, 1000, (12,), generator=torch.Generator().manual_seed(1)).to(DEV)
    outs = []
    for fuse in (True, False):
        dec = TrellisDecoder(cfg, device=DEV, seed=3, max_len=64, fuse_epilogues=fuse)
        dec.prefill(ids)
        outs.append(dec._step().float())
    assert rel(outs[0], outs[1].cpu().numpy()) < 2e-2


@pytest.mark.parametrize("rope", [1, 0])
def test_fused_qkv_rope_store_is_bit_identical(rope):
    from glq_amd import decoder as D
    say("fused qkv rope", rope)
    g = torch.Generator(device=DEV).manual_seed(5)
    hidden, heads, kvh, hd, L = 2048, 16, 4, 128, 64
    q, k, v = (D._Linear(heads * hd, hidden, 4, g, DEV), D._Linear(kvh * hd, hidden, 4, g, DEV),
               D._Linear(kvh * hd, hidden, 4, g, DEV))
    h = torch.randn(1, hidden, generator=g, device=DEV).to(torch.bfloat16)
    pos = torch.tensor([37], device=DEV)
    inv = 1.0 / (2e6 ** (torch.arange(0, hd, 2, device=DEV, dtype=torch.float32) / hd))
    ang = torch.arange(L, device=DEV, dtype=torch.float32)[:, None] * inv[None]
    ang = torch.cat((ang, ang), -1)
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
    lib = D._lib.load()
    qkv = D._group(h, (q, k, v))
    nq, nk = q.m, k.m
    qr0 = torch.zeros(1, nq, dtype=torch.bfloat16, device=DEV)
    kc0 = torch.zeros(kvh, L, hd, dtype=torch.bfloat16, device=DEV)
    vc0 = torch.zeros_like(kc0)
    D.check(lib.glqh_rope_kv_store_bf16(qkv[:, :nq].data_ptr(), qkv[:, nq:nq + nk].data_ptr(), qkv[:, nq + nk:].data_ptr(),
                                        pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), qr0.data_ptr(), kc0.data_ptr(),
                                        vc0.data_ptr(), 1, heads, kvh, hd, L, rope, D._stream()))
    qr1, kc1, vc1 = torch.zeros_like(qr0), torch.zeros_like(kc0), torch.zeros_like(vc0)
    D._qkv_rope_store(q, k, v, h, pos, cos, sin, qr1, kc1, vc1, hd, L, rope)
    assert torch.count_nonzero(qr0) > 0 and torch.count_nonzero(kc0[:, 37]) > 0
    assert torch.equal(qr0, qr1) and torch.equal(kc0, kc1) and torch.equal(vc0, vc1)
    # and with the attention in the same launch: earlier cache rows are random, row 37 is new
    kc0[:, :37] = torch.randn(kvh, 37, hd, generator=g, device=DEV).to(torch.bfloat16)
    vc0[:, :37] = torch.randn(kvh, 37, hd, generator=g, device=DEV).to(torch.bfloat16)
    a0 = torch.zeros(1, nq, dtype=torch.bfloat16, device=DEV)
    D.check(lib.glqh_attn_decode_bf16(qr0.data_ptr(), kc0.data_ptr(), vc0.data_ptr(), pos.data_ptr(), a0.data_ptr(),
                                      heads, kvh, hd, L, D._stream()))
    kc2, vc2 = kc0.clone(), vc0.clone()
    kc2[:, 37] = 0
    vc2[:, 37] = 0
    a2 = torch.zeros_like(a0)
    D._qkv_rope_attn(q, k, v, h, pos, cos, sin, kc2, vc2, a2, heads, kvh, hd, L, rope)
    assert torch.count_nonzero(a0) > 0
    assert torch.equal(a0, a2) and torch.equal(kc0, kc2) and torch.equal(vc0, vc2)
    pos0 = torch.tensor([0], device=DEV)                        # first position: only the new row
    kc3, vc3, a3 = torch.zeros_like(kc0), torch.zeros_like(vc0), torch.zeros_like(a0)
    D._qkv_rope_attn(q, k, v, h, pos0, cos, sin, kc3, vc3, a3, heads, kvh, hd, L, rope)
    assert torch.equal(a3.view(heads, hd), vc3[:, 0].repeat_interleave(heads // kvh, 0))


@pytest.mark.parametrize("L,positions", [(4096, (0, 700, 1023, 1024, 1535, 1536, 2600, 4095)), (1536, (1023, 1400, 1535)),
                                         (20000, (19999,))])
def test_attention_with_shared_keys(L, positions):
    """From 1024 cached positions on, up to eight workgroups per head take a share of the keys and the last one to
    finish merges them: against the one-workgroup entry (same bits below 1024 positions, rounding above), against
    softmax(q K^T) V in fp64 from the cache the launch left, the state buffer back to zero, two calls the same bits.
    A cache of 20000 positions only fits the score buffer with shares."""
    from glq_amd import decoder as D
    say("shared-key attention", L, positions)
    g = torch.Generator(device=DEV).manual_seed(11)
    hidden, heads, kvh, hd = 2048, 16, 4, 128
    q, k, v = (D._Linear(heads * hd, hidden, 4, g, DEV), D._Linear(kvh * hd, hidden, 4, g, DEV),
               D._Linear(kvh * hd, hidden, 4, g, DEV))
    h = torch.randn(1, hidden, generator=g, device=DEV).to(torch.bfloat16)
    inv = 1.0 / (2e6 ** (torch.arange(0, hd, 2, device=DEV, dtype=torch.float32) / hd))
    ang = torch.arange(L, device=DEV, dtype=torch.float32)[:, None] * inv[None]
    ang = torch.cat((ang, ang), -1)
    cos, sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
    kc0 = (torch.randn(kvh, L, hd, generator=g, device=DEV) * 2.0).to(torch.bfloat16)
    vc0 = torch.randn(kvh, L, hd, generator=g, device=DEV).to(torch.bfloat16)
    state = D.attn_state(heads, L, DEV)
    assert state is not None and int(state.count_nonzero()) == 0
    for p in positions:
        pos = torch.tensor([p], device=DEV)
        kc1, vc1, a1 = kc0.clone(), vc0.clone(), torch.zeros(1, heads * hd, dtype=torch.bfloat16, device=DEV)
        D._qkv_rope_attn(q, k, v, h, pos, cos, sin, kc1, vc1, a1, heads, kvh, hd, L, 1, state)
        torch.cuda.synchronize()
        assert int(state[:1024].count_nonzero()) == 0, p          # the counters are back at zero
        kc2, vc2, a2 = kc0.clone(), vc0.clone(), torch.zeros_like(a1)
        D._qkv_rope_attn(q, k, v, h, pos, cos, sin, kc2, vc2, a2, heads, kvh, hd, L, 1, state)
        assert torch.equal(a1, a2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2), p
        n = p + 1
        if L <= 8192:                                             # the one-workgroup entry holds max_len scores in LDS
            kc3, vc3, a3 = kc0.clone(), vc0.clone(), torch.zeros_like(a1)
            D._qkv_rope_attn(q, k, v, h, pos, cos, sin, kc3, vc3, a3, heads, kvh, hd, L, 1, None)
            assert torch.equal(kc1, kc3) and torch.equal(vc1, vc3), p
            if n < 1024:
                assert torch.equal(a1, a3), p
            else:
                assert rel(a1, a3.float().cpu().numpy()) < 6e-3, (p, rel(a1, a3.float().cpu().numpy()))
        # reference from the cache rows the launch wrote and the query it used: q is not returned, so take it
        # from the store-only entry
        qr = torch.zeros(1, heads * hd, dtype=torch.bfloat16, device=DEV)
        kc4, vc4 = kc0.clone(), vc0.clone()
        D._qkv_rope_store(q, k, v, h, pos, cos, sin, qr, kc4, vc4, hd, L, 1)
        assert torch.equal(kc4, kc1) and torch.equal(vc4, vc1), p
        qd = qr.view(heads, hd).double()
        Kd = kc1[:, :n].double().repeat_interleave(heads // kvh, 0)
        Vd = vc1[:, :n].double().repeat_interleave(heads // kvh, 0)
        sc = torch.einsum("hd,hnd->hn", qd, Kd) / (hd ** 0.5)
        ref = torch.einsum("hn,hnd->hd", torch.softmax(sc, -1), Vd).reshape(1, -1)
        e = rel(a1, ref.cpu().numpy())
        assert e < 6e-3, (p, e)


@pytest.mark.parametrize("hidden,vocab", [(2048, 128256), (4096, 1000), (2048, 7)])
def test_output_head_and_argmax(hidden, vocab):
    """Logits of the library's output head against a float64 product, its arg-max against the
    arg-max of its own logits, ties to the lowest row; with and without the logits buffer."""
    from glq_amd import _lib
    from glq_amd._lib import check
    say("lm head", hidden, vocab)
    lib = _lib.load()
    g = torch.Generator().manual_seed(vocab)
    E = (torch.randn(vocab, hidden, generator=g) * 0.02).to(torch.bfloat16)
    h = torch.randn(1, hidden, generator=g).to(torch.bfloat16)
    E[vocab - 1] = E[3]                                        # an exact tie between rows 3 and vocab-1
    h = (E[3:4].float() * 40).to(torch.bfloat16) if vocab <= 1000 else h   # make that pair the maximum
    Ed, hd = E.to(DEV), h.to(DEV)
    logits = torch.empty(1, vocab, dtype=torch.float32, device=DEV)
    tok = torch.full((1,), -1, dtype=torch.int64, device=DEV)
    ws = torch.empty(int(lib.glqh_lm_head_workspace_bytes()), dtype=torch.uint8, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    check(lib.glqh_lm_head_argmax_bf16(hd.data_ptr(), Ed.data_ptr(), vocab, hidden, logits.data_ptr(),
                                       tok.data_ptr(), ws.data_ptr(), ws.numel(), st))
    ref = (h.double() @ E.double().t()).numpy()
    assert rel(logits, ref) < 1e-5, rel(logits, ref)
    lg = logits[0].cpu()
    top = int(tok.item())
    assert lg[top] == lg.max() and top == int((lg == lg.max()).nonzero()[0])
    if vocab <= 1000:
        assert top == 3 and lg[3] == lg[vocab - 1]
    tok2 = torch.full((1,), -1, dtype=torch.int64, device=DEV)
    check(lib.glqh_lm_head_argmax_bf16(hd.data_ptr(), Ed.data_ptr(), vocab, hidden, None, tok2.data_ptr(),
                                       ws.data_ptr(), ws.numel(), st))
    assert int(tok2.item()) == top
    with pytest.raises(RuntimeError, match="hidden size"):
        check(lib.glqh_lm_head_argmax_bf16(hd.data_ptr(), Ed.data_ptr(), vocab, 1024, None, tok2.data_ptr(),
                                           ws.data_ptr(), ws.numel(), st))


def test_positions_outside_the_cache_are_skipped_not_written():
    """Device-side positions are compared with max_len inside the kernels: a position outside
    [0, max_len) writes no cache row and no output row (the kernels return before any access
    that depends on it), and generate() refuses a run that would pass the end of the cache."""
    from glq_amd import _lib
    say("decoder position guard")
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device=DEV).manual_seed(4)
    T, heads, kvh, hd, L = 3, 4, 2, 128, 16
    q = torch.randn(T, heads, hd, generator=g, device=DEV).to(torch.bfloat16)
    k = torch.randn(T, kvh, hd, generator=g, device=DEV).to(torch.bfloat16)
    v = torch.randn(T, kvh, hd, generator=g, device=DEV).to(torch.bfloat16)
    cos = torch.ones(L, hd, dtype=torch.bfloat16, device=DEV)
    sin = torch.zeros(L, hd, dtype=torch.bfloat16, device=DEV)
    kc = torch.full((kvh, L, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    vc = torch.full((kvh, L, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    qo = torch.full((T, heads, hd), 5.0, dtype=torch.bfloat16, device=DEV)
    pos = torch.tensor([L, 2, -1], device=DEV)                 # first and last token out of range
    _lib.check(lib.glqh_rope_kv_store_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), pos.data_ptr(),
                                           cos.data_ptr(), sin.data_ptr(), qo.data_ptr(), kc.data_ptr(),
                                           vc.data_ptr(), T, heads, kvh, hd, L, 1, st))
    assert torch.equal(qo[1], q[1]) and torch.all(qo[0] == 5.0) and torch.all(qo[2] == 5.0)
    assert torch.equal(kc[:, 2], k[1]) and torch.equal(vc[:, 2], v[1])
    keep = [i for i in range(L) if i != 2]
    assert torch.all(kc[:, keep] == 7.0) and torch.all(vc[:, keep] == 7.0)
    out = torch.full((heads, hd), 3.0, dtype=torch.bfloat16, device=DEV)
    for bad in (L, L + 5, -1):
        p1 = torch.tensor([bad], device=DEV)
        _lib.check(lib.glqh_attn_decode_bf16(q[0].contiguous().data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                             p1.data_ptr(), out.data_ptr(), heads, kvh, hd, L, st))
        assert torch.all(out == 3.0)
    # the fused finishing launches: a decode step at pos == max_len leaves the caches untouched
    dec = _small()
    ids = torch.randint(0, 1000, (10,), generator=torch.Generator().manual_seed(2)).to(DEV)
    dec.prefill(ids)
    dec.pos.fill_(dec.max_len)
    kc0, vc0 = dec.kc.clone(), dec.vc.clone()
    dec._step()
    torch.cuda.synchronize()
    assert torch.equal(dec.kc, kc0) and torch.equal(dec.vc, vc0)
    with pytest.raises(RuntimeError, match="exceed max_len"):
        dec.generate(ids, dec.max_len, use_graph=False)
