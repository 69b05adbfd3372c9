#!/usr/bin/env python3
"""Headline benchmark: 4 bpw trellis-3INST batch-1 decode over SmolLM3-3B linear shapes.

One "step" is the quantized-linear forward of the seven linears of one decoder layer
(q, k, v, o, gate, up, down; input RHT -> fused decode GEMV -> output RHT each) at batch
1 with bf16 activations.  The step's weights come from a pool of distinct layers that is
walked round-robin, so every launch streams its packed weights from HBM rather than from
the 256 MB Infinity Cache.  `value` is compressed-weight bytes per second over the timed
steps (inputs resident in HBM, whole steps replayed from one HIP graph).

Prints ONE JSON line on stdout; everything else goes to stderr.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--no-cpu-baseline]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = 2500.0          # dense fp16 / bf16
# (name, out_features, in_features) of one SmolLM3-3B decoder layer
LINEARS = [("q", 2048, 2048), ("k", 512, 2048), ("v", 512, 2048), ("o", 2048, 2048),
           ("gate", 11008, 2048), ("up", 11008, 2048), ("down", 2048, 11008)]
K_BITS = 4


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_pool(torch, hadamard, n_layers, dev):
    """Random code bits (every bit pattern is a valid tail-biting trellis stream), seeded
    sign vectors, Wscale = 0.02 * opt_scale, i.e. weights of rms 0.02."""
    g = torch.Generator(device=dev).manual_seed(0)
    wscale = 0.02 * 0.8933837
    shapes = {}
    for name, m, n in LINEARS:
        if (m, n) in shapes:
            continue
        bn, bm = hadamard.block_decompose(n), hadamard.block_decompose(m)
        shapes[(m, n)] = dict(
            bn=torch.tensor(bn, dtype=torch.int64), bm=torch.tensor(bm, dtype=torch.int64),
            bn_meta=hadamard.pack_block_meta(bn).to(dev), bm_meta=hadamard.pack_block_meta(bm).to(dev))
    pool = []
    for _ in range(n_layers):
        layer = []
        for name, m, n in LINEARS:
            packed = torch.randint(-32768, 32768, ((m // 16) * (n // 16), 16 * K_BITS),
                                   generator=g, device=dev, dtype=torch.int16)
            su = (torch.randint(0, 2, (m,), generator=g, device=dev) * 2 - 1).to(torch.float16)
            sv = (torch.randint(0, 2, (n,), generator=g, device=dev) * 2 - 1).to(torch.float16)
            layer.append(dict(name=name, m=m, n=n, packed=packed, su=su, sv=sv, wscale=wscale,
                              **shapes[(m, n)]))
        pool.append(layer)
    return pool


def cpu_baseline(n_calls=10):
    """The reference's CPU path for the same step (decode once and cache, then per call
    FHT -> fp32 matmul -> FHT, glq/quantized_linear.py:986-1010), restated in the oracle,
    on this host's cores.  Sample: one decoder layer (7 linears), weights decoded once
    (timed separately), then n_calls forward steps."""
    import numpy as np
    from oracle import glq_oracle as O
    rng = np.random.default_rng(0)
    layers = []
    t0 = time.perf_counter()
    for i, (name, m, n) in enumerate(LINEARS):
        packed = O.random_packed(m, n, K_BITS, seed=i)
        su, sv = O.rht_signs(m, n, 42 + i)
        W = O.decode_layer(packed, m, n, fast=True) * np.float32(0.02 * 0.8933837)
        layers.append((m, n, W, su, sv, O.block_decompose(n), O.block_decompose(m)))
    t_decode = time.perf_counter() - t0
    xs = [rng.standard_normal((1, n)).astype(np.float32) for _, _, n in LINEARS]

    def step():
        for (m, n, W, su, sv, bn, bm), x in zip(layers, xs):
            O.linear_forward_rht(x, W, su, sv, bn, bm, n, m)
    step()
    t0 = time.perf_counter()
    for _ in range(n_calls):
        step()
    dt = (time.perf_counter() - t0) / n_calls
    bytes_step = sum(m * n * K_BITS // 8 for _, m, n in LINEARS)
    return {"value": round(bytes_step / dt / 1e9, 3), "unit": "GB/s", "cores": os.cpu_count(),
            "kind": "port",
            "sample": (f"one decoder layer (7 linears, 4 bpw, batch 1): weights decoded once in "
                       f"{t_decode:.1f} s (not timed), then {n_calls} forward steps of fp32 FHT + "
                       f"cached dense matmul + FHT, {dt * 1e3:.2f} ms/step; numpy with "
                       f"multi-threaded BLAS for the matmul, single-threaded butterflies")}


def cpu_baseline_more():
    """The other CPU legs, on bounded samples (a few seconds each), each with its core count:
    E8 two-stage 4096 x 14336 at one token "cold" (the weight re-decoded by table gather on every
    call, as the reference's E8 CPU path does, glq/quantized_linear.py:1175-1195) and "warm" (decoded
    weight cached, as its trellis path does), and three tokens of the 36-layer decoder of configs[4]
    through cached transform-domain weights (four distinct decoded layers walked round-robin -- 1.25 GB
    of fp32 weights, beyond any cache -- instead of 36, which would take minutes to decode)."""
    import numpy as np
    from oracle import cpu_decoder as CD
    from oracle import glq_oracle as O
    legs = []
    cores = os.cpu_count()
    # E8 two stages, 4096 x 14336, one token
    m, n = 4096, 14336
    rng = np.random.default_rng(1)
    q1 = rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16)
    q2 = rng.integers(0, 65536, size=(m, n // 8)).astype(np.uint16).view(np.int16)
    su, sv = O.rht_signs(m, n, 42)
    art = {"Qidxs": q1, "Qidxs2": q2, "inv_resid_scale": np.float32(1 / 3.0), "SU": su.astype(np.float16),
           "SV": sv.astype(np.float16), "Wscale": np.float32(0.02), "blocks_m": O.block_decompose(m),
           "blocks_n": O.block_decompose(n)}
    x = rng.standard_normal((1, n)).astype(np.float32)
    O.e8_linear_forward(x, art, n, m)
    t0 = time.perf_counter()
    for _ in range(3):
        O.e8_linear_forward(x, art, n, m)
    cold = (time.perf_counter() - t0) / 3
    W = (O.e8_dequant(q1, q2, 1 / 3.0) * np.float32(0.02)).astype(np.float32)
    suf, svf = su.astype(np.float32), sv.astype(np.float32)
    O.linear_forward_rht(x, W, suf, svf, art["blocks_n"], art["blocks_m"], n, m)
    t0 = time.perf_counter()
    for _ in range(10):
        O.linear_forward_rht(x, W, suf, svf, art["blocks_n"], art["blocks_m"], n, m)
    warm = (time.perf_counter() - t0) / 10
    eb = m * (n // 8) * 4
    legs.append({"config": "configs[2]: E8 two-stage 4 bpw 4096x14336, one token, cold (weight decoded every call)",
                 "value": round(eb / cold / 1e9, 3), "unit": "GB/s", "ms_per_call": round(cold * 1e3, 2), "cores": cores,
                 "kind": "port", "sample": "3 calls after one warm-up"})
    legs.append({"config": "configs[2]: E8 two-stage 4 bpw 4096x14336, one token, warm (decoded weight cached)",
                 "value": round(eb / warm / 1e9, 3), "unit": "GB/s", "ms_per_call": round(warm * 1e3, 2), "cores": cores,
                 "kind": "port", "sample": "10 calls after one warm-up"})
    del W, q1, q2
    # configs[4]: the 36-layer decoder, 3 tokens
    hidden, heads, kv, hd, ffn, vocab, L = 2048, 16, 4, 128, 11008, 128256, 36
    shapes = CD.linear_shapes(hidden, heads, kv, hd, ffn)
    distinct = [CD.make_layer(shapes, K_BITS, s) for s in range(4)]
    emb = (rng.standard_normal((vocab, hidden)) * 0.02).astype(np.float32)
    dec = CD.CpuDecoder([distinct[i % 4] for i in range(L)], emb, hidden, heads, kv, hd, max_len=16)
    tok = 1
    tok = int(dec.step(tok).argmax())                          # warm-up token
    t0 = time.perf_counter()
    for _ in range(3):
        tok = int(dec.step(tok).argmax())
    per_tok = (time.perf_counter() - t0) / 3
    legs.append({"config": "configs[4]: 36-layer SmolLM3-3B-shape decoder, trellis 4 bpw, greedy batch-1 decode",
                 "value": round(1.0 / per_tok, 3), "unit": "tok/s", "ms_per_token": round(per_tok * 1e3, 1),
                 "cores": cores, "kind": "port",
                 "sample": "3 tokens after one warm-up token at context 1-4; 36 layers walking 4 distinct decoded "
                           "weight sets (1.25 GB fp32), fp32 tied output head"})
    return legs


def _graph_time(torch, fn, n_inner, reps=10):
    """us per inner call of fn(), replayed from a HIP graph between HIP events."""
    fn()
    torch.cuda.synchronize()
    st = torch.cuda.Stream()
    st.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(st):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            keep = fn()
        g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(reps):
            g.replay()
        e1.record(st)
        e1.synchronize()
    del keep
    return e0.elapsed_time(e1) * 1e3 / (reps * n_inner)


def moe_setup(torch, dev):
    """Routed experts of one mixture-of-experts layer, Qwen3-30B-A3B expert shapes (128 experts of
    2048 -> 2 x 768 -> 2048, top-8, 4 bpw, random code bits: 302 MB of streams, more than the 256 MB
    Infinity Cache).  Returns the op's weight arguments, a maker of (x, eight routing tables) for a
    token count, and the packed bytes of one expert.  Up to 95 slots every slot reads its expert's
    stream; from 96 on the rows are grouped by expert, and from 24 rows per expert on average (384 tokens)
    the sorted rows go through the tile kernel."""
    from glq_amd import hadamard as H
    E, hid, inter, K = 128, 2048, 768, 8
    gen = torch.Generator().manual_seed(0)

    def proj(m, n):
        return [torch.randint(-32768, 32768, (E, (m // 16) * (n // 16), 64), device=dev, dtype=torch.int16),
                torch.zeros(E, 1, 1, dtype=torch.int16, device=dev),
                torch.ones(E, m, dtype=torch.float16, device=dev), torch.ones(n, dtype=torch.float16, device=dev),
                torch.full((E,), 0.02, device=dev), torch.zeros(E, device=dev)]

    def meta(n):
        b = H.block_decompose(n)
        return torch.tensor(b), H.pack_block_meta(b).to(dev)
    (bn13, bn13m), (bm13, bm13m), (bn2, bn2m), (bm2, bm2m) = meta(hid), meta(2 * inter), meta(inter), meta(hid)
    args = proj(2 * inter, hid) + proj(hid, inter) + [hid, inter, 2 * inter, hid, 2 * inter, inter, hid,
                                                      bn13, bm13, bn13m, bm13m, bn2, bm2, bn2m, bm2m, 0]

    def routes_for(T):
        xb = torch.randn(T, hid, device=dev).to(torch.bfloat16)
        return xb, [(torch.stack([torch.randperm(E, generator=gen)[:K] for _ in range(T)]).to(dev),
                     torch.rand(T, K, generator=gen).to(dev)) for _ in range(8)]
    return args, routes_for, 3 * inter * hid // 2


def extras(torch, ext, dev):
    """Side measurements of the other benchmark configurations (bounded, a few seconds): whole-model
    batch-1 decode tok/s (config 5), large-layer GEMV rates where the kernels are not launch
    bound, and the prefill tiles (config 4 shape)."""
    out = {}
    roof = out["_roofline_extra"] = []

    def hbm(kernel, config, nbytes, us):
        gbs = nbytes / us / 1e3
        roof.append({"kernel": kernel, "config": config, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4), "us": round(us, 2)})

    def mfma(kernel, config, flop, us):
        tf = flop / us / 1e6
        roof.append({"kernel": kernel, "config": config, "bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS, 4), "us": round(us, 2)})
    tr_default, e8_default = ext.TRELLIS_BATCH_MAX, ext.E8_BATCH_MAX
    try:
        # what one more kernel node costs in a captured stream: 2000 dependent one-workgroup fill
        # kernels (the floor under each of the step's eight launches)
        tiny = torch.empty(1, device=dev)
        out["graph_node_floor_us"] = round(_graph_time(
            torch, lambda: [tiny.zero_() for _ in range(2000)], 2000), 2)
    except Exception as e:
        out["graph_node_floor_error"] = f"{type(e).__name__}: {e}"
    try:
        from glq_amd.decoder import TrellisDecoder
        dec = TrellisDecoder(max_len=1024)
        ids = torch.randint(0, 128256, (512,), generator=torch.Generator().manual_seed(0))
        dec.generate(ids, 8)                                  # warm-up + graph capture
        _, t_prefill, t_decode = dec.generate(ids, 256)
        out["decode_tok_s_3b_shape"] = round(256 / t_decode, 1)
        out["decode_ms_per_token"] = round(t_decode / 256 * 1e3, 3)
        out["prefill_512_ms"] = round(t_prefill * 1e3, 2)
        out["decoder"] = ("36 layers, hidden 2048, 16/4 heads x 128, FFN 11008, vocab 128256, all 7 linears "
                          "trellis 4 bpw (random bits), 512-token prompt then 256 greedy tokens, decode step "
                          "replayed from one HIP graph")
        del dec
        torch.cuda.empty_cache()
    except Exception as e:                                    # report, never hide
        out["decoder_error"] = f"{type(e).__name__}: {e}"
    try:
        m = n = 16384
        packs = [torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
                 for _ in range(4)]
        part = torch.empty(64 * m, dtype=torch.float32, device=dev)
        for B in (1, 16):
            xh = torch.randn(B, n, device=dev).to(torch.float16)
            pb = torch.empty(64 * B * m, dtype=torch.float32, device=dev)
            us = _graph_time(torch, lambda: [ext.trellis_gemv_partials(xh, p, m, n, pb) for p in packs], len(packs))
            out[f"trellis_gemv_16384x16384_B{B}_GBs"] = round(m * n / 2 / us / 1e3, 1)
            hbm("tr_mma_kernel<4> (decode launch alone, partial sums)", f"trellis 4 bpw 16384x16384, {B} token(s), "
                "4 weight sets of 134 MB in rotation", m * n // 2, us)
        del packs, part
        # 4096 x 4096, one token: the shape of the reference's own GEMV table
        # (benchmarks/_trellis_rvq_decode.md:41-52), single stage and 4+2 bits, rotating over 36
        # weight sets (302 MB of 4-bit streams, more than the 256 MB Infinity Cache)
        from glq_amd import hadamard as H
        m = n = 4096
        bn = H.block_decompose(n)
        bnt, bnm = torch.tensor(bn), H.pack_block_meta(bn).to(dev)
        sv = torch.ones(n, dtype=torch.float16, device=dev)
        p4 = [torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
              for _ in range(36)]
        p2 = [torch.randint(-32768, 32768, ((m // 16) * (n // 16), 32), device=dev, dtype=torch.int16)
              for _ in range(36)]
        xh = torch.randn(1, n, device=dev).to(torch.float16)
        pb = torch.empty(64 * m, dtype=torch.float32, device=dev)
        out["trellis_gemv_4096x4096_B1_us"] = round(_graph_time(
            torch, lambda: [ext.trellis_gemv_partials(xh, p, m, n, pb) for p in p4], len(p4)), 2)
        xb = xh.to(torch.bfloat16)
        out["trellis_linear_4096x4096_B1_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_trellis_3inst_cuda(xb, sv, sv, p, bnt, bnt, bnm, bnm, 0.02, n, m, n, m,
                                                                    out_dtype=torch.bfloat16) for p in p4], len(p4)), 2)
        out["trellis_linear_4096x4096_6bpw_B1_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_trellis_3inst_rvq2_cuda(xb, sv, sv, a, b, bnt, bnt, bnm, bnm, 0.02, 0.3,
                                                                         n, m, n, m, out_dtype=torch.bfloat16)
                            for a, b in zip(p4, p2)], len(p4)), 2)
        xb4 = torch.randn(4, n, device=dev).to(torch.bfloat16)
        out["trellis_linear_4096x4096_6bpw_B4_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_trellis_3inst_rvq2_cuda(xb4, sv, sv, a, b, bnt, bnt, bnm, bnm, 0.02, 0.3,
                                                                         n, m, n, m, out_dtype=torch.bfloat16)
                            for a, b in zip(p4, p2)], len(p4)), 2)
        # fused q/k/v of a 6 bpw 4096-wide model (4096 + 1024 + 1024 rows), one token: both streams of the three
        # layers in one decode launch, one finishing launch
        rows = (4096, 1024, 1024)
        groups = [[(sv, sv[:r], p4[3 * g + i][:(r // 16) * (n // 16)], p2[3 * g + i][:(r // 16) * (n // 16)], 0.02, 0.3, r, r)
                   for i, r in enumerate(rows)] for g in range(12)]
        out["trellis_group_qkv_4096_6bpw_B1_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_trellis_3inst_group_rvq2(xb, sh, bnt, bnm, n, n, out_dtype=torch.bfloat16)
                            for sh in groups], len(groups)), 2)
        xb8 = torch.randn(8, n, device=dev).to(torch.bfloat16)
        out["trellis_group_qkv_4096_6bpw_B8_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_trellis_3inst_group_rvq2(xb8, sh, bnt, bnm, n, n, out_dtype=torch.bfloat16)
                            for sh in groups], len(groups)), 2)
        del p4, p2, groups
        # the merged linear of the serving layer (fused q/k/v of a 2048-wide 4 bpw model) at 8 and 512 tokens: the
        # library's grouped calls, its default, against the reference's per-shard op sequence
        try:
            from glq_amd import custom_ops, linear_method as LM
            custom_ops.register()
            nq = 2048
            ml = LM.MergedTrellisLinear(nq, [2048, 512, 512], bpw=4)
            ml.trellis_packed = LM.GLQShards(torch.randint(-32768, 32768, ((r // 16) * (nq // 16), 64), dtype=torch.int16)
                                             for r in (2048, 512, 512))
            ml.Wscale = LM.GLQShards(torch.tensor(0.02) for _ in range(3))
            ml.process_weights_after_loading(dev)
            for Bm in (8, 512):
                xm = torch.randn(Bm, nq, device=dev).to(torch.bfloat16)
                for tag, grouped in (("", True), ("_reference_sequence", False)):
                    LM._GLQ_MERGED_GROUPED = grouped
                    out[f"merged_qkv_2048_4bpw_B{Bm}{tag}_us"] = round(_graph_time(
                        torch, lambda: [ml.apply(xm) for _ in range(10)], 10, reps=5), 2)
            LM._GLQ_MERGED_GROUPED = True
            del ml
        except Exception as e:
            out["merged_linear_error"] = f"{type(e).__name__}: {e}"
        m, n, M = 14336, 4096, 4096
        p = torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
        xh = torch.randn(M, n, device=dev).to(torch.float16)
        o = torch.empty(M, m, dtype=torch.float32, device=dev)
        us = _graph_time(torch, lambda: ext.glq_decode_matmul_trellis_3inst_cuda(xh, p, m, n, 1.0, out=o), 1, reps=5)
        out["trellis_prefill_14336x4096_M4096_TFLOPs"] = round(2.0 * M * m * n / us / 1e6, 1)
        mfma("tr_tile_kernel<4,4> + activation repack (matmul entry on transformed rows)",
             "configs[3]: trellis 4 bpw 14336x4096, 4096 tokens", 2.0 * M * m * n, us)
        xh = torch.randn(256, n, device=dev).to(torch.float16)
        o = torch.empty(256, m, dtype=torch.float32, device=dev)
        us = _graph_time(torch, lambda: ext.glq_decode_matmul_trellis_3inst_cuda(xh, p, m, n, 1.0, out=o), 1, reps=10)
        out["trellis_prefill_14336x4096_M256_TFLOPs"] = round(2.0 * 256 * m * n / us / 1e6, 1)
        mfma("tr_tile_pc_kernel<4,4> + activation repack + K-slot sum", "configs[3]: trellis 4 bpw 14336x4096, 256 tokens",
             2.0 * 256 * m * n, us)
        del p, xh, o
        torch.cuda.empty_cache()
    except Exception as e:
        out["large_layer_error"] = f"{type(e).__name__}: {e}"
    try:
        # config 3: E8 two-stage 4 bpw GEMV, 4096 x 14336, indices from quantizing N(0,1)
        # vectors with the GPU encoder.  GB/s = algorithmic bytes (2 bytes per 8 weights and stage) per
        # second; the kernel itself streams the folded copy of the indices, 3 bytes per index
        # (made by the load-time step ext.e8_prepare, outside the timed region; GLQ_E8_FOLD=0 for the
        # indices themselves)
        from glq_amd.checkpoint import load_shell_table
        cb = load_shell_table(None).to(dev)
        m, n = 4096, 14336
        W = torch.randn(m * (n // 8), 8, device=dev)
        d1, i1 = ext.e8_quantize(W, cb)
        _, i2 = ext.e8_quantize((W - d1) * 3.0, cb)
        del W, d1

        def to16(i):
            return (i.to(torch.int32) - ((i >= 32768).to(torch.int32) << 16)).to(torch.int16).reshape(m, n // 8)
        # 10 rotated index sets x 29.4 MB = 294 MB > the 256 MB Infinity Cache: every launch streams from HBM
        qs = [(to16(i1.roll(r * 977)).contiguous(), to16(i2.roll(r * 977)).contiguous()) for r in range(E8_SETS)]
        for a, b in qs:                                        # the load-time step: packed table, folded streams
            ext.e8_prepare(a, cb, b, cb)
        for B in (1, 16):
            xh = torch.randn(B, n, device=dev).to(torch.float16)
            us = _graph_time(torch, lambda: [ext.glq_dequant_matmul_cuda(xh, a, cb, 0.02, b, cb, 1 / 3.0)
                                             for a, b in qs], len(qs))
            out[f"e8_2stage_gemv_4096x14336_B{B}_GBs"] = round(m * (n // 8) * 4 / us / 1e3, 1)
            hbm("e8_mma_kernel<2,FOLD> (whole unfused call; algorithmic bytes = 2 B per index and stage)",
                f"configs[2]: E8 two-stage 4 bpw 4096x14336, {B} token(s), 10 index sets in rotation",
                m * (n // 8) * 4, us)
        # the same kernel where the launch's fixed costs amortise: 16384 x 16384, two stages, uniformly random
        # indices, three index sets in rotation
        try:
            mm = nn = 16384
            big = [tuple(torch.randint(-32768, 32768, (mm, nn // 8), device=dev, dtype=torch.int16) for _ in range(2))
                   for _ in range(3)]
            for a, b in big:
                ext.e8_prepare(a, cb, b, cb)
            xh = torch.randn(1, nn, device=dev).to(torch.float16)
            us = _graph_time(torch, lambda: [ext.glq_dequant_matmul_cuda(xh, a, cb, 0.02, b, cb, 1 / 3.0) for a, b in big],
                             len(big))
            out["e8_2stage_gemv_16384x16384_B1_GBs"] = round(mm * (nn // 8) * 4 / us / 1e3, 1)
            hbm("e8_mma_kernel<2,FOLD> (+ K-slot sum where the plan splits K across workgroups)",
                "E8 two-stage 4 bpw 16384x16384, 1 token, 3 index sets of 134 MB in rotation", mm * (nn // 8) * 4, us)
            for a, b in big:
                ext.e8_release(a, b)
            del big
            torch.cuda.empty_cache()
        except Exception as e:
            out["e8_large_error"] = f"{type(e).__name__}: {e}"
        # config 4, E8 half: the many-token kernel on the same quantized indices (kernel + K-slot sum),
        # also at 4096 tokens, where the library route is the default
        ext.E8_BATCH_MAX = 1 << 30
        for M in (256, 4096):
            xh = torch.randn(M, n, device=dev).to(torch.float16)
            us = _graph_time(torch, lambda: ext.glq_dequant_matmul_cuda(xh, qs[0][0], cb, 0.02, qs[0][1], cb, 1 / 3.0),
                             1, reps=5)
            out[f"e8_2stage_matmul_4096x14336_M{M}_TFLOPs"] = round(2.0 * M * m * n / us / 1e6, 1)
            mfma(("e8_tile_small_kernel<2,8,2>" if M <= 256 else "e8_tile_kernel<2,4,FOLD>") +
                 " + activation repack + K-slot sum (matmul entry on transformed rows)",
                 f"configs[3]: E8 two-stage 4 bpw 4096x14336, {M} tokens", 2.0 * M * m * n, us)
        ext.E8_BATCH_MAX = e8_default
        del qs, i1, i2
        # whole two-stage E8 linear (both transforms), 4096 x 4096, one token, rotating over 36 index sets
        # (302 MB): the E8 counterpart of trellis_linear_4096x4096_B1_us
        from glq_amd import hadamard as H
        m = n = 4096
        bn = H.block_decompose(n)
        bnt, bnm = torch.tensor(bn), H.pack_block_meta(bn).to(dev)
        sv = torch.ones(n, dtype=torch.float16, device=dev)
        cbh = cb.half()
        q4 = [(torch.randint(-32768, 32768, (m, n // 8), device=dev, dtype=torch.int16),
               torch.randint(-32768, 32768, (m, n // 8), device=dev, dtype=torch.int16)) for _ in range(36)]
        for a, b in q4:
            ext.e8_prepare(a, cbh, b, cbh)
        xb = torch.randn(1, n, device=dev).to(torch.bfloat16)
        out["e8_2stage_linear_4096x4096_B1_us"] = round(_graph_time(
            torch, lambda: [ext.glq_fused_linear_block_diag_cuda(xb, sv, sv, a, cbh, 0.02, n, m, n, m, bnt, bnt, bnm, bnm,
                                                                 b, cbh, 1 / 3.0, out_dtype=torch.bfloat16)
                            for a, b in q4], len(q4)), 2)
        del q4
        torch.cuda.empty_cache()
    except Exception as e:
        out["e8_error"] = f"{type(e).__name__}: {e}"
    try:
        # config 4: whole fused linears (both transforms included) at 14336 x 4096, trellis 4 bpw
        # and E8 two-stage 4 bpw (random code bits), in the route the library picks by itself
        from glq_amd import hadamard as H
        from glq_amd.checkpoint import load_shell_table
        cbh = load_shell_table(None).to(dev).half()
        m, n = 14336, 4096
        bn, bm = H.block_decompose(n), H.block_decompose(m)
        bnt, bmt = torch.tensor(bn), torch.tensor(bm)
        bnm, bmm = H.pack_block_meta(bn).to(dev), H.pack_block_meta(bm).to(dev)
        sv = torch.ones(n, dtype=torch.float16, device=dev)
        su = torch.ones(m, dtype=torch.float16, device=dev)
        p = torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
        q1 = torch.randint(-32768, 32768, (m, n // 8), device=dev, dtype=torch.int16)
        q2 = torch.randint(-32768, 32768, (m, n // 8), device=dev, dtype=torch.int16)
        ext.e8_prepare(q1, cbh, q2, cbh)
        e8_fold_default = ext.E8_FOLD_BATCH_MAX
        for M, route in ((256, ""), (4096, ""), (4096, "_library"), (8192, ""), (8192, "_library"),
                         (8192, "_compressed")):
            # "" = the route the library picks (compressed up to 8192 tokens for the trellis, 4096 for E8: the
            # tile kernels on the packed stream / the folded streams; dequantize + library GEMM above);
            # "_library" / "_compressed" = a route forced, for the comparison at the threshold and beyond it
            lim = {"": None, "_library": 64, "_compressed": 1 << 30}[route]
            ext.TRELLIS_BATCH_MAX = tr_default if lim is None else lim
            ext.E8_BATCH_MAX = e8_default if lim is None else lim
            ext.E8_FOLD_BATCH_MAX = e8_fold_default if lim is None else lim
            xb = torch.randn(M, n, device=dev).to(torch.bfloat16)
            us = _graph_time(torch, lambda: ext.glq_fused_linear_trellis_3inst_cuda(
                xb, sv, su, p, bnt, bmt, bnm, bmm, 0.02, n, m, n, m, out_dtype=torch.bfloat16), 1, reps=5)
            out[f"trellis_linear_14336x4096_M{M}{route}_TFLOPs"] = round(2.0 * M * m * n / us / 1e6, 1)
            us = _graph_time(torch, lambda: ext.glq_fused_linear_block_diag_cuda(
                xb, sv, su, q1, cbh, 0.02, n, m, n, m, bnt, bmt, bnm, bmm, q2, cbh, 1 / 3.0,
                out_dtype=torch.bfloat16), 1, reps=5)
            out[f"e8_2stage_linear_14336x4096_M{M}{route}_TFLOPs"] = round(2.0 * M * m * n / us / 1e6, 1)
        ext.E8_FOLD_BATCH_MAX = e8_fold_default
        ext.TRELLIS_BATCH_MAX, ext.E8_BATCH_MAX = tr_default, e8_default
        # the same two linears at 32 tokens (a batched decode step): the small-tile kernels
        xb = torch.randn(32, n, device=dev).to(torch.bfloat16)
        out["trellis_linear_14336x4096_M32_us"] = round(_graph_time(torch, lambda: ext.glq_fused_linear_trellis_3inst_cuda(
            xb, sv, su, p, bnt, bmt, bnm, bmm, 0.02, n, m, n, m, out_dtype=torch.bfloat16), 1, reps=10), 1)
        out["e8_2stage_linear_14336x4096_M32_us"] = round(_graph_time(torch, lambda: ext.glq_fused_linear_block_diag_cuda(
            xb, sv, su, q1, cbh, 0.02, n, m, n, m, bnt, bmt, bnm, bmm, q2, cbh, 1 / 3.0,
            out_dtype=torch.bfloat16), 1, reps=10), 1)
        # a stacked 6 bpw (4 + 2) layer of the same shape at 256 and 1024 tokens: both streams decoded into one
        # operand by the decoding waves of the 256-token tiles
        p2 = torch.randint(-32768, 32768, ((m // 16) * (n // 16), 32), device=dev, dtype=torch.int16)
        for M in (256, 1024):
            xb = torch.randn(M, n, device=dev).to(torch.bfloat16)
            us = _graph_time(torch, lambda: ext.glq_fused_linear_trellis_3inst_rvq2_cuda(
                xb, sv, su, p, p2, bnt, bmt, bnm, bmm, 0.02, 0.25, n, m, n, m, out_dtype=torch.bfloat16), 1, reps=5)
            out[f"trellis_linear_14336x4096_6bpw_M{M}_us"] = round(us, 1)
            out[f"trellis_linear_14336x4096_6bpw_M{M}_TFLOPs"] = round(2.0 * M * m * n / us / 1e6, 1)
        del p, p2, q1, q2
        torch.cuda.empty_cache()
    except Exception as e:
        out["prefill_linear_error"] = f"{type(e).__name__}: {e}"
    try:
        args, routes_for, per_slot_bytes = moe_setup(torch, dev)
        # 8 / 128 slots per expert stream, 1024 / 2048 grouped by expert, 8192 / 32768 through the tile kernel
        for T in (1, 16, 128, 256, 1024, 4096):
            xb, routes = routes_for(T)
            us = _graph_time(torch, lambda: [ext.glq_fused_moe_trellis_3inst_cuda(xb, i, w, *args) for i, w in routes],
                             len(routes), reps=20 if T <= 256 else 5)
            out[f"moe_experts_qwen3_30b_shape_T{T}_us"] = round(us, 2)
            if T == 1:                                        # eight expert streams read once each
                out["moe_experts_qwen3_30b_shape_T1_GBs"] = round(per_slot_bytes * 8 / us / 1e3, 1)
            if T >= 1024:                                     # two flops per weight and slot (4 bits per weight)
                out[f"moe_experts_qwen3_30b_shape_T{T}_TFLOPs"] = round(2 * per_slot_bytes * 2 * 8 * T / us / 1e6, 1)
        del args
        torch.cuda.empty_cache()
    except Exception as e:
        out["moe_error"] = f"{type(e).__name__}: {e}"
    return out


CASES = ("trellis_gemv_16384", "e8_gemv_16384", "trellis_prefill_4096", "trellis_prefill_256", "e8_gemv_2stage", "e8_prefill_4096",
         "e8_prefill_256", "e8_prefill_32", "trellis_prefill_32", "decoder", "batch1_step", "moe_experts_1", "moe_experts_16", "moe_experts_128", "moe_experts_256", "moe_experts_1024", "moe_experts_4096")
E8_SETS = 10            # rotated E8 index sets of 29.4 MB: 294 MB, more than the 256 MB Infinity Cache


def run_case(torch, ext, dev, name, steps):
    """One side measurement alone, `steps` launches back to back (eager, so that a profiler
    sees plain kernel dispatches): the command behind the per-kernel summaries in profiles/."""
    import time
    res = {"case": name, "steps": steps}
    if name == "trellis_gemv_16384":
        m = n = 16384
        packs = [torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
                 for _ in range(4)]
        xh = torch.randn(1, n, device=dev).to(torch.float16)
        pb = torch.empty(64 * m, dtype=torch.float32, device=dev)
        fn = lambda i: ext.trellis_gemv_partials(xh, packs[i % 4], m, n, pb)
        res["bytes_per_launch"] = m * n // 2
    elif name == "e8_gemv_16384":
        # the E8 counterpart of trellis_gemv_16384: two stages, uniformly random indices, three index sets of
        # 134 MB (402 MB of indices, 604 MB of folded streams) in rotation
        from glq_amd.checkpoint import load_shell_table
        cb = load_shell_table(None).to(dev)
        m = n = 16384
        qs = [tuple(torch.randint(-32768, 32768, (m, n // 8), device=dev, dtype=torch.int16) for _ in range(2))
              for _ in range(3)]
        for a, b in qs:
            ext.e8_prepare(a, cb, b, cb)
        xh = torch.randn(1, n, device=dev).to(torch.float16)
        fn = lambda i: ext.glq_dequant_matmul_cuda(xh, qs[i % 3][0], cb, 0.02, qs[i % 3][1], cb, 1 / 3.0)
        res["bytes_per_launch"] = m * (n // 8) * 4
    elif name in ("trellis_prefill_4096", "trellis_prefill_256", "trellis_prefill_32"):
        m, n, M = 14336, 4096, int(name.rsplit("_", 1)[1])
        p = torch.randint(-32768, 32768, ((m // 16) * (n // 16), 64), device=dev, dtype=torch.int16)
        xh = torch.randn(M, n, device=dev).to(torch.float16)
        o = torch.empty(M, m, dtype=torch.float32, device=dev)
        fn = lambda i: ext.glq_decode_matmul_trellis_3inst_cuda(xh, p, m, n, 1.0, out=o)
        res["flop_per_launch"] = 2.0 * M * m * n
    elif name in ("e8_gemv_2stage", "e8_prefill_4096", "e8_prefill_256", "e8_prefill_32"):
        from glq_amd.checkpoint import load_shell_table
        cb = load_shell_table(None).to(dev)
        m, n = 4096, 14336
        W = torch.randn(m * (n // 8), 8, device=dev)
        d1, i1 = ext.e8_quantize(W, cb)
        _, i2 = ext.e8_quantize((W - d1) * 3.0, cb)
        del W, d1

        def to16(i):
            return (i.to(torch.int32) - ((i >= 32768).to(torch.int32) << 16)).to(torch.int16).reshape(m, n // 8)
        qs = [(to16(i1.roll(r * 977)).contiguous(), to16(i2.roll(r * 977)).contiguous()) for r in range(E8_SETS)]
        for a, b in qs:                                        # the load-time step: packed table, folded streams
            ext.e8_prepare(a, cb, b, cb)
        M = 1 if name == "e8_gemv_2stage" else int(name.rsplit("_", 1)[1])
        xh = torch.randn(M, n, device=dev).to(torch.float16)
        fn = lambda i: ext.glq_dequant_matmul_cuda(xh, qs[i % E8_SETS][0], cb, 0.02, qs[i % E8_SETS][1], cb, 1 / 3.0)
        res["bytes_per_launch"] = m * (n // 8) * 4
        res["flop_per_launch"] = 2.0 * M * m * n
    elif name == "batch1_step":
        # the step of the headline measurement, eager: the four grouped calls of one decoder layer
        # (decode launch + output-transform launch each), rotating over four weight sets
        from glq_amd import hadamard
        pool = build_pool(torch, hadamard, 4, dev)
        xs = {n: torch.randn(1, n, generator=torch.Generator(device=dev).manual_seed(1), device=dev)
              .to(torch.bfloat16) for _, _, n in LINEARS}

        def fn(i):
            by = {lin["name"]: lin for lin in pool[i % 4]}
            for names in (("q", "k", "v"), ("o",), ("gate", "up"), ("down",)):
                lins = [by[nm] for nm in names]
                a = lins[0]
                ext.glq_fused_linear_trellis_3inst_group(
                    xs[a["n"]], [(l["sv"], l["su"], l["packed"], l["wscale"], l["m"], l["m"]) for l in lins],
                    a["bn"], a["bn_meta"], a["n"], a["n"], out_dtype=torch.bfloat16)
        res["bytes_per_launch"] = sum(m * n * K_BITS // 8 for _, m, n in LINEARS)
    elif name.startswith("moe_experts_"):
        T = int(name.rsplit("_", 1)[1])
        args, routes_for, per_slot_bytes = moe_setup(torch, dev)
        xb, routes = routes_for(T)
        fn = lambda i: ext.glq_fused_moe_trellis_3inst_cuda(xb, *routes[i % 8], *args)
        res["slots"] = T * 8
        res["bytes_per_slot"] = per_slot_bytes
    elif name == "decoder":
        from glq_amd.decoder import TrellisDecoder
        dec = TrellisDecoder(max_len=1024)
        ids = torch.randint(0, 128256, (512,), generator=torch.Generator().manual_seed(0))
        dec.generate(ids, 4)
        _, _, t_decode = dec.generate(ids, steps)
        res["decode_tok_s"] = round(steps / t_decode, 1)
        print(json.dumps(res), flush=True)
        return
    else:
        raise SystemExit(f"unknown case {name}; one of {CASES}")
    for i in range(8):
        fn(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(i)
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) * 1e6 / steps
    res["us_per_launch_eager"] = round(us, 2)
    print(json.dumps(res), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=720)
    ap.add_argument("--warmup", type=int, default=72)
    ap.add_argument("--layers", type=int, default=36, help="distinct weight sets in the pool")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--ungrouped", action="store_true", help="seven separate fused linears per step")
    ap.add_argument("--no-extras", action="store_true", help="skip the decoder / large-layer side measurements")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch a plain 256 MiB read + 256 MiB write elementwise kernel three times "
                         "(calibration of the FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc)")
    ap.add_argument("--case", choices=CASES, default=None,
                    help="run one side measurement alone (for profiling) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1).")
        sys.exit(2)

    import torch
    from glq_amd import _lib, ext, hadamard
    _lib.load()                                       # fails loudly if the HIP library is absent
    if not torch.cuda.is_available():
        log("bench.py needs a GPU: the HIP path has no CPU fallback.")
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if args.case:
        run_case(torch, ext, dev, args.case, max(1, args.steps if args.steps != 720 else 40))
        return
    L = max(1, args.layers)
    pool = build_pool(torch, hadamard, L, dev)
    xs = {n: torch.randn(1, n, generator=torch.Generator(device=dev).manual_seed(1), device=dev)
          .to(torch.bfloat16) for _, _, n in LINEARS}
    bytes_step = sum(m * n * K_BITS // 8 for _, m, n in LINEARS)
    log(f"pool: {L} layers x {bytes_step / 1e6:.2f} MB packed = {L * bytes_step / 1e9:.2f} GB")

    def one(lin):
        return ext.glq_fused_linear_trellis_3inst_cuda(
            xs[lin["n"]], lin["sv"], lin["su"], lin["packed"], lin["bn"], lin["bm"],
            lin["bn_meta"], lin["bm_meta"], lin["wscale"], lin["n"], lin["m"], lin["n"],
            lin["m"], out_dtype=torch.bfloat16)

    GROUPS = (("q", "k", "v"), ("o",), ("gate", "up"), ("down",))

    def run_step(layer, decode_only=False):
        """q/k/v and gate/up read the same activations and go out as one grouped call each,
        as a merged linear does (glq_vllm/linear_method.py:664-710); o and down are groups of
        one.  Every call is one decode launch plus one output-transform launch."""
        by = {lin["name"]: lin for lin in layer}
        if args.ungrouped and not decode_only:
            return [one(lin) for lin in layer]
        outs = []
        for names in GROUPS:
            lins = [by[nm] for nm in names]
            a = lins[0]
            outs.append(ext.glq_fused_linear_trellis_3inst_group(
                xs[a["n"]], [(l["sv"], l["su"], l["packed"], l["wscale"], l["m"], l["m"]) for l in lins],
                a["bn"], a["bn_meta"], a["n"], a["n"], out_dtype=torch.bfloat16, decode_only=decode_only))
        return outs

    # eager warm-up (also initialises the library outside of graph capture)
    for i in range(min(L, 4)):
        run_step(pool[i])
    torch.cuda.synchronize()

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        def capture(n_steps):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=stream):
                keep = [run_step(pool[i % L]) for i in range(n_steps)]
            return g, keep
        full, keep_full = capture(L)
        K, W = args.steps, args.warmup
        rem_graphs = {}

        def replay_steps(n):
            q, r = divmod(n, L)
            for _ in range(q):
                full.replay()
            if r:
                if r not in rem_graphs:
                    rem_graphs[r] = capture(r)
                rem_graphs[r][0].replay()
        # capture any remainder graph before timing
        for n in (W, K):
            if n % L and (n % L) not in rem_graphs:
                rem_graphs[n % L] = capture(n % L)
        replay_steps(W)
        torch.cuda.synchronize()
        # exactly K steps between two HIP events on the replay stream (device time: a host clock
        # around a millisecond of work mostly measures the submission), host clock kept beside it
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        ev0.record(stream)
        replay_steps(K)
        ev1.record(stream)
        torch.cuda.synchronize()
        dt_host = time.perf_counter() - t0
        dt = ev0.elapsed_time(ev1) * 1e-3
        # distribution: the whole pool (L steps) replayed 200 times, one event pair per replay
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(200)]
        for a, b in evs:
            a.record(stream)
            full.replay()
            b.record(stream)
        torch.cuda.synchronize()
        per_step = sorted(a.elapsed_time(b) * 1e3 / L for a, b in evs)
    ms_per_step = dt / K * 1e3
    value = bytes_step / (dt / K) / 1e9
    stats = {"us_per_step_median": round(per_step[len(per_step) // 2], 2),
             "us_per_step_p10": round(per_step[len(per_step) // 10], 2),
             "us_per_step_p90": round(per_step[(len(per_step) * 9) // 10], 2),
             "replays": len(per_step), "steps_per_replay": L,
             "us_per_step_host_clock": round(dt_host / K * 1e6, 2),
             "method": "HIP events on the replay stream; value is from the K timed steps, the "
                       "distribution from 200 further replays of the whole weight pool"}
    log(f"timed {K} steps: {ms_per_step * 1e3:.1f} us/step (host clock {dt_host / K * 1e6:.1f}), "
        f"{value:.1f} GB/s packed weights; median {stats['us_per_step_median']} us "
        f"(p10 {stats['us_per_step_p10']}, p90 {stats['us_per_step_p90']})")

    # ---- roofline leg: the decode launches alone, HIP events on their own stream ---------
    # The same grouped calls as the timed steps, stopped after the decode kernel (input
    # transform + packed-stream GEMV into split-K partials), over the whole pool.
    with torch.cuda.stream(stream):
        run_step(pool[0], decode_only=True)
        torch.cuda.synchronize()
        gk = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gk, stream=stream):
            for layer in pool:
                run_step(layer, decode_only=True)
        gk.replay()
        torch.cuda.synchronize()
        reps = 10
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            gk.replay()
        e1.record(stream)
        e1.synchronize()
        n_launch = reps * L * len(GROUPS)
        avg_us = e0.elapsed_time(e1) * 1e3 / n_launch
    bytes_launch = bytes_step / len(GROUPS)
    achieved = bytes_launch / (avg_us * 1e-6) / 1e9
    # HBM bytes per launch from the committed counter summary (FETCH_SIZE / WRITE_SIZE runs)
    traffic = None
    traffic_source = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic_tr_mma_fusein_kernels_smollm3_4bpw_batch1.txt")
    if os.path.exists(tpath):
        import re
        mt = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)", open(tpath).read(), re.M)
        traffic = int(mt.group(1)) if mt else None
        if traffic is not None:
            traffic_source = ("not measured by this run: FETCH_SIZE + WRITE_SIZE of two rocprofv3 --pmc runs of this "
                              "command, recorded in profiles/" + os.path.basename(tpath))
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                "kernel": ("tr_mma_fusein_kernel<4,bf16,1> (o, down) and tr_mma_fusein_group_kernel<4,bf16,1> "
                           "(q/k/v, gate/up): the fused-input decode launch, averaged over the four "
                           "groups of a step"),
                "avg_launch_us": round(avg_us, 3),
                "bytes_per_launch": int(bytes_launch),
                "method": (f"{n_launch} back-to-back decode launches (the 4 grouped calls of a step: q/k/v, o, "
                           f"gate/up, down; x {L} distinct weight sets), stopped before the output "
                           f"transform, replayed from a HIP graph between two HIP events on the launch "
                           f"stream; bytes = packed weights of the step / 4 launches")}
    log(f"decode launches alone: {avg_us:.2f} us/launch avg, {achieved:.0f} GB/s "
        f"({100 * achieved / HBM_PEAK_GBS:.1f}% of HBM peak)")

    if args.copy_probe:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 1.0, out=dst)                      # 268435456 B read, 268435456 B written
        torch.cuda.synchronize()
        del src, dst

    extra, roofline_extra = {}, []
    if not args.no_extras:
        extra = extras(torch, ext, dev)
        roofline_extra = extra.pop("_roofline_extra", [])

    result = {
        "metric": "4bpw GEMV effective HBM GB/s (% of peak); batch-1 decode tok/s, 3B shape",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16",
        "data": "synthetic (random code bits, seeded signs, N(0,1) bf16 activations)",
        "config": {"workload": "configs[1]: trellis-3INST 4 bpw linear set, SmolLM3-3B shapes "
                               "(q/o 2048x2048, k/v 2048x512, gate/up 2048x11008, down 11008x2048), "
                               "batch-1 fused linear (input RHT + GEMV + output RHT) per layer; q/k/v and "
                               "gate/up issued as grouped calls (2 launches per group)",
                   "step": "7 linears of one decoder layer", "packed_bytes_per_step": bytes_step,
                   "distinct_layers": L, "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
                   "linear_only_tok_s_36_layers": round(1e3 / (ms_per_step * 36), 1)},
        "roofline": roofline,
        "roofline_extra": roofline_extra,
        "timing": stats,
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        log("timing the CPU baseline (oracle port of the reference CPU path) ...")
        result["cpu_baseline"] = cpu_baseline()
        try:
            result["cpu_baseline"]["more"] = cpu_baseline_more()
        except Exception as e:                                # report, never hide
            result["cpu_baseline"]["more_error"] = f"{type(e).__name__}: {e}"
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
