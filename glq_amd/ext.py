"""The reference's native-extension surface, served by libglq_hip.so.

Every function here has the name and positional signature of the matching pybind
function of the reference extension (``glq._C`` / JIT ``glq_cuda``,
glq/csrc/glq_bindings.cpp:334-550), so this module can stand where
``glq.inference_kernel._glq_cuda`` stands; call sites probe capabilities with
``hasattr(ext, "<name>")`` exactly as they do there.  Tensors are checked, outputs
and scratch are allocated with torch (caching allocator, graph-capture friendly) and
raw pointers go to the C ABI on the current stream.  Nothing is computed in Python.

Two deliberate extensions beyond the reference: activations may be bf16 as well as
fp16 (the reference casts to fp16 first), and the fused linears accept ``out_dtype``
so the result can be written in the caller's dtype without a cast kernel.
"""
from __future__ import annotations

import ctypes as C
import os
import warnings
import weakref

import torch

from . import _lib
from ._lib import GLQH_BF16, GLQH_F16, GLQH_F32, check

_DT = {torch.float16: GLQH_F16, torch.bfloat16: GLQH_BF16, torch.float32: GLQH_F32}

# Small and medium token counts are served on the compressed weights: 1-16 tokens by the GEMV /
# small-batch kernels, above by the tile kernels that decode each weight once per 128-row x
# 512-token tile (csrc/trellis_tile.hip, csrc/e8_tile.hip).  Beyond a few thousand tokens the
# reference's own many-token route -- dequantize the weight to fp16 once with the HIP kernel, then
# one library GEMM (glq/csrc/glq_trellis.cu:1265-1268, 1322-1334) -- is a few per cent faster on this
# chip, at the price of a transient fp16 copy of the weight.  Whole fused linear, compressed / library,
# us, on 14336 x 4096 and 4096 x 14336: trellis 175 / 206 and 160 / 205 at 1024 tokens, 340 / 335 and
# 267 / 300 at 2048, 565 / 545 and 481 / 487 at 4096, 1034 / 980 and 976 / 895 at 8192; E8 two-stage on
# the indices 201 / 211 and 196 / 209 at 1024, 400 / 335 and 312 / 327 at 2048, 639 / 552 and 553 / 511 at
# 4096 (the 14336-row shape pays for 448 and 896 tiles on 256 CUs).  The thresholds are the reference's
# tunable and its E8 counterpart: GLQ_TRELLIS_BATCH_MAX=<n> / GLQ_E8_BATCH_MAX=<n> send calls above n
# tokens to the library route (a large n keeps every call compressed).  Trellis, after the tile kernel's
# staged output and grouped launches: 562 / 611 and 472 / 480 at 4096 tokens, 1129 / 1089 and 994 / 981 at 8192,
# 2147 / 2061 and 2004 / 1872 at 16384; 4096 x 4096 306 / 312 at 8192, 641 / 610 at 16384; 11008 x 2048 520 / 562
# and 1058 / 1105: level at 8192 tokens, so trellis calls stay compressed up to there.
TRELLIS_BATCH_MAX = max(1, int(os.environ.get("GLQ_TRELLIS_BATCH_MAX", "8192")))
# Stacked (two-stage) layers decode two streams per tile of at most 256 tokens, and the library route adds
# the second stage once: compressed / library, us, 4 + 2 bits, 14336 x 4096 and 4096 x 14336: 119 / 223 and
# 109 / 243 at 512 tokens, 216 / 280 and 192 / 290 at 1024, 419 / 404 and 365 / 409 at 2048, 811 / 682 and
# 766 / 597 at 4096, 1581 / 1191 and 1528 / 1051 at 8192 (4096 x 4096: 126 / 140 at 2048, 229 / 203 at 4096).
# They take the library route above the smaller of the two limits.
TRELLIS_STACKED_BATCH_MAX = max(1, int(os.environ.get("GLQ_TRELLIS_BATCH_MAX", "2048")))
# GLQ_TRELLIS_DENSE (set to anything) sends every fused trellis call to that dense route, the
# reference's A/B switch of the same name (glq/csrc/glq_trellis.cu:1023-1029, 1269).
TRELLIS_DENSE = "GLQ_TRELLIS_DENSE" in os.environ
E8_BATCH_MAX = max(1, int(os.environ.get("GLQ_E8_BATCH_MAX", "1024")))
# On the folded streams (see E8_FOLD below) the E8 tile kernel looks nothing up outside LDS and expands
# nothing, and the compressed route wins or ties up to 4096 tokens (whole two-stage linear, compressed /
# library, us: 268 / 322 and 300 / 321 at 2048 tokens on 4096 x 14336 and 14336 x 4096, 519 / 516 and
# 585 / 595 at 4096, 1087 / 984 and 1146 / 1047 at 8192).  The larger of the two limits applies there.
E8_FOLD_BATCH_MAX = max(1, int(os.environ.get("GLQ_E8_BATCH_MAX", "4096")))


def _e8_dense_route(B, n_pad, folded=False):
    """Dequantize + library GEMM: on request, and above 16 tokens for the widths the tile kernel does
    not take (n_pad must be a multiple of 32 on folded streams, of 256 on the indices themselves)."""
    limit = max(E8_BATCH_MAX, E8_FOLD_BATCH_MAX) if folded else E8_BATCH_MAX
    return B > limit or (B > 16 and int(n_pad) % (32 if folded else 256) != 0)


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _chk(t, name, dtype=None, dev=True):
    if dev and not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")


def _ws(nbytes, device):
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


def _host_i64(t):
    """CPU int64 block list -> (ctypes array, count)."""
    if t is None:
        return None, 0
    vals = [int(v) for v in (t.tolist() if isinstance(t, torch.Tensor) else t)]
    return (C.c_int64 * len(vals))(*vals), len(vals)


def _meta_ptr(meta):
    if meta is None or (isinstance(meta, torch.Tensor) and meta.numel() == 0):
        return C.c_void_p(0)
    _chk(meta, "block meta", torch.int32)
    return _p(meta)

def _skey(t):
    return (t.data_ptr(), t._version, tuple(t.shape), t.dtype, str(t.device))


class _DerivedCache:
    """Device data derived once from a source tensor (a packed table, a folded index stream, block
    sizes read back to the host).  An entry is keyed by the source's bytes -- address, version
    counter, shape, dtype, device -- and guarded by a weak reference to its storage: a fresh view
    of the same memory hits, a new tensor at a reused address does not, an in-place write misses,
    and the entry goes when the storage is freed."""

    def __init__(self):
        self._d = {}

    def get(self, t, extra=()):
        hit = self._d.get(_skey(t) + extra)
        if hit is not None and hit[0]() is t.untyped_storage():
            return hit[1]
        return None

    def put(self, t, value, extra=()):
        key = _skey(t) + extra
        store = t.untyped_storage()
        d = self._d
        for k in [k for k, v in d.items() if v[0]() is None or (v[0]() is store and k[0] == key[0] and k[1] != key[1]
                                                                and k[2:] == key[2:])]:
            del d[k]                                           # dead sources, older versions of this one

        def drop(ref, key=key):
            if d.get(key, (None,))[0] is ref:
                del d[key]
        d[key] = (weakref.ref(store, drop), value)
        return value

    def values(self):
        return [v[1] for v in self._d.values() if v[0]() is not None]

    def __len__(self):
        return len(self._d)

    def holds(self, t):
        """True when some entry was derived from `t`'s bytes (any version, any table)."""
        return any(k[0] == t.data_ptr() and v[0]() is t.untyped_storage() for k, v in self._d.items())


# --------------------------------------------------------------------------- trellis
def glq_trellis_kernel_supported(m, k):
    return bool(_lib.load().glqh_trellis_kernel_supported(int(m), int(k)))


def glq_decompress_trellis_3inst_cuda(trellis_packed, m, k, allow_r1=False):
    lib = _lib.load()
    _chk(trellis_packed, "trellis_packed", torch.int16)
    if trellis_packed.dim() != 2:
        raise RuntimeError("trellis_packed must be 2-D [(m/16)*(k/16), 16*R]")
    out = torch.empty((int(m), int(k)), dtype=torch.float16, device=trellis_packed.device)
    with torch.cuda.device(trellis_packed.device):
        check(lib.glqh_decompress_trellis_3inst(_p(trellis_packed), trellis_packed.shape[0],
                                                trellis_packed.shape[1], int(m), int(k),
                                                int(bool(allow_r1)), _p(out), _stream()))
    return out


def _trellis_matmul(x2d, trellis_packed, m, k, wscale, out, accum):
    lib = _lib.load()
    _chk(x2d, "x", torch.float16)
    _chk(trellis_packed, "trellis_packed", torch.int16)
    if trellis_packed.dim() != 2:
        raise RuntimeError("trellis_packed must be 2-D [(m/16)*(k/16), 16*R]")
    B = x2d.shape[0]
    if accum and out is None:
        raise RuntimeError("accumulate mode needs the caller's `out` (stage 1 is the initializer)")
    if out is None:
        out = torch.empty((B, int(m)), dtype=torch.float32, device=x2d.device)
    else:
        if not (out.is_contiguous() and out.numel() == B * int(m) and out.dtype == torch.float32):
            raise RuntimeError("out must be a contiguous fp32 tensor of B*m elements")
    with torch.cuda.device(x2d.device):
        nb = lib.glqh_trellis_gemv_workspace_bytes(int(m), int(k), B)
        ws = _ws(nb, x2d.device)
        check(lib.glqh_decode_matmul_trellis_3inst(
            _p(x2d), B, _p(trellis_packed), trellis_packed.shape[0], trellis_packed.shape[1],
            int(m), int(k), float(wscale), _p(out), int(m), int(bool(accum)),
            _p(ws), ws.numel(), _stream()))
    return out


def glq_decode_matvec_trellis_3inst_cuda(x, trellis_packed, m, k, wscale=1.0, out=None, accum=False):
    if x.numel() != int(k):
        raise RuntimeError(f"x must have k elements, got {x.numel()}")
    y = _trellis_matmul(x.reshape(1, -1), trellis_packed, m, k, wscale,
                        None if out is None else out, accum)
    return y.reshape(int(m)) if out is None else out


def glq_decode_matmul_trellis_3inst_cuda(x, trellis_packed, m, k, wscale=1.0, out=None, accum=False):
    if x.dim() != 2 or x.shape[1] != int(k):
        raise RuntimeError(f"x must be (B, k), got {tuple(x.shape)}")
    return _trellis_matmul(x, trellis_packed, m, k, wscale, out, accum)


def trellis_gemv_partials(x2d, trellis_packed, m, k, part):
    """Decode kernel alone: raw split-K partial sums into `part` (fp32, caller-owned);
    returns the number of K slots written.  Not part of the reference surface."""
    lib = _lib.load()
    _chk(x2d, "x", torch.float16)
    _chk(trellis_packed, "trellis_packed", torch.int16)
    _chk(part, "part", torch.float32)
    ks = C.c_int(0)
    with torch.cuda.device(x2d.device):
        check(lib.glqh_trellis_gemv_partials(
            _p(x2d), x2d.shape[0], _p(trellis_packed), trellis_packed.shape[0],
            trellis_packed.shape[1], int(m), int(k), _p(part), part.numel() * 4, C.byref(ks),
            _stream()))
    return ks.value


# --------------------------------------------------------------------------- RHT
def glq_input_rht_cuda(x, sv, out, in_features, stride_x, rsqrt_n, n_pad, log_n):
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(sv, "sv", torch.float16)
    _chk(out, "out", (torch.float32, torch.float16))
    B = x.shape[0] if x.dim() == 2 else 1
    if (1 << int(log_n)) != int(n_pad):
        raise RuntimeError(f"n_pad={n_pad} is not 2**log_n")
    with torch.cuda.device(x.device):
        check(lib.glqh_input_rht(_p(x), _DT[x.dtype], int(stride_x), _p(sv), _p(out), _DT[out.dtype],
                                 B, int(in_features), int(n_pad), None, None, 1, float(rsqrt_n),
                                 _stream()))


def glq_output_rht_cuda(y_rht, su, out, out_features, m_pad, log_m, rsqrt_m):
    lib = _lib.load()
    _chk(y_rht, "y_rht", torch.float32)
    _chk(su, "su", torch.float16)
    _chk(out, "out", (torch.float16, torch.bfloat16, torch.float32))
    B = y_rht.shape[0] if y_rht.dim() == 2 else 1
    if (1 << int(log_m)) != int(m_pad):
        raise RuntimeError(f"m_pad={m_pad} is not 2**log_m")
    with torch.cuda.device(y_rht.device):
        check(lib.glqh_output_rht(_p(y_rht), int(m_pad), _p(su), _p(out), _DT[out.dtype],
                                  int(out_features), B, int(out_features), int(m_pad), None, None, 1,
                                  float(rsqrt_m), _stream()))


def glq_input_rht_blockdiag_cuda(x, sv, x_rht, in_features, n_pad, blocks_n, blocks_n_meta):
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(sv, "sv", torch.float16)
    _chk(x_rht, "x_rht", (torch.float32, torch.float16))
    arr, nb = _host_i64(blocks_n)
    B = x.shape[0]
    with torch.cuda.device(x.device):
        check(lib.glqh_input_rht(_p(x), _DT[x.dtype], x.shape[1], _p(sv), _p(x_rht), _DT[x_rht.dtype],
                                 B, int(in_features), int(n_pad), _meta_ptr(blocks_n_meta) if nb > 1 else None,
                                 arr, nb, 0.0, _stream()))


def glq_output_rht_blockdiag_cuda(y_rht, su, y, out_features, m_pad, blocks_m, blocks_m_meta):
    lib = _lib.load()
    _chk(y_rht, "y_rht", torch.float32)
    _chk(su, "su", torch.float16)
    _chk(y, "y", (torch.float16, torch.bfloat16, torch.float32))
    arr, nb = _host_i64(blocks_m)
    B = y_rht.shape[0]
    with torch.cuda.device(y_rht.device):
        check(lib.glqh_output_rht(_p(y_rht), int(m_pad), _p(su), _p(y), _DT[y.dtype], y.shape[1], B,
                                  int(out_features), int(m_pad),
                                  _meta_ptr(blocks_m_meta) if nb > 1 else None, arr, nb, 0.0, _stream()))


def _dense_matmul_output(x_rht, W, wscale, su, y, out_features, m_pad, blocks_m, blocks_m_meta):
    """Tail of the many-token route: one library GEMM with fp32 output, then the output
    transform with Wscale applied on the way in (no separate pass over y_rht)."""
    lib = _lib.load()
    y_rht = torch.mm(x_rht, W.t(), out_dtype=torch.float32)
    arr, nb = _host_i64(blocks_m)
    with torch.cuda.device(y_rht.device):
        check(lib.glqh_output_rht_scaled(_p(y_rht), float(wscale), _p(su), _p(y), _DT[y.dtype], y.shape[1],
                                         y_rht.shape[0], int(out_features), int(m_pad),
                                         _meta_ptr(blocks_m_meta) if nb > 1 else None, arr, nb, _stream()))
    return y


def glq_output_rht_shards_cuda(y_rht, su, y, out_features, shard_meta, max_bs):
    lib = _lib.load()
    _chk(y_rht, "y_rht", torch.float32)
    _chk(su, "su", torch.float16)
    _chk(y, "y", (torch.float16, torch.bfloat16, torch.float32))
    _chk(shard_meta, "shard_meta", torch.int32)
    B, total_m = y_rht.shape
    if int(out_features) != total_m or y.shape[1] != int(out_features):
        raise RuntimeError("output_rht_shards needs out_features == total_m == y.shape[1]")
    with torch.cuda.device(y_rht.device):
        check(lib.glqh_output_rht_shards(_p(y_rht), _p(su), _p(y), _DT[y.dtype], B, int(out_features),
                                         total_m, _p(shard_meta), shard_meta.shape[0], int(max_bs),
                                         _stream()))


# --------------------------------------------------------------------------- fused trellis
def _fused_trellis(x, sv, su, packed, packed2, blocks_n, blocks_m, bn_meta, bm_meta, wscale,
                   inv_rs2, in_features, out_features, n_pad, m_pad, y, y_rht_out, out_dtype):
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(sv, "sv", torch.float16)
    _chk(packed, "trellis_packed", torch.int16)
    if packed.dim() != 2:
        raise RuntimeError("trellis_packed must be 2-D [(m/16)*(k/16), 16*R]")
    has2 = packed2 is not None and packed2.numel() > 0
    if has2:
        _chk(packed2, "trellis_packed2", torch.int16)
    B = x.shape[0]
    bn, nbn = _host_i64(blocks_n)
    bm, nbm = _host_i64(blocks_m)
    if y is None and y_rht_out is None:
        _chk(su, "su", torch.float16)
        y = torch.empty((B, int(out_features)), dtype=out_dtype or torch.float16, device=x.device)
    ystride = 0
    yrp, yrs = C.c_void_p(0), 0
    if y_rht_out is not None:
        yrp, yrs = y_rht_out
    batch_max = min(TRELLIS_BATCH_MAX, TRELLIS_STACKED_BATCH_MAX) if has2 else TRELLIS_BATCH_MAX
    if (TRELLIS_DENSE or B > batch_max) and y_rht_out is None:
        if (packed2 is not None and packed2.numel() > 0) != (float(inv_rs2) != 0.0):
            raise RuntimeError("trellis RVQ stage 2 is half-configured: trellis_packed2 is "
                               f"{'present' if has2 else 'absent'} but inv_resid_scale2 = {inv_rs2}")
        return _trellis_dense(x, sv, su, packed, packed2 if has2 else None, blocks_n, blocks_m,
                              bn_meta, bm_meta, wscale, inv_rs2, in_features, out_features, n_pad,
                              m_pad, y)
    with torch.cuda.device(x.device):
        nb = lib.glqh_fused_linear_trellis_workspace_bytes(B, int(n_pad), int(m_pad))
        ws = _ws(nb, x.device)
        check(lib.glqh_fused_linear_trellis_3inst(
            _p(x), _DT[x.dtype], x.shape[1], B, _p(sv), _p(su) if su is not None else None,
            _p(packed), packed.shape[0], packed.shape[1],
            _p(packed2) if has2 else None, packed2.shape[0] if has2 else 0,
            packed2.shape[1] if has2 else 0,
            bn, nbn, bm, nbm, _meta_ptr(bn_meta) if nbn > 1 else None,
            _meta_ptr(bm_meta) if nbm > 1 else None,
            float(wscale), float(inv_rs2), int(in_features), int(out_features), int(n_pad), int(m_pad),
            _p(y) if y is not None else None, _DT[y.dtype] if y is not None else GLQH_F16,
            y.shape[1] if y is not None else ystride, yrp, int(yrs), _p(ws), ws.numel(), _stream()))
    return y


def _trellis_dense(x, sv, su, packed, packed2, blocks_n, blocks_m, bn_meta, bm_meta, wscale,
                   inv_rs2, in_features, out_features, n_pad, m_pad, y):
    """Many tokens: input RHT (fp16) -> fp16 weight from the decompress kernel -> one GEMM
    with fp32 accumulation -> x wscale -> output RHT."""
    B = x.shape[0]
    x_rht = torch.empty((B, int(n_pad)), dtype=torch.float16, device=x.device)
    glq_input_rht_blockdiag_cuda(x, sv, x_rht, in_features, n_pad, blocks_n, bn_meta)
    W = glq_decompress_trellis_3inst_cuda(packed, m_pad, n_pad)
    if packed2 is not None:
        W.add_(glq_decompress_trellis_3inst_cuda(packed2, m_pad, n_pad, allow_r1=True),
               alpha=float(inv_rs2))
    return _dense_matmul_output(x_rht, W, wscale, su, y, out_features, m_pad, blocks_m, bm_meta)


def glq_fused_linear_trellis_3inst_cuda(x, sv, su, trellis_packed, blocks_n, blocks_m,
                                        blocks_n_meta, blocks_m_meta, wscale, in_features,
                                        out_features, n_pad, m_pad, out_dtype=None):
    return _fused_trellis(x, sv, su, trellis_packed, None, blocks_n, blocks_m, blocks_n_meta,
                          blocks_m_meta, wscale, 0.0, in_features, out_features, n_pad, m_pad,
                          None, None, out_dtype)


def glq_fused_linear_trellis_3inst_rvq2_cuda(x, sv, su, trellis_packed, trellis_packed2, blocks_n,
                                             blocks_m, blocks_n_meta, blocks_m_meta, wscale,
                                             inv_resid_scale2, in_features, out_features, n_pad,
                                             m_pad, out_dtype=None):
    if trellis_packed2 is None or trellis_packed2.numel() == 0:
        raise RuntimeError("trellis RVQ stage 2 is half-configured: trellis_packed2 is absent "
                           f"but inv_resid_scale2 = {inv_resid_scale2}")
    return _fused_trellis(x, sv, su, trellis_packed, trellis_packed2, blocks_n, blocks_m,
                          blocks_n_meta, blocks_m_meta, wscale, inv_resid_scale2, in_features,
                          out_features, n_pad, m_pad, None, None, out_dtype)


class _TrellisShard(C.Structure):
    _fields_ = [("sv_f16", C.c_void_p), ("su_f16", C.c_void_p), ("packed", C.c_void_p),
                ("packed_rows", C.c_int64), ("packed_cols", C.c_int64), ("wscale", C.c_double),
                ("out_features", C.c_int64), ("m_pad", C.c_int64), ("y", C.c_void_p)]


def glq_fused_linear_trellis_3inst_group(x, shards, blocks_n, blocks_n_meta, in_features, n_pad,
                                         out_dtype=None, decode_only=False, separate=False):
    """Several separately quantized trellis layers on the same x (fused q/k/v, gate/up) with
    one decode launch and one output-transform launch: the per-shard loop of the reference's
    vLLM linear method (glq_vllm/linear_method.py:664-710) as a single call.

    shards: sequence of (sv, su, trellis_packed, wscale, out_features, m_pad).  Returns one
    (B, sum(out_features)) tensor, shard s in columns [off_s, off_s + out_features_s).
    Up to four layers.  1..4 tokens: one decode launch; 5..64: one decode launch per layer (the small-batch
    kernel to 16 tokens, the small-tile kernel above) between one transform launch per sign vector and one
    finishing launch; more than 64: one launch of the many-token kernel over the row tiles of all of them.
    Single-stage layers of one rate and block_decompose block sizes; raises RuntimeError otherwise (callers then use the per-layer op).
    decode_only=True stops after the decode launch (no output transform, returns None): a measurement
    hook.  separate=True (more than 64 tokens): a list of contiguous (B, out_features_s) tensors instead."""
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    B = x.shape[0]
    dt = out_dtype or torch.float16
    total_out = sum(int(s[4]) for s in shards)
    total_m = sum(int(s[5]) for s in shards)
    y = None if decode_only else torch.empty((B, total_out), dtype=dt, device=x.device)
    if separate and y is not None:
        if B <= 64:
            raise RuntimeError("separate outputs need more than 64 tokens")
        y = y.view(-1)                                           # layer s: rows packed at element B * off_s
    arr = (_TrellisShard * len(shards))()
    off = 0
    esz = torch.empty((), dtype=dt).element_size() * (B if separate else 1)
    for i, (sv, su, packed, wscale, out_f, m_pad) in enumerate(shards):
        _chk(sv, "sv", torch.float16)
        _chk(su, "su", torch.float16)
        _chk(packed, "trellis_packed", torch.int16)
        if packed.dim() != 2:
            raise RuntimeError("trellis_packed must be 2-D [(m/16)*(k/16), 16*R]")
        arr[i] = _TrellisShard(_p(sv), _p(su), _p(packed), packed.shape[0], packed.shape[1], float(wscale),
                               int(out_f), int(m_pad), None if y is None else y.data_ptr() + off * esz)
        off += int(out_f)
    bn, nbn = _host_i64(blocks_n)
    with torch.cuda.device(x.device):
        nb = lib.glqh_fused_linear_trellis_group_workspace_bytes(B, int(n_pad), total_m, len(shards))
        ws = _ws(max(nb, 256), x.device)
        check(lib.glqh_fused_linear_trellis_3inst_group(
            _p(x), _DT[x.dtype], x.shape[1], B, C.addressof(arr), len(shards), bn, nbn,
            _meta_ptr(blocks_n_meta) if nbn > 1 else None, int(in_features), int(n_pad), _DT[dt],
            0 if separate else total_out, _p(ws), ws.numel(), _stream()))
    if separate and y is not None:
        outs, off = [], 0
        for s in shards:
            outs.append(y[B * off:B * (off + int(s[4]))].view(B, int(s[4])))
            off += int(s[4])
        return outs
    return y


class _TrellisStage2(C.Structure):
    _fields_ = [("packed2", C.c_void_p), ("packed2_rows", C.c_int64), ("packed2_cols", C.c_int64),
                ("inv_resid_scale2", C.c_double)]


def glq_fused_linear_trellis_3inst_group_rvq2(x, shards, blocks_n, blocks_n_meta, in_features, n_pad,
                                              out_dtype=None):
    """The grouped call for stacked (two-stage) layers at 1..64 tokens: the decode step of fused q/k/v or
    gate/up of a 5-8 bpw checkpoint, whose per-shard loop in the reference is
    fused_linear_trellis_3inst_yrht_rvq2 per shard + output_rht_shards (glq_vllm/linear_method.py:664-710).
    One token: one decode launch for both streams of every shard; 2..64: one transform launch per distinct
    sign vector and one decode launch per shard (the small-batch kernel to 16 tokens, the small-tile kernel
    above); one finishing launch either way.

    shards: sequence of (sv, su, trellis_packed, trellis_packed2, wscale, inv_resid_scale2, out_features,
    m_pad); first stages of 4 bpw, second stages of one common rate.  Returns (B, sum(out_features)).
    Raises RuntimeError for other token counts or rates (callers then use the per-layer op)."""
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    B = x.shape[0]
    dt = out_dtype or torch.float16
    total_out = sum(int(s[6]) for s in shards)
    total_m = sum(int(s[7]) for s in shards)
    y = torch.empty((B, total_out), dtype=dt, device=x.device)
    arr = (_TrellisShard * len(shards))()
    arr2 = (_TrellisStage2 * len(shards))()
    off = 0
    esz = torch.empty((), dtype=dt).element_size()
    for i, (sv, su, packed, packed2, wscale, inv2, out_f, m_pad) in enumerate(shards):
        _chk(sv, "sv", torch.float16)
        _chk(su, "su", torch.float16)
        _chk(packed, "trellis_packed", torch.int16)
        _chk(packed2, "trellis_packed2", torch.int16)
        if packed.dim() != 2 or packed2.dim() != 2:
            raise RuntimeError("trellis_packed / trellis_packed2 must be 2-D [(m/16)*(k/16), 16*R]")
        arr[i] = _TrellisShard(_p(sv), _p(su), _p(packed), packed.shape[0], packed.shape[1], float(wscale),
                               int(out_f), int(m_pad), y.data_ptr() + off * esz)
        arr2[i] = _TrellisStage2(_p(packed2), packed2.shape[0], packed2.shape[1], float(inv2))
        off += int(out_f)
    bn, nbn = _host_i64(blocks_n)
    with torch.cuda.device(x.device):
        nb = lib.glqh_fused_linear_trellis_group_workspace_bytes(B, int(n_pad), total_m, len(shards))
        ws = _ws(max(nb, 256), x.device)
        check(lib.glqh_fused_linear_trellis_3inst_group_rvq2(
            _p(x), _DT[x.dtype], x.shape[1], B, C.addressof(arr), C.addressof(arr2), len(shards), bn, nbn,
            _meta_ptr(blocks_n_meta) if nbn > 1 else None, int(in_features), int(n_pad), _DT[dt], total_out,
            _p(ws), ws.numel(), _stream()))
    return y


class _MoeProj(C.Structure):
    _fields_ = [("packed", C.c_void_p), ("packed_rows", C.c_int64), ("packed_cols", C.c_int64),
                ("packed2", C.c_void_p), ("packed2_cols", C.c_int64), ("su", C.c_void_p), ("sv", C.c_void_p),
                ("wscale", C.c_void_p), ("inv_rs2", C.c_void_p), ("blocks_n", C.c_void_p),
                ("n_blocks_n", C.c_int64), ("bn_meta", C.c_void_p), ("blocks_m", C.c_void_p),
                ("n_blocks_m", C.c_int64), ("in_features", C.c_int64), ("out_features", C.c_int64),
                ("n_pad", C.c_int64), ("m_pad", C.c_int64)]


def _moe_proj(what, packed, packed2, su, sv, wscale, inv_rs2, blocks_n, blocks_m, bn_meta, in_f, out_f, n_pad,
              m_pad, keep):
    _chk(packed, f"{what}_trellis_packed", torch.int16)
    if packed.dim() != 3:
        raise RuntimeError(f"{what}_trellis_packed must be (E, tiles, 16*R)")
    E = packed.shape[0]
    _chk(su, f"{what}_SU", torch.float16)
    _chk(sv, f"{what}_SV", torch.float16)
    if su.shape != (E, int(m_pad)) or sv.numel() != int(n_pad):
        raise RuntimeError(f"{what}: SU must be (E, m_pad) and SV (n_pad,), got {tuple(su.shape)} and {tuple(sv.shape)}")
    ws32 = wscale.to(device=packed.device, dtype=torch.float32).contiguous()
    if ws32.numel() != E:
        raise RuntimeError(f"{what}_Wscale must hold one scale per expert")
    keep.append(ws32)
    # a second stage registered as the (E, 1, 1) placeholder is "absent" (glq/csrc/glq_cuda.cu:5083-5088)
    has2 = packed2 is not None and packed2.numel() > E
    p2 = irs = None
    if has2:
        _chk(packed2, f"{what}_trellis_packed2", torch.int16)
        if packed2.dim() != 3 or packed2.shape[0] != E or packed2.shape[1] != packed.shape[1]:
            raise RuntimeError(f"trellis MoE {what} stage-2 tile count {tuple(packed2.shape)} != stage-1 "
                               f"{tuple(packed.shape)}")
        p2 = packed2
        irs = inv_rs2.to(device=packed.device, dtype=torch.float32).contiguous()
        if irs.numel() != E:
            raise RuntimeError(f"{what}_inv_resid_scale2 must hold one value per expert")
        keep.append(irs)
    bn, nbn = _host_i64(blocks_n)
    bm, nbm = _host_i64(blocks_m)
    keep += [bn, bm]
    return _MoeProj(_p(packed).value, packed.shape[1], packed.shape[2], _p(p2).value if has2 else None,
                    p2.shape[2] if has2 else 0, _p(su).value, _p(sv).value, _p(ws32).value,
                    _p(irs).value if has2 else None, C.cast(bn, C.c_void_p).value, nbn,
                    _meta_ptr(bn_meta).value if nbn > 1 else None, C.cast(bm, C.c_void_p).value, nbm,
                    int(in_f), int(out_f), int(n_pad), int(m_pad))


def glq_fused_moe_trellis_3inst_cuda(x, topk_ids, topk_weights,
                                     w13_trellis_packed, w13_trellis_packed2, w13_SU, w13_SV, w13_Wscale,
                                     w13_inv_resid_scale2,
                                     w2_trellis_packed, w2_trellis_packed2, w2_SU, w2_SV, w2_Wscale,
                                     w2_inv_resid_scale2,
                                     hidden_size, intermediate_size, w13_out_features,
                                     n_pad_w13, m_pad_w13, n_pad_w2, m_pad_w2,
                                     blocks_n_w13, blocks_m_w13, blocks_n_w13_meta, blocks_m_w13_meta,
                                     blocks_n_w2, blocks_m_w2, blocks_n_w2_meta, blocks_m_w2_meta,
                                     activation_type, out_dtype=None):
    """The routed-expert step of a mixture-of-experts layer on stacked trellis-3INST experts, one
    host call with the routing read on the device (argument order of the reference's binding,
    glq/csrc/glq_bindings.cpp:509-525; glq/csrc/glq_cuda.cu:5030-5250).  Returns (num_tokens,
    hidden) in the input's 16-bit dtype (the reference returns fp16)."""
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    if x.dim() != 2 or x.shape[1] != int(hidden_size):
        raise RuntimeError(f"x must be (num_tokens, hidden), got {tuple(x.shape)}")
    if topk_ids.dim() != 2 or topk_ids.shape != topk_weights.shape or topk_ids.shape[0] != x.shape[0]:
        raise RuntimeError("topk_ids and topk_weights must be (num_tokens, top_k)")
    if int(activation_type) not in (0, 1, 2):
        raise RuntimeError(f"trellis MoE path supports gated activations (0/1/2) only, got {activation_type}")
    T, K = topk_ids.shape
    if T == 0 or K == 0:                                      # an empty batch (or no choices): nothing to launch
        return torch.zeros((T, int(hidden_size)), dtype=out_dtype or x.dtype, device=x.device)
    ids = topk_ids.to(device=x.device, dtype=torch.int64).contiguous()
    tw = topk_weights.to(device=x.device, dtype=torch.float32).contiguous()
    keep = []
    w13 = _moe_proj("w13", w13_trellis_packed, w13_trellis_packed2, w13_SU, w13_SV, w13_Wscale,
                    w13_inv_resid_scale2, blocks_n_w13, blocks_m_w13, blocks_n_w13_meta, hidden_size,
                    w13_out_features, n_pad_w13, m_pad_w13, keep)
    w2 = _moe_proj("w2", w2_trellis_packed, w2_trellis_packed2, w2_SU, w2_SV, w2_Wscale, w2_inv_resid_scale2,
                   blocks_n_w2, blocks_m_w2, blocks_n_w2_meta, intermediate_size, hidden_size, n_pad_w2,
                   m_pad_w2, keep)
    dt = out_dtype or x.dtype
    out = torch.empty((T, int(hidden_size)), dtype=dt, device=x.device)
    with torch.cuda.device(x.device):
        nb = lib.glqh_fused_moe_trellis_workspace_bytes(T, K, w13_trellis_packed.shape[0], C.addressof(w13),
                                                        C.addressof(w2))
        if nb == 0:
            # the entry itself reports what is wrong with the shapes
            nb = 256
        ws = _ws(nb, x.device)
        check(lib.glqh_fused_moe_trellis_3inst(
            _p(x), _DT[x.dtype], x.shape[1], T, _p(ids), _p(tw), K, w13_trellis_packed.shape[0],
            C.addressof(w13), C.addressof(w2), int(intermediate_size), int(activation_type), _p(out), _DT[dt],
            out.shape[1], _p(ws), ws.numel(), _stream()))
    return out


def _yrht_slice(y_rht_out, col, m_pad):
    _chk(y_rht_out, "y_rht_out", torch.float32)
    if y_rht_out.dim() != 2 or int(col) < 0 or int(col) + int(m_pad) > y_rht_out.shape[1]:
        raise RuntimeError("y_rht_out must be (B, total_m) with col + m_pad <= total_m")
    return C.c_void_p(y_rht_out.data_ptr() + 4 * int(col)), y_rht_out.shape[1]


def glq_fused_linear_trellis_3inst_yrht_cuda(x, sv, trellis_packed, blocks_n, blocks_n_meta, wscale,
                                             in_features, n_pad, m_pad, y_rht_out, col):
    if y_rht_out.shape[0] != x.shape[0]:
        raise RuntimeError("y_rht_out rows must equal the token count")
    _fused_trellis(x, sv, None, trellis_packed, None, blocks_n, None, blocks_n_meta, None, wscale,
                   0.0, in_features, m_pad, n_pad, m_pad, None, _yrht_slice(y_rht_out, col, m_pad),
                   None)


def glq_fused_linear_trellis_3inst_yrht_rvq2_cuda(x, sv, trellis_packed, trellis_packed2, blocks_n,
                                                  blocks_n_meta, wscale, inv_resid_scale2,
                                                  in_features, n_pad, m_pad, y_rht_out, col):
    if y_rht_out.shape[0] != x.shape[0]:
        raise RuntimeError("y_rht_out rows must equal the token count")
    if trellis_packed2 is None or trellis_packed2.numel() == 0:
        raise RuntimeError("trellis RVQ stage 2 is half-configured: trellis_packed2 is absent "
                           f"but inv_resid_scale2 = {inv_resid_scale2}")
    _fused_trellis(x, sv, None, trellis_packed, trellis_packed2, blocks_n, None, blocks_n_meta, None,
                   wscale, inv_resid_scale2, in_features, m_pad, n_pad, m_pad, None,
                   _yrht_slice(y_rht_out, col, m_pad), None)


_META_BLOCKS = _DerivedCache()


def _meta_blocks(meta, num_blocks):
    """Block sizes of a device meta tensor, read back once per tensor (a device-to-host copy on
    every call would stall the batch-1 path and cannot run under graph capture)."""
    hit = _META_BLOCKS.get(meta, (int(num_blocks),))
    if hit is None:
        hit = _META_BLOCKS.put(meta, [int(v) for v in meta[:num_blocks, 1].tolist()], (int(num_blocks),))
    return hit


def glq_decode_matvec_trellis_3inst_fusein_cuda(x_raw, sv, trellis_packed, m, k, in_features,
                                                wscale=1.0, blocks_n_meta=None, num_blocks=1,
                                                max_bs=0, out=None):
    """B=1 GEMV on the raw activations: input RHT + decode + x wscale, (m,) fp32."""
    x2 = x_raw.reshape(1, -1)
    if num_blocks > 1:
        if blocks_n_meta is None:
            raise RuntimeError("block-diagonal fused-input GEMV needs blocks_n_meta")
        blocks = _meta_blocks(blocks_n_meta, int(num_blocks))
    else:
        blocks = [int(k)]
    if out is None:
        out = torch.empty(int(m), dtype=torch.float32, device=x_raw.device)
    _fused_trellis(x2.contiguous(), sv, None, trellis_packed, None, blocks, None, blocks_n_meta, None,
                   wscale, 0.0, in_features, m, k, m, None, (C.c_void_p(out.data_ptr()), int(m)), None)
    return out


# --------------------------------------------------------------------------- E8 shell
_TABLES = _DerivedCache()


def _packed_table(codebook):
    """Nibble-packed copy of an (N, 8) fp16 E8 table, built once per table (the check of the
    table's values reads one word back: made ahead of time by `e8_prepare`, it never runs under
    stream capture)."""
    hit = _TABLES.get(codebook)
    if hit is not None:
        return hit
    lib = _lib.load()
    _chk(codebook, "codebook", torch.float16)
    if codebook.dim() != 2 or codebook.shape[1] != 8 or not 1 <= codebook.shape[0] <= 65536:
        raise RuntimeError(f"codebook must be (N<=65536, 8) fp16, got {tuple(codebook.shape)}")
    packed = torch.empty(codebook.shape[0], dtype=torch.int32, device=codebook.device)
    bad = torch.zeros(1, dtype=torch.int32, device=codebook.device)
    with torch.cuda.device(codebook.device):
        check(lib.glqh_e8_pack_table(_p(codebook), codebook.shape[0], _p(packed), _p(bad), _stream()))
    nbad = int(bad.item())
    if nbad:
        raise RuntimeError(f"codebook has {nbad} rows outside the E8 half-integer grid "
                           "{-3, -2.5, ..., 3}; only E8 shell tables are supported")
    return _TABLES.put(codebook, packed)


_HALF_TABLES = _DerivedCache()


def _half_table(codebook):
    """The table as fp16 (exact for E8 values); converted once per table."""
    if codebook.dtype == torch.float16:
        return codebook
    hit = _HALF_TABLES.get(codebook)
    if hit is None:
        hit = _HALF_TABLES.put(codebook, codebook.to(torch.float16).contiguous())
    return hit


_DEV_TABLES = _DerivedCache()


def _on_device(codebook, dev):
    """`codebook` on `dev`; a table kept on another device (the reference keeps its codebooks on
    the CPU until first use) is copied once per table, so the packed table built from the copy
    is found again on the next call."""
    if codebook.device == dev:
        return codebook
    hit = _DEV_TABLES.get(codebook, (str(dev),))
    if hit is None:
        hit = _DEV_TABLES.put(codebook, codebook.to(dev), (str(dev),))
    return hit


def _per_row(t, n, name):
    """(n,) fp32 per-row scale; a one-element tensor is broadcast."""
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name} must be float32, got {t.dtype}")
    if t.numel() == 1:
        return t.reshape(1).expand(n).contiguous()
    if t.numel() != n:
        raise RuntimeError(f"{name} has {t.numel()} entries, expected {n} (one per row)")
    return t.reshape(n).contiguous()


def glq_embedding_dequant(input_ids, qidxs, sv, wscale, codebook, qidxs2=None, inv_resid_scale=None,
                          codebook2=None, n_pad=None, embedding_dim=None, embed_scale=1.0, out_dtype=None):
    """Rows `input_ids` of a quantized embedding: gather + E8 decode + inverse transform + scale.

    Argument order and semantics of `_dequant_embedding_rows`
    (glq/quantized_linear.py:1277-1340; op schema glq_vllm/custom_ops.py:301-308): returns
    `(*input_ids.shape, embedding_dim)` in `out_dtype` (default: `sv.dtype`).  The tables may
    be fp32 or fp16 `(N, 8)`; `wscale` / `inv_resid_scale` hold one fp32 per row.
    """
    lib = _lib.load()
    _chk(qidxs, "qidxs", torch.int16)
    _chk(sv, "sv", torch.float16)
    dev = qidxs.device
    vocab, nblk = qidxs.shape
    n_pad = int(nblk * 8 if n_pad is None else n_pad)
    if n_pad != nblk * 8:
        raise RuntimeError(f"n_pad={n_pad} but qidxs has {nblk} index columns (n_pad/8 expected)")
    embedding_dim = int(n_pad if embedding_dim is None else embedding_dim)
    if sv.numel() != n_pad:
        raise RuntimeError(f"sv has {sv.numel()} entries, expected n_pad={n_pad}")
    ids = input_ids.reshape(-1).to(device=dev, dtype=torch.int64).contiguous()
    t1 = _primary_table(_half_table(_on_device(codebook, dev)))
    two = qidxs2 is not None and codebook2 is not None and inv_resid_scale is not None
    q2 = t2 = inv = None
    n2 = 0
    if two:
        _chk(qidxs2, "qidxs2", torch.int16)
        if tuple(qidxs2.shape) != (vocab, nblk):
            raise RuntimeError(f"qidxs2 shape {tuple(qidxs2.shape)} != qidxs shape {(vocab, nblk)}")
        q2 = qidxs2
        t2 = _packed_table(_half_table(_on_device(codebook2, dev)))
        n2 = t2.shape[0]
        inv = _per_row(inv_resid_scale.to(dev), vocab, "inv_resid_scale")
    ws = _per_row(wscale.to(dev), vocab, "wscale")
    dt = sv.dtype if out_dtype is None else out_dtype
    if dt not in _DT:
        raise RuntimeError(f"unsupported output dtype {dt}")
    out = torch.empty((ids.numel(), embedding_dim), dtype=dt, device=dev)
    with torch.cuda.device(dev):
        check(lib.glqh_e8_embedding_rows(_p(ids), ids.numel(), _p(qidxs), _p(q2) if two else None, _p(t1),
                                         _p(t2) if two else None, n2, _p(ws), _p(inv) if two else None,
                                         _p(sv), n_pad, embedding_dim, vocab, float(embed_scale), _p(out),
                                         _DT[dt], embedding_dim, _stream()))
    return out.reshape(*input_ids.shape, embedding_dim)


# Folded copies of the index streams (include/glq_hip.h, glqh_e8_fold_table): made by `e8_prepare`
# at load time -- the place the reference prepares its layers is process_weights_after_loading,
# glq_vllm/linear_method.py:1031 -- and kept while the index tensor's storage lives, 1.5 times the
# bytes of the indices they copy.  The forward path only looks them up: a layer that was never
# prepared runs on its indices.  GLQ_E8_FOLD=0 keeps every layer on the indices;
# GLQ_E8_FOLD_MAX_BYTES=<n> bounds the total of the copies (layers prepared after the bound is
# reached stay on their indices).
E8_FOLD = os.environ.get("GLQ_E8_FOLD", "1") != "0"
E8_FOLD_MAX_BYTES = int(os.environ.get("GLQ_E8_FOLD_MAX_BYTES", "0"))       # 0 = no bound
_FOLD_TABLES = _DerivedCache()
_FOLD_STREAMS = _DerivedCache()
_fold_warned = set()


class _E8Folded(C.Structure):
    _fields_ = [("lo16", C.c_void_p * 4), ("hi8", C.c_void_p * 4), ("halves1", C.c_void_p),
                ("n_halves1", C.c_int64), ("halves2", C.c_void_p), ("n_halves2", C.c_int64)]


def _fold_table(packed):
    """(half codewords (n, 4) fp16, map) of a nibble-packed table tensor, once per table; (None, None)
    for a table with more than 2048 distinct half codewords (no E8 shell table has: the full one has
    1286), which the kernels then read through its indices.  Copies the table to the host and
    synchronizes: load time only."""
    hit = _FOLD_TABLES.get(packed)
    if hit is not None:
        return hit
    lib = _lib.load()
    halves = torch.empty((2048, 4), dtype=torch.float16, device=packed.device)
    fmap = torch.empty(packed.shape[0], dtype=torch.int32, device=packed.device)
    n = C.c_int64(0)
    with torch.cuda.device(packed.device):
        rc = lib.glqh_e8_fold_table(_p(packed), packed.shape[0], _p(halves), 2048, _p(fmap), C.addressof(n), _stream())
    if rc != 0 and n.value <= 2048:
        check(rc)
    return _FOLD_TABLES.put(packed, (halves[:n.value].clone(), fmap) if rc == 0 else (None, None))


def _fold_stream(q, packed):
    """(16-bit words, bytes) of one stage's index tensor against its packed table; made once per
    index tensor and table."""
    extra = (packed.data_ptr(),)
    hit = _FOLD_STREAMS.get(q, extra)
    if hit is not None and hit[0]() is packed:
        return hit[1], hit[2]
    lib = _lib.load()
    _, fmap = _fold_table(packed)
    count = lib.glqh_e8_folded_count(q.shape[0], q.shape[1])
    lo16 = torch.empty(count, dtype=torch.int16, device=q.device)
    hi8 = torch.empty(count, dtype=torch.uint8, device=q.device)
    with torch.cuda.device(q.device):
        check(lib.glqh_e8_fold_indices(_p(q), q.shape[0], q.shape[1], _p(fmap), packed.shape[0], _p(lo16), _p(hi8),
                                       _stream()))
    _FOLD_STREAMS.put(q, (weakref.ref(packed), lo16, hi8), extra)
    return lo16, hi8


def e8_fold_bytes():
    """Device bytes held by folded index streams right now."""
    return sum(v[1].numel() * 2 + v[2].numel() for v in _FOLD_STREAMS.values())


def e8_prepare(qidxs, codebook, qidxs2=None, codebook2=None, qidxs3=None, qidxs4=None):
    """Load-time preparation of an E8 layer: the packed table(s) and, for a layer the folded kernels
    serve, the folded copy of every stage's indices.  Call once per layer after its buffers are on
    the GPU and before any stream capture (it allocates, launches and synchronizes); calling it again
    is cheap.  Returns the number of bytes of folded streams the layer holds (0: the layer runs on
    its indices -- too small, `GLQ_E8_FOLD=0`, or the `GLQ_E8_FOLD_MAX_BYTES` bound is reached).

    The reference's counterpart is `GLQLinearMethod.process_weights_after_loading`
    (glq_vllm/linear_method.py:1031-1110), which moves buffers, caches scalars and loads tables."""
    _chk(qidxs, "qidxs", torch.int16)
    dev = qidxs.device
    t1 = _primary_table(_half_table(_on_device(codebook, dev)))
    stages = [(qidxs, t1)]
    if not _absent(qidxs2):
        cb2 = codebook if _absent(codebook2) else codebook2
        stages.append((qidxs2, _packed_table(_half_table(_on_device(cb2, dev)))))
    stages += [(q, t1) for q in (qidxs3, qidxs4) if not _absent(q)]
    M, nblk = qidxs.shape
    lib = _lib.load()
    if not E8_FOLD or not any(lib.glqh_e8_fold_eligible(M, nblk * 8, B) for B in (1, 4, 16, 17, 64)):
        return 0
    need = sum(3 * lib.glqh_e8_folded_count(q.shape[0], q.shape[1]) for q, t in stages
               if _FOLD_STREAMS.get(q, (t.data_ptr(),)) is None)
    if E8_FOLD_MAX_BYTES and e8_fold_bytes() + need > E8_FOLD_MAX_BYTES:
        return 0
    if any(_fold_table(t)[0] is None for _, t in stages):
        return 0
    total = 0
    for q, t in stages:
        _chk(q, "qidxs", torch.int16)
        lo16, hi8 = _fold_stream(q, t)
        total += lo16.numel() * 2 + hi8.numel()
    return total


def e8_release(*qidxs):
    """Drop the folded copies of the given index tensors now (they also go with their storage)."""
    for q in qidxs:
        if q is None:
            continue
        for k in [k for k in _FOLD_STREAMS._d if k[0] == q.data_ptr()]:
            del _FOLD_STREAMS._d[k]


def _e8_folded(B, qidxs, t1, q2, t2, q3, q4):
    """The folded streams of a layer as the C struct (and what must stay alive during the call), or
    (None, None) when the call would not read them or `e8_prepare` has not made them.  Looks up
    only: nothing is allocated, launched or synchronized here, so it is safe under stream capture."""
    M, nblk = qidxs.shape
    if not E8_FOLD or not qidxs.is_contiguous():
        return None, None
    lib = _lib.load()
    if not lib.glqh_e8_fold_eligible(M, nblk * 8, B):
        return None, None
    stages = [(qidxs, t1)] + ([(q2, t2)] if q2 is not None else []) + [(q, t1) for q in (q3, q4) if q is not None]
    keep, f = [], _E8Folded()
    for s, (q, t) in enumerate(stages):
        hit = _FOLD_STREAMS.get(q, (t.data_ptr(),))
        if hit is None or hit[0]() is not t:
            key = (qidxs.data_ptr(), tuple(qidxs.shape))
            if key not in _fold_warned and len(_fold_warned) < 4096:
                _fold_warned.add(key)
                warnings.warn(f"E8 layer {M}x{nblk * 8} was not prepared (glq_amd.ext.e8_prepare / "
                              "E8RHTLinear.prepare): it runs on its indices, which is slower at 1-4096 "
                              "tokens" + (" -- first seen under stream capture, the graph keeps that form"
                                          if torch.cuda.is_current_stream_capturing() else ""),
                              RuntimeWarning, stacklevel=4)
            return None, None
        keep += [hit[1], hit[2]]
        f.lo16[s], f.hi8[s] = hit[1].data_ptr(), hit[2].data_ptr()
    tables = [t1] + ([t2] if q2 is not None and t2 is not t1 else [])
    halves = [_FOLD_TABLES.get(t) for t in tables]
    if any(h is None or h[0] is None for h in halves):
        return None, None
    keep += [h[0] for h in halves]
    f.halves1, f.n_halves1 = halves[0][0].data_ptr(), halves[0][0].shape[0]
    if len(tables) == 2:
        f.halves2, f.n_halves2 = halves[1][0].data_ptr(), halves[1][0].shape[0]
    return f, keep


def _primary_table(codebook):
    """Packed first-stage table: the kernels index it with the full 16-bit pattern and keep
    its low-norm prefix in LDS, so it must be the whole 65536-entry table (the reference's
    first-stage codebook always is, glq/codebook.py:169-192)."""
    if codebook.dim() != 2 or codebook.shape[0] != 65536:
        raise RuntimeError(f"the first-stage E8 table must have 65536 entries, got {tuple(codebook.shape)}")
    return _packed_table(codebook)


def _absent(t):
    return t is None or t.numel() == 0


def _e8_args(qidxs, codebook, qidxs2, codebook2, inv_rs, qidxs3, inv_rs2, qidxs4, inv_rs3):
    _chk(qidxs, "qidxs", torch.int16)
    t1 = _primary_table(codebook)
    q2 = None if _absent(qidxs2) or float(inv_rs) == 0.0 else qidxs2
    t2, n2 = None, 0
    if q2 is not None:
        _chk(q2, "qidxs2", torch.int16)
        t2 = _packed_table(codebook if _absent(codebook2) else codebook2)
        n2 = t2.shape[0]
    q3 = None if q2 is None or _absent(qidxs3) or float(inv_rs2) == 0.0 else qidxs3
    q4 = None if q3 is None or _absent(qidxs4) or float(inv_rs3) == 0.0 else qidxs4
    for q, nme in ((q3, "qidxs3"), (q4, "qidxs4")):
        if q is not None:
            _chk(q, nme, torch.int16)
    return t1, q2, t2, n2, q3, q4


def _e8_dense_weight(qidxs, t1, q2, t2, n2, q3, q4, inv_rs, inv_rs2, inv_rs3):
    lib = _lib.load()
    M, nblk = qidxs.shape
    W = torch.empty((M, nblk * 8), dtype=torch.float16, device=qidxs.device)
    with torch.cuda.device(qidxs.device):
        check(lib.glqh_e8_decompress(_p(qidxs), _p(q2), _p(q3), _p(q4), _p(t1), _p(t2), n2,
                                     float(inv_rs), float(inv_rs2), float(inv_rs3), M, nblk * 8,
                                     _p(W), _stream()))
    return W


def _e8_matmul_tables(x, qidxs, t1, q2, t2, n2, q3, q4, wscale, inv_rs, inv_rs2, inv_rs3):
    """(B, N) fp16 x against packed tables -> (B, M) fp32."""
    lib = _lib.load()
    _chk(x, "x", torch.float16)
    B = x.shape[0]
    M, nblk = qidxs.shape
    if x.shape[1] != nblk * 8:
        raise RuntimeError(f"x has {x.shape[1]} columns, qidxs implies {nblk * 8}")
    folded, keep = None, None
    if not _e8_dense_route(B, nblk * 8, True):
        with torch.cuda.device(x.device):
            folded, keep = _e8_folded(B, qidxs, t1, q2, t2, q3, q4)
    if _e8_dense_route(B, nblk * 8, folded is not None):
        W = _e8_dense_weight(qidxs, t1, q2, t2, n2, q3, q4, inv_rs, inv_rs2, inv_rs3)
        return torch.mm(x, W.t(), out_dtype=torch.float32).mul_(float(wscale))
    out = torch.empty((B, M), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        nb = lib.glqh_e8_matmul_workspace_bytes(M, nblk * 8, B)
        ws = _ws(nb, x.device)
        check(lib.glqh_e8_dequant_matmul_folded(
            _p(x), B, _p(qidxs), _p(q2), _p(q3), _p(q4), _p(t1), _p(t2), n2, float(wscale),
            float(inv_rs), float(inv_rs2), float(inv_rs3), M, nblk * 8,
            _p(out), _p(ws), ws.numel(), _stream(), C.addressof(folded) if folded is not None else None))
    del keep
    return out


def glq_dequant_matmul_cuda(x, qidxs, codebook, wscale, qidxs2=None, codebook2=None,
                            inv_resid_scale=0.0, codebook_abs=None, qidxs3=None, codebook3=None,
                            inv_resid_scale2=0.0, qidxs4=None, codebook4=None, inv_resid_scale3=0.0):
    """(B, N) fp16 RHT-domain activations -> (B, M) fp32."""
    t1, q2, t2, n2, q3, q4 = _e8_args(qidxs, codebook, qidxs2, codebook2, inv_resid_scale, qidxs3,
                                      inv_resid_scale2, qidxs4, inv_resid_scale3)
    return _e8_matmul_tables(x, qidxs, t1, q2, t2, n2, q3, q4, wscale, inv_resid_scale,
                             inv_resid_scale2, inv_resid_scale3)


def glq_dequant_matvec_cuda(x, qidxs, codebook, wscale, qidxs2=None, codebook2=None,
                            inv_resid_scale=0.0, codebook_abs=None):
    """(N,) fp16 -> (M,) fp32."""
    return glq_dequant_matmul_cuda(x.reshape(1, -1), qidxs, codebook, wscale, qidxs2, codebook2,
                                   inv_resid_scale).reshape(-1)


_REPACKED = _DerivedCache()


def _repacked_table(codebook_packed):
    """The reference's `codebook_packed` (65536 int32, nibble c = column c,
    glq/codebook.py:102-115) in the kernels' nibble order, converted once per table."""
    _chk(codebook_packed, "codebook_packed", torch.int32)
    if codebook_packed.dim() != 1 or codebook_packed.shape[0] != 65536:
        raise RuntimeError("codebook_packed must hold 65536 int32 words, got "
                           f"{tuple(codebook_packed.shape)}")
    hit = _REPACKED.get(codebook_packed)
    if hit is not None:
        return hit
    lib = _lib.load()
    out = torch.empty_like(codebook_packed)
    bad = torch.zeros(1, dtype=torch.int32, device=codebook_packed.device)
    with torch.cuda.device(codebook_packed.device):
        check(lib.glqh_e8_repack_table(_p(codebook_packed), 65536, _p(out), _p(bad), _stream()))
    nbad = int(bad.item())
    if nbad:
        raise RuntimeError(f"codebook_packed has {nbad} words with a code above 12; only E8 shell "
                           "tables are supported")
    return _REPACKED.put(codebook_packed, out)


def glq_dequant_matmul_packed_cuda(x, qidxs, codebook_packed, wscale):
    """Single-stage (B, N) fp16 -> (B, M) fp32 against the 4-bit packed table
    (glq/csrc/glq_bindings.cpp:45-50; caller glq/inference_kernel.py:1047-1054)."""
    _chk(qidxs, "qidxs", torch.int16)
    t1 = _repacked_table(codebook_packed)
    return _e8_matmul_tables(x, qidxs, t1, None, None, 0, None, None, wscale, 0.0, 0.0, 0.0)


def glq_dequant_matvec_packed_cuda(x, qidxs, codebook_packed, wscale):
    """Single-stage (N,) fp16 -> (M,) fp32 (glq/csrc/glq_bindings.cpp:38-43)."""
    return glq_dequant_matmul_packed_cuda(x.reshape(1, -1), qidxs, codebook_packed, wscale).reshape(-1)


def _fused_e8(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad, m_pad,
              blocks_n, blocks_m, bn_meta, bm_meta, qidxs2, codebook2, inv_rs, qidxs3, inv_rs2,
              qidxs4, inv_rs3, out_dtype):
    lib = _lib.load()
    _chk(x, "x", (torch.float16, torch.bfloat16))
    _chk(sv, "sv", torch.float16)
    _chk(su, "su", torch.float16)
    t1, q2, t2, n2, q3, q4 = _e8_args(qidxs, codebook, qidxs2, codebook2, inv_rs, qidxs3, inv_rs2,
                                      qidxs4, inv_rs3)
    if tuple(qidxs.shape) != (int(m_pad), int(n_pad) // 8):
        raise RuntimeError(f"qidxs shape {tuple(qidxs.shape)} != (m_pad, n_pad/8)")
    B = x.shape[0]
    bn, nbn = _host_i64(blocks_n)
    bm, nbm = _host_i64(blocks_m)
    y = torch.empty((B, int(out_features)), dtype=out_dtype or torch.float16, device=x.device)
    folded, keep = None, None
    if not _e8_dense_route(B, n_pad, True):
        with torch.cuda.device(x.device):
            folded, keep = _e8_folded(B, qidxs, t1, q2, t2, q3, q4)
    if _e8_dense_route(B, n_pad, folded is not None):
        x_rht = torch.empty((B, int(n_pad)), dtype=torch.float16, device=x.device)
        glq_input_rht_blockdiag_cuda(x, sv, x_rht, in_features, n_pad, blocks_n, bn_meta)
        W = _e8_dense_weight(qidxs, t1, q2, t2, n2, q3, q4, inv_rs, inv_rs2, inv_rs3)
        return _dense_matmul_output(x_rht, W, wscale, su, y, out_features, m_pad, blocks_m, bm_meta)
    with torch.cuda.device(x.device):
        nb = lib.glqh_fused_linear_e8_workspace_bytes(B, int(n_pad), int(m_pad))
        ws = _ws(nb, x.device)
        check(lib.glqh_fused_linear_e8_folded(
            _p(x), _DT[x.dtype], x.shape[1], B, _p(sv), _p(su), _p(qidxs), _p(q2), _p(q3), _p(q4),
            _p(t1), _p(t2), n2, float(wscale), float(inv_rs), float(inv_rs2), float(inv_rs3),
            bn, nbn, bm, nbm, _meta_ptr(bn_meta) if nbn > 1 else None,
            _meta_ptr(bm_meta) if nbm > 1 else None, int(in_features), int(out_features), int(n_pad),
            int(m_pad), _p(y), _DT[y.dtype], y.shape[1], _p(ws), ws.numel(), _stream(),
            C.addressof(folded) if folded is not None else None))
    del keep
    return y


def glq_fused_linear_cuda(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad,
                          m_pad, log_n, log_m, qidxs2=None, codebook2=None, inv_resid_scale=0.0,
                          qidxs3=None, codebook3=None, inv_resid_scale2=0.0, qidxs4=None,
                          codebook4=None, inv_resid_scale3=0.0, out_dtype=None):
    if (1 << int(log_n)) != int(n_pad) or (1 << int(log_m)) != int(m_pad):
        raise RuntimeError("glq_fused_linear_cuda needs power-of-two n_pad and m_pad")
    return _fused_e8(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad, m_pad,
                     [int(n_pad)], [int(m_pad)], None, None, qidxs2, codebook2, inv_resid_scale,
                     qidxs3, inv_resid_scale2, qidxs4, inv_resid_scale3, out_dtype)


def glq_fused_linear_block_diag_cuda(x, sv, su, qidxs, codebook, wscale, in_features, out_features,
                                     n_pad, m_pad, blocks_n, blocks_m, blocks_n_meta, blocks_m_meta,
                                     qidxs2=None, codebook2=None, inv_resid_scale=0.0, qidxs3=None,
                                     codebook3=None, inv_resid_scale2=0.0, qidxs4=None,
                                     codebook4=None, inv_resid_scale3=0.0, out_dtype=None):
    return _fused_e8(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad, m_pad,
                     blocks_n, blocks_m, blocks_n_meta, blocks_m_meta, qidxs2, codebook2,
                     inv_resid_scale, qidxs3, inv_resid_scale2, qidxs4, inv_resid_scale3, out_dtype)


# ---- encode side ----------------------------------------------------------------------
def e8_quantize(x, codebook, codebook_norms=None, return_decoded=True):
    """E8ShellCodebook.quantize (glq/codebook.py:227-278) on the GPU: nearest row of
    `codebook` (K, 8) for every row of x (N, 8), lowest index on ties.  fp32 arithmetic in
    coordinate order, the reference's CPU branch.  Returns (decoded fp32 (N, 8), idx int64)."""
    lib = _lib.load()
    if x.dim() != 2 or x.shape[1] != 8:
        raise RuntimeError(f"x must be (N, 8), got {tuple(x.shape)}")
    xf = x.contiguous().to(torch.float32)
    _chk(xf, "x", torch.float32)
    cb = codebook.contiguous().to(torch.float32)
    norms = (cb * cb).sum(-1) if codebook_norms is None else codebook_norms.contiguous().to(torch.float32)
    N = xf.shape[0]
    idx = torch.empty(N, dtype=torch.int64, device=x.device)
    dec = torch.empty(N, 8, dtype=torch.float32, device=x.device) if return_decoded else None
    if N:
        with torch.cuda.device(x.device):
            check(lib.glqh_e8_quantize(_p(xf), _p(cb), _p(norms), N, cb.shape[0], _p(idx), _p(dec), _stream()))
    return dec, idx


def trellis_quantize_tiles(tiles, K):
    """bitshift_codebook.quantize (glq/trellis.py:467-484) on the GPU: (B, 256) tiles in step
    order -> (hat (B, 256) fp32, states (B, 256) int32), tail-biting Viterbi, K = 1..4."""
    lib = _lib.load()
    if tiles.dim() != 2 or tiles.shape[1] != 256:
        raise RuntimeError(f"tiles must be (B, 256), got {tuple(tiles.shape)}")
    x = tiles.contiguous().to(torch.float32)
    _chk(x, "tiles", torch.float32)
    B = x.shape[0]
    states = torch.empty(B, 256, dtype=torch.int32, device=x.device)
    hat = torch.empty(B, 256, dtype=torch.float32, device=x.device)
    if B:
        with torch.cuda.device(x.device):
            nb = lib.glqh_trellis_quantize_workspace_bytes(int(K), B)
            ws = _ws(max(nb, 256), x.device)
            check(lib.glqh_trellis_quantize_tiles(_p(x), B, int(K), _p(states), _p(hat), _p(ws), ws.numel(),
                                                  _stream()))
    return hat, states


def viterbi_acs_step(cost, x, lut, K, prev_out, cost_out=None):
    """One add-compare-select step (bitshift_codebook.update, glq/trellis.py:230-251): cost
    (B, 65536) fp32, x (B) fp16 (the step's inputs), lut (65536) fp32 -> new cost; the int32
    predecessors go to prev_out (B, 2^(16-K))."""
    lib = _lib.load()
    _chk(cost, "cost", torch.float32)
    _chk(x, "x", torch.float16)
    _chk(lut, "lut", torch.float32)
    _chk(prev_out, "prev_out", torch.int32)
    B = cost.shape[0]
    if cost.dim() != 2 or cost.shape[1] != 65536 or x.numel() != B or lut.numel() != 65536:
        raise RuntimeError(f"viterbi step: cost {tuple(cost.shape)}, x {tuple(x.shape)}, lut "
                           f"{tuple(lut.shape)} do not describe B sequences over 65536 states")
    if tuple(prev_out.shape) != (B, 1 << (16 - int(K))):
        raise RuntimeError(f"viterbi step: prev_out {tuple(prev_out.shape)} != (B, 2^(16-K))")
    if cost_out is None:
        cost_out = torch.empty_like(cost)
    else:
        _chk(cost_out, "cost_out", torch.float32)
    with torch.cuda.device(cost.device):
        check(lib.glqh_viterbi_acs_step(_p(cost), _p(x), _p(lut), _p(cost_out), _p(prev_out), B, int(K),
                                        _stream()))
    return cost_out


def _step_permutation(device):
    """Position (row*16 + col) of trellis step t = 8l + j inside its 16x16 tile
    (glq/trellis.py:99-101)."""
    t = torch.arange(256, device=device)
    l, j = t >> 3, t & 7
    row = (l >> 2) + 8 * ((j >> 1) & 1)
    col = 2 * (l & 3) + 8 * (j >> 2) + (j & 1)
    return row * 16 + col


def trellis_matrix_to_tiles(W):
    """(m, n) -> (tiles, 256) in trellis-step order, tiles row-major (glq/trellis.py:679-681)."""
    m, n = W.shape
    nat = W.reshape(m // 16, 16, n // 16, 16).permute(0, 2, 1, 3).reshape(-1, 256)
    return nat[:, _step_permutation(W.device)].contiguous()


def trellis_tiles_to_matrix(tiles, m, n):
    inv = torch.empty(256, dtype=torch.int64, device=tiles.device)
    inv[_step_permutation(tiles.device)] = torch.arange(256, device=tiles.device)
    nat = tiles[:, inv].reshape(m // 16, n // 16, 16, 16).permute(0, 2, 1, 3)
    return nat.reshape(m, n).contiguous()


def trellis_pack_states(states, m, n, K):
    """(tiles, 256) int32 states -> trellis_packed ((m/16)(n/16), 16K) int16
    (glq/trellis.py:486-510, 580-619)."""
    lib = _lib.load()
    _chk(states, "states", torch.int32)
    if states.shape != ((int(m) // 16) * (int(n) // 16), 256):
        raise RuntimeError(f"states must be ((m/16)(n/16), 256), got {tuple(states.shape)}")
    packed = torch.empty((states.shape[0], 16 * int(K)), dtype=torch.int16, device=states.device)
    with torch.cuda.device(states.device):
        check(lib.glqh_trellis_pack_states(_p(states), int(m), int(n), int(K), _p(packed), _stream()))
    return packed


def trellis_quantize_matrix(W_rht, K):
    """Normalised RHT-domain weight (m, n) -> (trellis_packed, reconstruction (m, n) fp32):
    tiles -> tail-biting Viterbi -> pack (the identity-Hessian case of
    quantize_layer_trellis_rht, glq/trellis.py:649-688)."""
    m, n = W_rht.shape
    hat, states = trellis_quantize_tiles(trellis_matrix_to_tiles(W_rht.to(torch.float32)), K)
    return trellis_pack_states(states, m, n, K), trellis_tiles_to_matrix(hat, m, n)
