"""The reference's `glq.inference_kernel` surface on the HIP library.

Mirrors what call sites reach through that module: the extension handle and its status
functions (glq/inference_kernel.py:185-346: `_glq_cuda`, `_try_load_cuda_ext`,
`cuda_ext_status`, `require_cuda_ext`) and the E8 dispatcher `glq_dequant_matmul`
(glq/inference_kernel.py:952-1191).  `_glq_cuda` is `glq_amd.ext`, whose functions carry
the reference's pybind names.  The reference's CPU branch (`_fallback_dequant_matmul`,
:1194-1216) has no counterpart: CPU tensors and a missing library raise.
"""
from __future__ import annotations

import torch

from . import _lib

_glq_cuda = None
_cuda_ext_available = False
_cuda_ext_error = None


def _try_load_cuda_ext() -> bool:
    """Load libglq_hip.so once; True when the kernels can be called."""
    global _glq_cuda, _cuda_ext_available, _cuda_ext_error
    if _glq_cuda is not None:
        return True
    ok, err = _lib.status()
    if ok:
        from . import ext
        _glq_cuda = ext
        _cuda_ext_available, _cuda_ext_error = True, None
    else:
        _cuda_ext_available, _cuda_ext_error = False, err
    return ok


def cuda_ext_status():
    """(available, error): error is the loader's own message, or None."""
    _try_load_cuda_ext()
    return _cuda_ext_available, _cuda_ext_error


def require_cuda_ext(symbol=None):
    """The extension module, or a named error: the library never loaded, or it loaded but
    lacks `symbol` (glq/inference_kernel.py:198-223)."""
    available, error = cuda_ext_status()
    if not available:
        raise RuntimeError("GLQ HIP extension is not available, so this kernel cannot run.\n"
                           f"{error}")
    if symbol is not None and not hasattr(_glq_cuda, symbol):
        raise RuntimeError(f"GLQ HIP extension is loaded but has no '{symbol}'")
    return _glq_cuda


def glq_dequant_matmul(x, Qidxs, codebook, Wscale, Qidxs2=None, codebook2=None, inv_resid_scale=0.0,
                       codebook_packed=None, Qidxs3=None, codebook3=None, inv_resid_scale2=0.0,
                       Qidxs4=None, codebook4=None, inv_resid_scale3=0.0):
    """Y = X @ dequant(Qidxs)^T * Wscale, X (B, N) -> Y (B, M) fp32.  Stage s is active
    when both its indices and its table are given (glq/inference_kernel.py:1001-1003); the
    routes are the reference's (:1038-1069): one token -> matvec, a single stage with
    `codebook_packed` -> the packed-table entry, everything else -> matmul.  One token with
    stages 3-4 goes to matmul, which sums all stages (the reference's matvec entry has no
    arguments for them)."""
    if not x.is_cuda:
        raise RuntimeError("glq_dequant_matmul is GPU only here; there is no CPU fallback")
    ext = require_cuda_ext()
    B, N = x.shape
    M, n_blocks = Qidxs.shape
    assert n_blocks == N // 8, f"Qidxs shape {tuple(Qidxs.shape)} incompatible with N={N}"
    assert codebook.shape[1] == 8
    x16 = x.half().contiguous()
    cb = ext._half_table(codebook)              # converted once per table tensor
    has2 = Qidxs2 is not None and codebook2 is not None
    has3 = Qidxs3 is not None and codebook3 is not None
    has4 = Qidxs4 is not None and codebook4 is not None
    q2 = Qidxs2.contiguous() if has2 else None
    cb2 = ext._half_table(codebook2) if has2 else None
    irs = float(inv_resid_scale) if has2 else 0.0
    if B == 1 and not has3 and not has4:
        return ext.glq_dequant_matvec_cuda(x16[0], Qidxs.contiguous(), cb, float(Wscale), q2, cb2,
                                           irs).unsqueeze(0)
    if not has2 and not has3 and not has4 and codebook_packed is not None:
        return ext.glq_dequant_matmul_packed_cuda(x16, Qidxs.contiguous(), codebook_packed, float(Wscale))
    return ext.glq_dequant_matmul_cuda(
        x16, Qidxs.contiguous(), cb, float(Wscale), q2, cb2, irs, None,
        Qidxs3.contiguous() if has3 else None, ext._half_table(codebook3) if has3 else None,
        float(inv_resid_scale2) if has3 else 0.0,
        Qidxs4.contiguous() if has4 else None, ext._half_table(codebook4) if has4 else None,
        float(inv_resid_scale3) if has4 else 0.0)
