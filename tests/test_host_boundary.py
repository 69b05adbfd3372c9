"""CPU-only checks of the drop-in boundary: the library loads, exports every symbol the
header declares, and the host helpers match the reference's integer bookkeeping."""
import os
import re

import numpy as np
import torch

from glq_amd import _lib, hadamard
from oracle import glq_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    syms = set()
    for name in sorted(os.listdir(os.path.join(ROOT, "include"))):
        if not name.endswith(".h"):
            continue
        txt = open(os.path.join(ROOT, "include", name)).read()
        txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
        syms |= set(re.findall(r"\b(glqh_[a-z0-9_]+)\s*\(", txt))
    return sorted(syms)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    syms = header_symbols()
    assert len(syms) >= 15
    for s in syms:
        assert hasattr(lib, s), f"libglq_hip.so does not export {s}"
    assert sorted(_lib.SIGNATURES) == syms, "ctypes table and header disagree"
    assert lib.glqh_version() >= 1


def test_shape_gate_needs_no_gpu():
    lib = _lib.load()
    assert lib.glqh_trellis_kernel_supported(2048, 11008) == 1
    assert lib.glqh_trellis_kernel_supported(2048 + 16, 2048) == 0
    assert lib.glqh_trellis_kernel_supported(2048, 2048 + 32) == 0


def test_block_helpers_match_oracle_and_doctests():
    for n in (2688, 4096, 5376, 960, 11008, 14336, 48, 10):
        assert hadamard.block_decompose(n) == O.block_decompose(n)
        meta = hadamard.pack_block_meta(hadamard.block_decompose(n))
        assert meta.dtype == torch.int32 and meta.device.type == "cpu"
        assert np.array_equal(meta.numpy(), O.pack_block_meta(O.block_decompose(n)))
    sb = [[2048], [512], [512, 256]]
    assert np.array_equal(hadamard.pack_shard_meta(sb).numpy(), O.pack_shard_meta(sb))
    assert hadamard.block_decompose(2688) == [2048, 512, 128]


def test_ext_has_the_reference_entry_names():
    from glq_amd import ext
    for name in ("glq_trellis_kernel_supported", "glq_decompress_trellis_3inst_cuda",
                 "glq_decode_matvec_trellis_3inst_cuda", "glq_decode_matmul_trellis_3inst_cuda",
                 "glq_decode_matvec_trellis_3inst_fusein_cuda",
                 "glq_fused_linear_trellis_3inst_cuda", "glq_fused_linear_trellis_3inst_rvq2_cuda",
                 "glq_fused_linear_trellis_3inst_yrht_cuda",
                 "glq_fused_linear_trellis_3inst_yrht_rvq2_cuda", "glq_output_rht_shards_cuda",
                 "glq_input_rht_cuda", "glq_output_rht_cuda", "glq_input_rht_blockdiag_cuda",
                 "glq_output_rht_blockdiag_cuda", "glq_dequant_matvec_cuda",
                 "glq_dequant_matmul_cuda", "glq_fused_linear_cuda",
                 "glq_fused_linear_block_diag_cuda"):
        assert callable(getattr(ext, name)), name
    assert ext.glq_trellis_kernel_supported(64, 128) and not ext.glq_trellis_kernel_supported(48, 128)
