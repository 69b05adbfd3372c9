"""glq_amd -- MI355X (gfx950) implementation of GLQ's quantized-linear forward.

The compute path is hand-written HIP in ``libglq_hip.so`` (C ABI, see
``include/glq_hip.h``); this package is the thin PyTorch-ROCm host side that mirrors
the reference's operator surface:

* ``glq_amd.ext``               the functions of the reference's pybind extension
                                (``glq._C`` / ``glq_cuda``), same names and arguments
* ``glq_amd.custom_ops``        the ``torch.ops.glq.*`` schemas of ``glq_vllm/custom_ops.py``
* ``glq_amd.quantized_linear``  ``E8RHTLinear`` with the reference's buffer names
* ``glq_amd.linear_method``     the serving layer's call sequence for merged trellis linears
                                (``glq_vllm/linear_method.py``) and the load-time step
* ``glq_amd.dequant``           dense weights from quantized layers (``glq_vllm/dequant.py``)
* ``glq_amd.inference_kernel``, ``glq_amd.hadamard``, ``glq_amd.codebook_kernel``,
  ``glq_amd.trellis_step_kernel``  the public functions of the reference's same-named
                                modules (``glq_dequant_matmul``, ``fast_hadamard_transform``,
                                ``triton_codebook_nn``, ``fused_update`` ...)

There is no CPU fallback: importing ``glq_amd.ext`` without the built library, or
calling an op without a GPU, raises.
"""

__version__ = "0.1.0"

from .hadamard import block_decompose, pack_block_meta, pack_shard_meta  # noqa: F401
