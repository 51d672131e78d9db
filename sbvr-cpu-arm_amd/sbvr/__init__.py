"""sbvr: SBVR ("sum of binary vectors") tensors and their compressed-domain
matrix products on MI355X.  Same names as the reference package
(sbvr/__init__.py:1-5 there): ``sbvr``, ``_sbvr_serialized``, ``load``, ``mm_T`` and
the ``_sbvr_*`` operators, the CUDA ones now backed by HIP kernels for gfx950.
The reference's ARM-NEON operators (``_sbvr_cpu_mm_T``, ``_sbvr_cpu_v2_mm_T`` and
their thread-pool calls) have no counterpart here."""
import torch

from .core import sbvr, _sbvr_serialized, load, mm_T
from .hip import (_sbvr_hip_init, _sbvr_cuda_init, _sbvr_mm_T, _sbvr_row_deq_mm_T,
                  _sbvr_linear_f16, _sbvr_linear_f16_swiglu, _sbvr_linear_f16_add_rmsnorm, SbvrHipError)
from .linear import SBVRLinear

torch.serialization.add_safe_globals([_sbvr_serialized])

__all__ = ["sbvr", "_sbvr_serialized", "load", "mm_T", "_sbvr_hip_init", "_sbvr_cuda_init",
           "_sbvr_mm_T", "_sbvr_row_deq_mm_T", "_sbvr_linear_f16", "_sbvr_linear_f16_swiglu",
           "_sbvr_linear_f16_add_rmsnorm", "SBVRLinear", "SbvrHipError"]
