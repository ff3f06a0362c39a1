"""The HIP kernels of the engine, as Python functions over device tensors."""
from .lib import KernelError, KernelLibraryError, library
from .kernels import (argmax, argmax_into, attention, attention_generic, rope_q_only, embed_gather, gemm, gemm_generic, policy, rmsnorm,
                      rope_kv_write, sample, swiglu)

from . import mfma                                   # noqa: E402  (installs the MFMA kernels)
from .mfma import (gemm_bf16, gemm_gated, gemv_norm, gemv_norm_rope, gemv_norm_rope_supported,
                   gemv_norm_supported)

__all__ = ["gemm_bf16", "gemm_gated", "gemv_norm_rope", "gemv_norm_rope_supported", "gemv_norm", "gemv_norm_supported", "mfma", "KernelError", "KernelLibraryError", "library", "argmax", "argmax_into", "attention", "attention_generic", "rope_q_only", "embed_gather",
           "gemm", "gemm_generic", "policy", "rmsnorm", "rope_kv_write", "sample", "swiglu"]
