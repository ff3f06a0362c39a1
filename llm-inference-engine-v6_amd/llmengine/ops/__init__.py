"""The HIP kernels of the engine, as Python functions over device tensors."""
from .lib import KernelError, KernelLibraryError, library
from .kernels import (argmax, attention, attention_generic, rope_q_only, embed_gather, gemm, gemm_generic, policy, rmsnorm,
                      rope_kv_write, sample, swiglu)

__all__ = ["KernelError", "KernelLibraryError", "library", "argmax", "attention", "attention_generic", "rope_q_only", "embed_gather",
           "gemm", "gemm_generic", "policy", "rmsnorm", "rope_kv_write", "sample", "swiglu"]
