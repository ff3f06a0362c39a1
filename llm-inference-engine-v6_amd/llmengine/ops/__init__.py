"""The HIP kernels of the engine, as Python functions over device tensors."""
from .lib import KernelError, KernelLibraryError, library, load_kernels
from .choices import KernelChoices
from .kernels import (ATTENTION_MAX_HEAD_DIM, argmax, argmax_into, attention, attention_generic, attention_project, block_weight, can_block, clear, embed_gather, gemm,
                      gemm_generic, is_blocked, policy, rmsnorm, rope_kv_write, rope_q_only, sample, sample_into, sampling_scratch, swiglu,
                      unblock_weight, weight_shape)

from . import mfma                                   # noqa: E402  (installs the MFMA kernels)
from .mfma import (gemm_bf16, gemm_gated, gemm_qkv_rope, gemm_qkv_rope_supported, gemv_norm, gemv_norm_rope, gemv_norm_rope_supported,
                   gemv_norm_supported, pair_rows_for_rotation)

__all__ = ["KernelChoices", "ATTENTION_MAX_HEAD_DIM", "gemm_bf16", "gemm_gated", "gemm_qkv_rope", "gemm_qkv_rope_supported", "gemv_norm_rope", "gemv_norm_rope_supported", "pair_rows_for_rotation", "gemv_norm", "gemv_norm_supported", "mfma", "KernelError", "KernelLibraryError", "library", "load_kernels", "argmax", "argmax_into", "attention", "attention_generic", "attention_project", "rope_q_only", "embed_gather", "block_weight", "can_block", "clear",
           "is_blocked", "unblock_weight", "weight_shape",
           "gemm", "gemm_generic", "policy", "rmsnorm", "rope_kv_write", "sample", "sample_into", "sampling_scratch", "swiglu"]
