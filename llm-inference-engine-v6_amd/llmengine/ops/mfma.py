"""The MFMA (matrix core) kernels: bfloat16 matrix products and, in a later section,
attention. Importing this module makes `ops.gemm` and `ops.attention` choose them where
operand types and sizes fit; what they refuse goes to the plain-precision kernels."""
from __future__ import annotations

import ctypes

import torch

from . import kernels
from .lib import check, declare, entry, ptr, require, stream

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

declare("llme_gemm_bf16", [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp])


def gemm_bf16_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and out.dtype in (torch.float32, torch.bfloat16)
            and not (accumulate and out.dtype != torch.float32)
            and a.shape[1] % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and out.data_ptr() % 16 == 0)


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, *,
              waves: int = 0, ksplit: int = 0, force_tile: bool = False) -> None:
    """bfloat16 a [M, K] and w [N, K] -> out [M, N] (float32 or bfloat16), 32-bit accumulation.
    K must be a multiple of 8. waves / ksplit / force_tile override the launch choices (tests)."""
    require(a, "a", torch.bfloat16, (None, None))
    M, K = a.shape
    require(w, "w", torch.bfloat16, (None, K))
    N = w.shape[0]
    require(out, "out", (torch.float32, torch.bfloat16), (M, N))
    if not gemm_bf16_supported(a, w, out, accumulate):
        raise kernels.KernelError(f"gemm_bf16: K={K} must be a multiple of 8, pointers 16-byte aligned, and "
                                  "accumulation needs a float32 output")
    check(entry("llme_gemm_bf16")(ptr(a), ptr(w), ptr(out), 0 if out.dtype == torch.float32 else 1, M, N, K,
                                  1 if accumulate else 0, waves, ksplit, 1 if force_tile else 0, stream()),
          "gemm_bf16")


def _fast_gemm(a, w, out, accumulate) -> bool:
    if a.dim() != 2 or w.dim() != 2 or not gemm_bf16_supported(a, w, out, accumulate):
        return False
    gemm_bf16(a, w, out, accumulate)
    return True


kernels._fast_gemm = _fast_gemm
