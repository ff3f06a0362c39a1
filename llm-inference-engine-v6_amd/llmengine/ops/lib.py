"""Loads the HIP kernel library and declares its entry points.

There is no other implementation behind these operations: if the library cannot
be built or loaded, the first use raises `KernelLibraryError`.
"""
from __future__ import annotations

import ctypes
import threading

import torch

from . import build as _build


class KernelLibraryError(RuntimeError):
    pass


class KernelError(RuntimeError):
    pass


F32, BF16 = 0, 1            # dtype codes of csrc/common.h
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None
_lock = threading.Lock()

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

_SIGNATURES = {
    "llme_embed_gather": [_vp, _i, _vp, _vp, _i, _i, _i, _vp],
    "llme_clear_f32": [_vp, ctypes.c_size_t, _vp],
    "llme_rmsnorm": [_vp, _vp, _i, _vp, _i, _vp, _i, _i, _f, _vp],
    "llme_swiglu": [_vp, _i, _vp, _i, _i, _i, _i, _vp],
    "llme_rope_kv_write": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i,
                           _i, _i, _i, _i, _i, _i, _i, _i, _vp],
    "llme_gemm_generic": [_vp, _i, _vp, _i, _vp, _i, _i, _i, _i, _i, _i, _vp],
    "llme_attention_generic": [_vp, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                               _f, _i, _vp],
    "llme_argmax": [_vp, _vp, _vp, _vp, _i, _i, _vp],
    "llme_argmax_to": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp],
    "llme_argmax_parts": [_i],
    "llme_compute_units": [],
    "llme_sample": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp],
    "llme_sample_to": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp],
}


def library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        try:
            path = _build.ensure_built()
            lib = ctypes.CDLL(path)
        except (OSError, _build.BuildError) as e:
            raise KernelLibraryError(
                f"the HIP kernel library is not available ({e}); this engine has no other "
                "implementation of its kernels") from e
        for name, argtypes in _SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError:
                continue        # optional entry points are checked where they are used
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        _lib = lib
        return lib


def declare(name: str, argtypes: list) -> None:
    """Adds an entry point's signature (kernel files added later register here)."""
    _SIGNATURES[name] = argtypes
    if _lib is not None and hasattr(_lib, name):
        fn = getattr(_lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int


def entry(name: str):
    lib = library()
    try:
        return getattr(lib, name)
    except AttributeError:
        raise KernelLibraryError(f"the kernel library has no entry point {name}") from None


_loaded_on: set = set()


def load_kernels() -> None:
    """Has the device code of every kernel file loaded onto the current device (the runtime would
    load a file's code at the first launch of one of its kernels, which must not happen while
    launches are being recorded into a graph). Cheap after the first call on a device."""
    device = torch.cuda.current_device()
    if device in _loaded_on:
        return
    import os
    for src in _build.sources():
        name = "llme_load_" + os.path.basename(src)[:-4]
        fn = entry(name)
        fn.argtypes, fn.restype = [], ctypes.c_int
        check(fn(), name)
    _loaded_on.add(device)


def code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, not {dtype}") from None


# The current stream's handle without the Stream object around it: asked for before every launch.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


def stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def check(status: int, what: str) -> None:
    if status != 0:
        if status == 10001:
            raise KernelError(f"{what}: the kernel refused its arguments")
        if status == 10002:
            raise KernelError(f"{what}: the kernel does not support this size")
        raise KernelError(f"{what}: HIP error {status}")


def require(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    """Host-side check of an operand before a launch: device, layout, type, shape."""
    # (called several times per launch: the passing case takes the short way)
    if type(t) is torch.Tensor and t.is_cuda and t.is_contiguous():
        if dtype is None or t.dtype is dtype or (type(dtype) is not torch.dtype and t.dtype in dtype):
            if shape is None:
                return
            have = t.shape
            if len(shape) == len(have):
                for s, d in zip(shape, have):
                    if s is not None and s != d:
                        break
                else:
                    return
    if not isinstance(t, torch.Tensor):
        raise KernelError(f"{name}: expected a tensor, got {type(t).__name__}")
    if t.device.type != "cuda":
        raise KernelError(f"{name}: must live on the GPU, is on {t.device}")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous")
    if dtype is not None:
        allowed = dtype if isinstance(dtype, (tuple, list)) else (dtype,)
        if t.dtype not in allowed:
            raise KernelError(f"{name}: dtype {t.dtype} not in {allowed}")
    if shape is not None:
        if len(shape) != t.dim() or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise KernelError(f"{name}: shape {tuple(t.shape)} does not match {tuple(shape)}")
