"""Reader and writer for the safetensors container.

Layout (reference: src/weights.cpp:151-242): 8 bytes little-endian header length
N, N bytes of JSON (`name -> {dtype, shape, data_offsets}`, plus an optional
`__metadata__`), then the raw tensor bytes; `data_offsets` count from the start
of the data section. The reader maps the file, checks every entry the way the
reference does (negative dims, overflow, offsets inside the data section, byte
count = numel * dtype size) and hands out tensors that alias the mapping.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Callable, Iterable, Mapping

import torch


class SafetensorsError(RuntimeError):
    pass


# safetensors dtype tag -> (torch dtype, bytes per element)
_DTYPES: dict[str, tuple[torch.dtype, int]] = {
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_TAGS = {v[0]: k for k, v in _DTYPES.items()}
_U64_MAX = (1 << 64) - 1


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: tuple[int, ...]
    begin: int          # offsets into the file's data section
    end: int
    file_index: int

    @property
    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n


class SafetensorsFile:
    def __init__(self, path: str, file_index: int = 0):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"safetensors file too small: {path}")
        self._fh = open(path, "rb")
        self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        (header_len,) = struct.unpack("<Q", self._map[:8])
        if header_len + 8 > size:
            raise SafetensorsError(f"safetensors header overruns file: {path}")
        try:
            header = json.loads(self._map[8:8 + header_len].decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"safetensors header is not valid JSON: {path} ({e})") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"safetensors header is not a JSON object: {path}")
        self.data_start = 8 + header_len
        data_bytes = size - self.data_start
        self.metadata = header.get("__metadata__") or {}
        self.entries: dict[str, TensorEntry] = {}
        for name, spec in header.items():
            if name == "__metadata__":
                continue
            try:
                tag, shape, offsets = spec["dtype"], spec["shape"], spec["data_offsets"]
            except (KeyError, TypeError):
                raise SafetensorsError(f"safetensors entry for {name} lacks dtype/shape/data_offsets") from None
            if tag not in _DTYPES:
                raise SafetensorsError(f"unsupported safetensors dtype {tag} for {name}")
            dtype, width = _DTYPES[tag]
            numel = 1
            for d in shape:
                if not isinstance(d, int) or d < 0:
                    raise SafetensorsError(f"safetensors negative shape dim for {name}")
                if d != 0 and numel > _U64_MAX // d:
                    raise SafetensorsError(f"safetensors numel overflow for {name}")
                numel *= d
            if numel > _U64_MAX // width:
                raise SafetensorsError(f"safetensors byte-count overflow for {name}")
            expected = numel * width
            if (not isinstance(offsets, list) or len(offsets) != 2
                    or not all(isinstance(o, int) and o >= 0 for o in offsets)
                    or offsets[1] < offsets[0] or offsets[1] > data_bytes):
                raise SafetensorsError(f"safetensors offsets out of range for {name}")
            actual = offsets[1] - offsets[0]
            if actual != expected:
                raise SafetensorsError(
                    f"safetensors byte-count mismatch for {name}: header says shape*dtype = "
                    f"{expected} bytes but data_offsets cover {actual}")
            self.entries[name] = TensorEntry(name, dtype, tuple(shape), offsets[0], offsets[1], file_index)

    def read(self, name: str) -> torch.Tensor:
        """A CPU tensor that aliases the mapping (read-only: copy before writing)."""
        e = self.entries[name]
        if e.numel == 0:
            return torch.empty(e.shape, dtype=e.dtype)
        buf = memoryview(self._map)[self.data_start + e.begin:self.data_start + e.end]
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")     # torch warns that the buffer is not writable
            flat = torch.frombuffer(buf, dtype=e.dtype)
        return flat.view(e.shape)

    def close(self) -> None:
        try:
            self._map.close()
        except BufferError:
            pass        # tensors that alias the mapping are still alive
        self._fh.close()


class TensorIndex:
    """Every tensor of every *.safetensors file directly in a model folder
    (sorted by file name; no index file is needed; src/weights.cpp:37-51,269-275)."""

    def __init__(self, model_dir: str):
        names = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
        if not names:
            raise SafetensorsError(f"no .safetensors files in {model_dir}")
        self.files = [SafetensorsFile(os.path.join(model_dir, n), i) for i, n in enumerate(names)]
        self.entries: dict[str, TensorEntry] = {}
        for f in self.files:
            self.entries.update(f.entries)

    def __contains__(self, name: str) -> bool:
        return name in self.entries

    def names(self) -> list[str]:
        return sorted(self.entries)

    def entry(self, name: str) -> TensorEntry:
        return self.entries[name]

    def read(self, name: str) -> torch.Tensor:
        return self.files[self.entries[name].file_index].read(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


def write_safetensors(path: str, specs: Mapping[str, tuple[torch.dtype, tuple[int, ...]]],
                      produce: Callable[[str], torch.Tensor],
                      metadata: Mapping[str, str] | None = None) -> None:
    """Writes tensors one at a time: `specs` fixes names, dtypes and shapes (the
    header needs all offsets first), `produce(name)` makes each tensor when its
    turn comes, so a model larger than memory can be written."""
    header: dict = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    order = list(specs)
    for name in order:
        dtype, shape = specs[name]
        if dtype not in _TAGS:
            raise SafetensorsError(f"cannot write dtype {dtype} for {name}")
        n = 1
        for d in shape:
            n *= d
        nbytes = n * _DTYPES[_TAGS[dtype]][1]
        header[name] = {"dtype": _TAGS[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + ".tmp"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            dtype, shape = specs[name]
            t = produce(name)
            if tuple(t.shape) != tuple(shape) or t.dtype != dtype:
                raise SafetensorsError(f"produced tensor {name} is {t.dtype}{tuple(t.shape)}, "
                                       f"header says {dtype}{tuple(shape)}")
            t = t.detach().contiguous().cpu()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else
                        t.reshape(1).view(torch.uint8).numpy().tobytes())
    os.replace(tmp, path)


def write_state_dict(path: str, tensors: Mapping[str, torch.Tensor],
                     metadata: Mapping[str, str] | None = None) -> None:
    specs = {k: (v.dtype, tuple(v.shape)) for k, v in tensors.items()}
    write_safetensors(path, specs, lambda name: tensors[name], metadata)
