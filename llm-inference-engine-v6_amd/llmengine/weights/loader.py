"""Loads a model's parameters from a folder of safetensors files, by tensor name.

The model tree says which names and shapes it reads; the files say what they
hold. Both lists are compared before anything is copied, and every problem is
reported in one error: missing tensors, unexpected tensors, wrong shapes (the
reference stops at the first one: "missing weight: <name>", "shape mismatch for
<name>: expected [..], got [..]", src/model.cpp:107-134; a transposed matrix has the
right element count and must still be refused).
"""
from __future__ import annotations

import torch

from ..parts.base import Part, Placement
from .safetensors_io import SafetensorsError, TensorIndex


class WeightError(RuntimeError):
    def __init__(self, message: str, missing=(), unexpected=(), wrong_shape=()):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)


def _fmt(shape) -> str:
    return "[" + ",".join(str(int(d)) for d in shape) + "]"


def check_names(model: Part, available: dict[str, tuple[int, ...]], where: str) -> None:
    """Raises one WeightError that lists every missing, unexpected and wrongly shaped tensor."""
    expected = model.named_specs()
    ignored = model.named_ignored()
    missing = sorted(n for n in expected if n not in available)
    unexpected = sorted(n for n in available if n not in expected and n not in ignored)
    wrong = sorted((n, expected[n].shape, available[n]) for n in expected
                   if n in available and tuple(available[n]) != tuple(expected[n].shape))
    if not (missing or unexpected or wrong):
        return
    lines = [f"weights in {where} do not fit the model:"]
    for n in missing:
        lines.append(f"  missing weight: {n} (expected shape {_fmt(expected[n].shape)})")
    for n, want, got in wrong:
        lines.append(f"  shape mismatch for {n}: expected {_fmt(want)}, got {_fmt(got)}")
    for n in unexpected:
        lines.append(f"  unexpected tensor: {n} {_fmt(available[n])}")
    raise WeightError("\n".join(lines), missing, unexpected, [w[0] for w in wrong])


def load_model_weights(model: Part, model_dir: str, placement: Placement) -> list[str]:
    """Fills the model's parts from the folder's tensors; returns the tensor names read."""
    index = TensorIndex(model_dir)
    try:
        check_names(model, {n: index.entry(n).shape for n in index.names()}, model_dir)
        read: list[str] = []

        def get(name: str) -> torch.Tensor:
            read.append(name)
            return index.read(name)

        model.load_tree(get, placement)
        if placement.device.type == "cuda":
            torch.cuda.synchronize(placement.device)     # copies out of the mapping are done
        return read
    finally:
        index.close()


def load_state_dict(model: Part, tensors: dict[str, torch.Tensor], placement: Placement) -> None:
    """The same from tensors in memory (random weights that are never written out)."""
    check_names(model, {n: tuple(t.shape) for n, t in tensors.items()}, "the given tensors")
    model.load_tree(lambda name: tensors[name], placement)
