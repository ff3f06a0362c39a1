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


def check_names(model: Part, available: dict[str, tuple[int, ...]], where: str, dtypes: dict | None = None) -> None:
    """Raises one WeightError that lists every missing, unexpected and wrongly shaped tensor.
    A tensor stored under a second name of another (a tied output head, src/weights.cpp:259-264)
    must agree with that tensor in shape and, where `dtypes` (name -> stored type) is given, type."""
    expected = model.named_specs()
    ignored = model.named_ignored()
    aliases = model.named_aliases()
    missing = sorted(n for n in expected if n not in available)
    unexpected = sorted(n for n in available if n not in expected and n not in ignored and n not in aliases)
    wrong = sorted((n, expected[n].shape, available[n]) for n in expected
                   if n in available and tuple(available[n]) != tuple(expected[n].shape))
    disagree = sorted((a, t) for a, t in aliases.items() if a in available and t in available and (
        tuple(available[a]) != tuple(available[t]) or (dtypes is not None and dtypes.get(a) != dtypes.get(t))))
    if not (missing or unexpected or wrong or disagree):
        return
    lines = [f"weights in {where} do not fit the model:"]
    for a, t in disagree:
        what = "tie_word_embeddings=true but " if a.endswith("lm_head.weight") else ""
        lines.append(f"  {what}{a} shape/dtype disagrees with {t} ({_fmt(available[a])}"
                     f"{' ' + str(dtypes[a]) if dtypes else ''} against {_fmt(available[t])}"
                     f"{' ' + str(dtypes[t]) if dtypes else ''})")
    for n in missing:
        lines.append(f"  missing weight: {n} (expected shape {_fmt(expected[n].shape)})")
    for n, want, got in wrong:
        lines.append(f"  shape mismatch for {n}: expected {_fmt(want)}, got {_fmt(got)}")
    for n in unexpected:
        lines.append(f"  unexpected tensor: {n} {_fmt(available[n])}")
    raise WeightError("\n".join(lines), missing, unexpected, [w[0] for w in wrong] + [a for a, _ in disagree])


def load_model_weights(model: Part, model_dir: str, placement: Placement) -> list[str]:
    """Fills the model's parts from the folder's tensors; returns the tensor names read."""
    index = TensorIndex(model_dir)
    try:
        check_names(model, {n: index.entry(n).shape for n in index.names()}, model_dir,
                    {n: index.entry(n).dtype for n in index.names()})
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
    check_names(model, {n: tuple(t.shape) for n, t in tensors.items()}, "the given tensors",
                {n: t.dtype for n, t in tensors.items()})
    model.load_tree(lambda name: tensors[name], placement)
