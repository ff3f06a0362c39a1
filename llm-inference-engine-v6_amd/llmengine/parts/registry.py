"""Registries of part kinds, so that a layer is data: names of kinds plus their
arguments (`LayerSpec`), chosen by the configuration layer by layer."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Mapping

_KINDS: dict[str, dict[str, Callable[..., Any]]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(kind: str, name: str, factory: Callable[..., Any], replace: bool = False) -> None:
    if kind not in _KINDS:
        raise ValueError(f"unknown kind of part {kind!r}; kinds: {sorted(_KINDS)}")
    if name in _KINDS[kind] and not replace:
        raise ValueError(f"{kind} {name!r} is already registered")
    _KINDS[kind][name] = factory


def make_part(kind: str, name: str, **args: Any) -> Any:
    try:
        factory = _KINDS[kind][name]
    except KeyError:
        raise ValueError(f"no {kind} named {name!r}; registered: {sorted(_KINDS.get(kind, {}))}") from None
    return factory(**args)


def registered(kind: str) -> list[str]:
    return sorted(_KINDS[kind])


@dataclass(frozen=True)
class PartChoice:
    name: str
    args: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer as data: which arrangement, mixer, feed-forward and norms, with
    their sizes. `position` is handed to the mixer as its position encoding."""
    block: PartChoice
    mixer: PartChoice
    feed_forward: PartChoice
    mixer_norm: PartChoice
    ffn_norm: PartChoice
    position: PartChoice | None = None


def build_layer(spec: LayerSpec, shared_positions: dict | None = None):
    """Instantiates the parts of a layer. Position encodings with equal choices are
    shared between layers through `shared_positions` (one table on the device)."""
    position = None
    if spec.position is not None:
        key = (spec.position.name, tuple(sorted((k, repr(v)) for k, v in spec.position.args.items())))
        if shared_positions is not None and key in shared_positions:
            position = shared_positions[key]
        else:
            position = make_part("position", spec.position.name, **spec.position.args)
            if shared_positions is not None:
                shared_positions[key] = position
    mixer_args = dict(spec.mixer.args)
    if position is not None:
        mixer_args["position"] = position
    return make_part(
        "block", spec.block.name,
        mixer=make_part("mixer", spec.mixer.name, **mixer_args),
        feed_forward=make_part("feed_forward", spec.feed_forward.name, **spec.feed_forward.args),
        mixer_norm=make_part("norm", spec.mixer_norm.name, **spec.mixer_norm.args),
        ffn_norm=make_part("norm", spec.ffn_norm.name, **spec.ffn_norm.args),
        **spec.block.args)
