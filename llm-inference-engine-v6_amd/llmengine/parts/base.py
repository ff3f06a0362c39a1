"""Interfaces of the parts a model is put together from.

A part owns its sizes and constants (constructor arguments), names the tensors it
reads from a checkpoint (`param_specs`), places them on the device in the layout
its kernels want (`load_params`) and runs on a step's flat batch (`forward`). No
part knows which model it is in: names under which a model stores a part's
tensors are given by whoever composes the parts.

Kinds of parts and what each must provide:

* `Norm`:      forward(x32 [T, H], out [R, H], rows=None)
* `PositionEncoding`: rotary_tables() -> (cos, sin, rotary_dim) or None, and
               apply(q, k, positions) for encodings that are not rotary tables
* `Mixer`:     cache_spec(), forward(x [T, H], step, cache, out32 [T, H], accumulate,
               write_cache)
* `FeedForward`: forward(x [T, H], step, out32 [T, H], accumulate)
* `Block`:     the arrangement of the four above around the 32-bit residual stream:
               forward(h32 [T, H], step, cache, write_cache)
* `TokenEmbedding`: forward(tokens [T] int32, out32 [T, H], step): the stream's first value
* `Head`:      forward(x [R, H], out32 [R, V], step) on normed rows; optionally
               fuses_norm(h32, norm, n_rows, step) / forward_normed_rows(h32, rows, norm, out32, step)

`step` is the engine's `StepContext` (tokens, positions, request index per token,
block tables, slots, scratch buffers); `cache` is the `LayerCache` that the cache
manager made from the mixer's `cache_spec`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Mapping

import torch


@dataclass(frozen=True)
class ParamSpec:
    """A tensor a part reads from the checkpoint: its exact shape there, and how a
    random model fills it ("linear": N(0, std); "norm": N(mean, std) around one)."""
    shape: tuple[int, ...]
    init: str = "linear"


@dataclass(frozen=True)
class Placement:
    """Where parameters live and in which precision the model computes."""
    device: torch.device
    compute_dtype: torch.dtype          # torch.float32 or torch.bfloat16

    def storage_dtype(self, stored: torch.dtype) -> torch.dtype:
        """A tensor's dtype on the device, given its dtype in the file. The 32-bit
        model widens everything; the bfloat16 model keeps bfloat16 tensors as they
        are and leaves tensors stored in 32-bit (or half, widened exactly) in
        32-bit; integer tables become int32."""
        if stored in (torch.int32, torch.int64):
            return torch.int32
        if self.compute_dtype == torch.float32:
            return torch.float32
        return torch.bfloat16 if stored == torch.bfloat16 else torch.float32

    def place(self, t: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
        dtype = dtype or self.storage_dtype(t.dtype)
        return t.to(device=self.device, dtype=dtype).contiguous()

    def matrix(self, w: torch.Tensor) -> torch.Tensor:
        """A weight matrix [N, K] that is already on the device, in the layout the matrix kernels
        stream fastest: blocked (a 5-d tensor, see ops.block_weight) where its type and sizes
        allow, otherwise as it is."""
        from .. import ops
        return ops.block_weight(w) if ops.can_block(w) else w

    def place_matrix(self, t: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
        return self.matrix(self.place(t, dtype))

    def common_dtype(self, tensors: list[torch.Tensor]) -> torch.dtype:
        """The storage dtype of a buffer that fuses several checkpoint tensors."""
        kinds = {self.storage_dtype(t.dtype) for t in tensors}
        return kinds.pop() if len(kinds) == 1 else torch.float32


Getter = Callable[[str], torch.Tensor]      # local tensor name -> CPU tensor as stored


class Part:
    # True if, for a step of one token of each request that wants its logits, forward() issues the
    # same launches with the same arguments whatever the requests are, reading what changes (tokens,
    # positions, tables, slots) from the step's device arrays only and never from its host-side
    # lists. Such steps are recorded once as a HIP graph and replayed. The step is recorded without
    # being run (the first replay is its first run), so it may advance state of its own. Tensors
    # that forward() makes while it is recorded belong to the recording; scratch memory from
    # `step.buffer` is the runner's.
    graph_safe = False

    def param_specs(self) -> dict[str, ParamSpec]:
        return {}

    def children(self) -> dict[str, "Part"]:
        """Sub-parts by the name prefix under which their tensors are stored."""
        return {}

    def ignored_names(self) -> set[str]:
        """Tensor names that a checkpoint may hold for this part and that are not read."""
        return set()

    def aliases(self) -> dict[str, str]:
        """Second names of tensors of this part: alias -> the name whose tensor it is (both
        relative to this part). A checkpoint may store an alias too; it is then not read, but its
        shape and type must agree with the tensor it stands for."""
        return {}

    def load_params(self, get: Getter, placement: Placement) -> None:
        """Reads the part's own tensors (children are loaded by the walker)."""

    def refusals(self) -> list[str]:
        """Sizes of this part that no kernel takes, each as a sentence that names the argument; asked
        when a runner is made, before any tensor is read, so that such a model is refused with the
        name of the size and not at its first step."""
        return []

    def tree_refusals(self, prefix: str = "") -> list[str]:
        out = [f"{prefix.rstrip('.') or 'model'}: {r}" for r in self.refusals()]
        for name, child in self.children().items():
            out += child.tree_refusals(f"{prefix}{name}.")
        return out

    # ---- walking a tree of parts ----
    def named_specs(self, prefix: str = "") -> dict[str, ParamSpec]:
        out = {prefix + k: v for k, v in self.param_specs().items()}
        for name, child in self.children().items():
            out.update(child.named_specs(f"{prefix}{name}."))
        return out

    def named_ignored(self, prefix: str = "") -> set[str]:
        out = {prefix + k for k in self.ignored_names()}
        for name, child in self.children().items():
            out |= child.named_ignored(f"{prefix}{name}.")
        return out

    def named_aliases(self, prefix: str = "") -> dict[str, str]:
        out = {prefix + a: prefix + t for a, t in self.aliases().items()}
        for name, child in self.children().items():
            out.update(child.named_aliases(f"{prefix}{name}."))
        return out

    def tree_graph_safe(self) -> bool:
        return bool(self.graph_safe) and all(c.tree_graph_safe() for c in self.children().values())

    def load_tree(self, get: Getter, placement: Placement, prefix: str = "") -> None:
        self.load_params(lambda local: get(prefix + local), placement)
        for name, child in self.children().items():
            child.load_tree(get, placement, f"{prefix}{name}.")


# --- what a mixer keeps between steps ---------------------------------------------------
PAGE = -1       # placeholder for the page size in a paged tensor's shape


@dataclass(frozen=True)
class CacheSpec:
    """What one mixer keeps for a request.

    paged: tensors kept per token, in pages: name -> shape of one page, with `PAGE`
           where the page size goes, or (shape, dtype) for a tensor that is not kept in
           the model's activation type. Layers with the same (kind, window) share a
           page pool and a block table (one page id covers all of them).
    kind:  "full": every token of the request stays; "window": only the last
           `window` tokens are ever read, pages behind them are given back.
    state: tensors of fixed size per request: name -> (shape, dtype), kept in the
           request's slot, zero when the request is admitted.
    """
    kind: str = "full"
    window: int = 0
    paged: Mapping[str, tuple] = field(default_factory=dict)
    state: Mapping[str, tuple[tuple[int, ...], torch.dtype]] = field(default_factory=dict)

    def __post_init__(self):
        if self.kind not in ("full", "window"):
            raise ValueError(f"cache kind {self.kind!r} is not 'full' or 'window'")
        if self.kind == "window" and self.window <= 0:
            raise ValueError("a window cache needs window > 0")

    def paged_tensors(self, default_dtype: torch.dtype) -> dict[str, tuple[tuple[int, ...], torch.dtype]]:
        """name -> (shape of one page, dtype), the model's activation type where none is given."""
        out = {}
        for name, value in self.paged.items():
            if len(value) == 2 and isinstance(value[1], torch.dtype):
                out[name] = (tuple(value[0]), value[1])
            else:
                out[name] = (tuple(value), default_dtype)
        return out

    @property
    def group_key(self) -> tuple:
        return (self.kind, self.window if self.kind == "window" else 0)


@dataclass
class LayerCache:
    """The device tensors of one mixer's cache, as the mixer sees them in a step."""
    paged: dict[str, torch.Tensor]          # name -> [num_pages, *page shape]
    state: dict[str, torch.Tensor]          # name -> [num_slots, *shape]
    page_size: int
    group: str | None                       # key into StepContext.block_tables


class Norm(Part):
    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
        raise NotImplementedError

    def fused_rms(self) -> tuple[torch.Tensor, float] | None:
        """(weight, eps) if this norm is exactly y = weight * x / sqrt(mean(x^2) + eps), so that a
        kernel which applies that formula in front of a projection may stand in for `forward`;
        None (the default) for every other formula: the norm then always runs as its own step."""
        return None


class PositionEncoding(Part):
    def rotary_tables(self):
        """(cos [P, r/2], sin [P, r/2], r) for rotate-half pairs (i, i + r/2): the mixer's kernels
        rotate q and k by them. None: the encoding is something else and transforms q and k itself
        in `apply`."""
        return None

    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """For encodings without rotary tables: transforms, in place, the step's projected queries
        q [T, n_q, hd] and keys k [T, n_kv, hd] (32-bit views, rows in batch order; k is None for a
        layer that reads another layer's keys) for the tokens at `positions` [T] (int32, on the
        device). Keys are cached as this leaves them. A part that computes on the host here must
        leave `graph_safe` False."""
        raise NotImplementedError(f"{type(self).__name__} has neither rotary tables nor apply()")

    @property
    def max_position(self) -> int:
        raise NotImplementedError


class Mixer(Part):
    def cache_spec(self) -> CacheSpec | None:
        return None

    def fuses_norm(self, h: torch.Tensor, norm: "Norm", step) -> bool:
        """True if, for this step, the part wants the un-normed 32-bit stream plus the norm in
        front of it (`forward(h, ..., pre_norm=norm)`) because a kernel of its own applies the
        norm. Parts that do not know about this are always given normed activations."""
        return False

    def decode_round(self) -> int:
        """After how many requests of a step of single decoded tokens the part's kernel has given every
        compute unit one piece of work, where it deals the requests out in turn (a scheduler that knows
        this can put long and short requests together); 0: no such number."""
        return 0

    def decode_plan_hint(self, lens: list[int], plan_len: int, choices) -> tuple | None:
        """For a step of single decoded tokens that is recorded once and replayed: what of the part's launch
        plan depends on the requests' lengths (lens: the keys each sees, in the step's order; plan_len: the
        length the recording is made for), as a pair (name of the plan, value), both hashable. The runner
        keeps one recording per value and hands the pair back in `step.plan_hints[name]` when it records.
        None: the part's launches depend on nothing but the step's shape."""
        return None

    def forward(self, x: torch.Tensor, step, cache: LayerCache | None, out: torch.Tensor,
                accumulate: bool, write_cache: bool = True) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def fuses_norm(self, h: torch.Tensor, norm: "Norm", step) -> bool:
        return False

    def forward(self, x: torch.Tensor, step, out: torch.Tensor, accumulate: bool) -> None:
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, h: torch.Tensor, step, cache: LayerCache | None, write_cache: bool = True) -> None:
        raise NotImplementedError


class TokenEmbedding(Part):
    """Token ids to the first value of the 32-bit residual stream. `vocab_size` and `hidden_size`
    are attributes. An embedding whose table an output head may share (tied weights) keeps it as
    `weight`, a matrix [vocab, hidden] in a layout that `ops.gemm` reads."""
    vocab_size: int
    hidden_size: int
    weight: torch.Tensor | None = None

    def forward(self, tokens: torch.Tensor, out: torch.Tensor, step=None) -> None:
        """out [T, H] (32-bit) = the rows of tokens [T] (int32, on the device), with whatever
        multiplier the architecture has."""
        raise NotImplementedError


class Head(Part):
    """The normed last rows of the stream to 32-bit logits. `vocab_size` is an attribute."""
    vocab_size: int

    def forward(self, x: torch.Tensor, out: torch.Tensor, step=None) -> None:
        """out [R, V] (32-bit) from x [R, H], rows that the final norm has been applied to."""
        raise NotImplementedError

    def fuses_norm(self, h: torch.Tensor, norm: "Norm", n_rows: int, step) -> bool:
        """True if, for `n_rows` wanted rows of this step, the head wants the un-normed 32-bit stream
        h [T, H] and applies `norm` itself in `forward_normed_rows` (a kernel of its own does both).
        The default never does: the model then norms the wanted rows and calls `forward`."""
        return False

    def forward_normed_rows(self, h: torch.Tensor, rows: torch.Tensor, norm: "Norm", out: torch.Tensor,
                            step=None) -> None:
        """out [R, V] = head(norm(h[rows])), rows [R] int32 on the device. Only called after
        `fuses_norm` said yes for the same step."""
        raise NotImplementedError
