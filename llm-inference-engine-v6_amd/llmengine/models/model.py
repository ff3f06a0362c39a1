"""A decoder as data: an embedding, a list of layers, the order in which the layers
run, a final norm and an output head. Nothing here names an architecture.

The order is a list of `LayerCall`s. A call names the layer to run and the cache it
works on; by default layer i runs once on cache i. A layer may be named twice, and
a call may read a cache that another call wrote (`write_cache=False`), so layers
that share keys and values, or a stack that is run twice, are a schedule and not
new model code.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from ..parts.base import Block, CacheSpec, Head, Norm, Part, TokenEmbedding


@dataclass(frozen=True)
class LayerCall:
    layer: int
    cache: int | None = None        # cache id; None: the layer's own (its index)
    write_cache: bool = True

    @property
    def cache_id(self) -> int:
        return self.layer if self.cache is None else self.cache


class DecoderModel(Part):
    graph_safe = True

    def __init__(self, config, embedding: TokenEmbedding, layers: list[Block], final_norm: Norm,
                 head: Head, schedule: list[LayerCall] | None = None, names: dict | None = None):
        self.config = config
        self.embedding, self.layers, self.final_norm, self.head = embedding, list(layers), final_norm, head
        self.schedule = list(schedule) if schedule is not None else [LayerCall(i) for i in range(len(layers))]
        for call in self.schedule:
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"schedule names layer {call.layer}, the model has {len(self.layers)}")
        self.names = {"embedding": "model.embed_tokens", "layers": "model.layers", "final_norm": "model.norm",
                      "head": "lm_head"}
        if names:
            self.names.update(names)

    # ---- parameters ----
    def children(self):
        n = self.names
        out: dict[str, Part] = {n["embedding"]: self.embedding}
        for i, layer in enumerate(self.layers):
            out[f"{n['layers']}.{i}"] = layer
        out[n["final_norm"]] = self.final_norm
        out[n["head"]] = self.head
        return out

    def aliases(self):
        # A tied head is the embedding table under a second name (src/weights.cpp:244-267): a
        # checkpoint may store it under both, and then both must agree in shape and type.
        if getattr(self.head, "tied_to", None) is self.embedding:
            return {f"{self.names['head']}.weight": f"{self.names['embedding']}.weight"}
        return {}

    # ---- caches ----
    def cache_specs(self) -> dict[int, CacheSpec | None]:
        """cache id -> what is kept there: the spec of the first call that writes it."""
        specs: dict[int, CacheSpec | None] = {}
        for call in self.schedule:
            if call.write_cache and call.cache_id not in specs:
                specs[call.cache_id] = self.layers[call.layer].mixer.cache_spec()
        for call in self.schedule:
            if call.cache_id not in specs:
                raise ValueError(f"layer {call.layer} reads cache {call.cache_id}, which no layer writes")
        return specs

    @property
    def vocab_size(self) -> int:
        return self.head.vocab_size

    @property
    def hidden_size(self) -> int:
        return self.embedding.hidden_size

    def decode_plan_hints(self, lens: list[int], plan_len: int, choices) -> tuple:
        """What of the layers' launch plans for a step of single decoded tokens depends on the requests'
        lengths: the mixers' hints (Mixer.decode_plan_hint), each name once, in a fixed order."""
        hints: dict = {}
        asked = set()
        for call in self.schedule:
            mixer = getattr(self.layers[call.layer], "mixer", None)
            if mixer is None or id(mixer) in asked:
                continue
            asked.add(id(mixer))
            sig = getattr(mixer, "plan_signature", None)
            if sig is not None:
                if sig in asked:
                    continue
                asked.add(sig)
            hint = mixer.decode_plan_hint(lens, plan_len, choices)
            if hint is not None:
                hints[hint[0]] = hint[1]
        return tuple(sorted(hints.items()))

    # ---- the forward pass of one step ----
    def forward(self, step, caches, logit_rows: torch.Tensor | None) -> torch.Tensor | None:
        """Runs the step's tokens through the schedule; returns 32-bit logits
        [len(logit_rows), vocab] for the wanted rows (None if none is wanted)."""
        T = step.num_tokens
        h = step.buffer("model.hidden", (T, self.hidden_size), torch.float32)
        self.embedding.forward(step.tokens, h, step)
        for call in self.schedule:
            self.layers[call.layer].forward(h, step, caches[call.cache_id], call.write_cache)
        if logit_rows is None or logit_rows.shape[0] == 0:
            return None
        R = logit_rows.shape[0]
        logits = step.buffer("model.logits", (R, self.vocab_size), torch.float32)
        if self.head.fuses_norm(h, self.final_norm, R, step):
            self.head.forward_normed_rows(h, logit_rows, self.final_norm, logits, step)
        else:
            x = step.buffer("model.head_in", (R, self.hidden_size), step.act_dtype)
            self.final_norm.forward(h, x, rows=logit_rows)
            self.head.forward(x, logits, step)
        return logits
