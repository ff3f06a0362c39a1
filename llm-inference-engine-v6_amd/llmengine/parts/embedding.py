"""Token embedding and output head.

Embedding: h = E[token] with no multiplier (src/kernels.cpp:59-66). Head:
logits = x . W^T in 32-bit (src/engine.cpp:242-249); a tied head is the embedding
table itself, one buffer under two names (src/weights.cpp:244-267, src/model.cpp:185-190).
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Getter, Head, ParamSpec, Placement, TokenEmbedding
from .registry import register_part


class Embedding(TokenEmbedding):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight: torch.Tensor | None = None

    def param_specs(self):
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size), "linear")}

    def load_params(self, get: Getter, placement: Placement) -> None:
        # (a tied head reads the table as a weight matrix: the gather takes either layout)
        self.weight = placement.place_matrix(get("weight"))

    def forward(self, tokens: torch.Tensor, out: torch.Tensor, step=None) -> None:
        ops.embed_gather(self.weight, tokens, out)


class OutputHead(Head):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied_to: TokenEmbedding | None = None):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tied_to = tied_to
        self._weight: torch.Tensor | None = None

    def param_specs(self):
        if self.tied_to is not None:
            return {}
        return {"weight": ParamSpec((self.vocab_size, self.hidden_size), "linear")}

    def load_params(self, get: Getter, placement: Placement) -> None:
        if self.tied_to is None:
            self._weight = placement.place_matrix(get("weight"))

    @property
    def weight(self) -> torch.Tensor:
        return self.tied_to.weight if self.tied_to is not None else self._weight

    def fuses_norm(self, h: torch.Tensor, norm, n_rows: int, step) -> bool:
        rms = norm.fused_rms()
        return (rms is not None and step.act_dtype == torch.bfloat16
                and ops.gemv_norm_supported(h, rms[0], self.weight, n_rows, gated=False, choices=step.choices))

    def forward(self, x: torch.Tensor, out: torch.Tensor, step=None) -> None:
        ops.gemm(x, self.weight, out, choices=getattr(step, "choices", None))

    def forward_normed_rows(self, h: torch.Tensor, rows: torch.Tensor, norm, out: torch.Tensor, step=None) -> None:
        """Logits of the chosen rows of the 32-bit stream, the final norm applied inside the product."""
        weight, eps = norm.fused_rms()
        ops.gemv_norm(h, weight, eps, self.weight, out, rows=rows)


register_part("embedding", "table", Embedding)
register_part("head", "linear", OutputHead)
