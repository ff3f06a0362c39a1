"""SiLU-gated feed-forward: down( silu(gate(x)) * up(x) ), no biases
(src/engine.cpp:213-217, src/kernels.cpp:26-31).

Gate and up rows are stored interleaved in groups of 16 in one matrix, so that one
product yields both and a 16-column group of its output holds the gate and the up
value of the same 16 units next to each other.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import FeedForward, Getter, ParamSpec, Placement
from .registry import register_part


class GatedMLP(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.group = 16 if self.intermediate_size % 16 == 0 else self.intermediate_size
        self.w_gate_up: torch.Tensor | None = None
        self.w_down: torch.Tensor | None = None

    def param_specs(self):
        H, FF = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": ParamSpec((FF, H)), "up_proj.weight": ParamSpec((FF, H)),
                "down_proj.weight": ParamSpec((H, FF))}

    def load_params(self, get: Getter, placement: Placement) -> None:
        H, FF, g = self.hidden_size, self.intermediate_size, self.group
        gate, up = get("gate_proj.weight"), get("up_proj.weight")
        dtype = placement.common_dtype([gate, up])
        fused = torch.empty((2 * FF, H), dtype=dtype, device=placement.device)
        view = fused.view(FF // g, 2, g, H)
        view[:, 0].copy_(gate.view(FF // g, g, H))
        view[:, 1].copy_(up.view(FF // g, g, H))
        self.w_gate_up = placement.matrix(fused)
        self.w_down = placement.place_matrix(get("down_proj.weight"))

    def fuses_norm(self, h, norm, step):
        # A few rows (decoding): one kernel applies the norm, both projections and the activation.
        rms = norm.fused_rms()
        return (rms is not None and self.group == 16 and step.act_dtype == torch.bfloat16
                and ops.gemv_norm_supported(h, rms[0], self.w_gate_up, h.shape[0], gated=True, choices=step.choices))

    def forward(self, x, step, out, accumulate, pre_norm=None):
        T = x.shape[0]
        FF = self.intermediate_size
        if pre_norm is not None:
            act = step.buffer("mlp.act", (T, FF), torch.bfloat16)
            weight, eps = pre_norm.fused_rms()
            ops.gemv_norm(x, weight, eps, self.w_gate_up, act, gated=True)
        else:
            act = step.buffer("mlp.act", (T, FF), x.dtype)
            ops.gemm_gated(x, self.w_gate_up, act, self.group,
                           lambda shape, dtype: step.buffer("mlp.gate_up", shape, dtype), choices=step.choices)
        ops.gemm(act, self.w_down, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)


register_part("feed_forward", "gated_mlp", GatedMLP)
