"""Grouped-query attention over the paged cache.

q, k, v = x Wq^T, x Wk^T, x Wv^T without biases; head j is the slice
[j hd, (j+1) hd); q and k are rotated at the token's position and k is cached after
rotation, v as it is (src/engine.cpp:142-170); query head h reads kv head
h / (n_q / n_kv); scores scale by head_dim^-1/2, softmax over the keys up to the
token's own position (src/kernels.cpp:413-474); out = concat(heads) Wo^T
(src/engine.cpp:193-194).

The three projections are one product against the row-concatenated matrix. The
step's own keys and values go into the pages first, then every token reads pages
only: whole prompts, portions with earlier context and single decoded tokens are
the same case. `window` > 0 restricts a token at position p to keys > p - window.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import PAGE, CacheSpec, Getter, Mixer, ParamSpec, Placement, PositionEncoding
from .registry import register_part


class Attention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position: PositionEncoding | None = None, scale: float | None = None, window: int = 0):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} key/value heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        self.position = position
        self.scale = float(scale) if scale is not None else float(head_dim) ** -0.5
        self.window = int(window)
        # (layers with the same head counts have the same launch plans: a model asks one of them)
        self.plan_signature = ("attention", int(num_heads), int(num_kv_heads), int(head_dim))
        self.q_dim = self.num_heads * self.head_dim
        self.kv_dim = self.num_kv_heads * self.head_dim
        self.w_qkv: torch.Tensor | None = None
        self.w_qkv_paired: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None

    def param_specs(self):
        H = self.hidden_size
        return {"q_proj.weight": ParamSpec((self.q_dim, H)), "k_proj.weight": ParamSpec((self.kv_dim, H)),
                "v_proj.weight": ParamSpec((self.kv_dim, H)), "o_proj.weight": ParamSpec((H, self.q_dim))}

    def load_params(self, get: Getter, placement: Placement) -> None:
        if self.position is not None and hasattr(self.position, "materialize"):
            self.position.materialize(placement)
        parts = [get("q_proj.weight"), get("k_proj.weight"), get("v_proj.weight")]
        dtype = placement.common_dtype(parts)
        fused = torch.empty((self.q_dim + 2 * self.kv_dim, self.hidden_size), dtype=dtype,
                            device=placement.device)
        row = 0
        for p in parts:
            fused[row:row + p.shape[0]].copy_(p)
            row += p.shape[0]
        # (queries alone are sliced off for layers that read another layer's cache: whole row groups)
        self.w_qkv = placement.matrix(fused) if self.q_dim % 16 == 0 else fused
        # A second copy for decoding, where norm, projection, rotation and cache write are one kernel:
        # that kernel wants each rotation pair inside one group of 16 rows (ops.pair_rows_for_rotation).
        # It costs the matrix's memory once more and no traffic: a step reads one copy or the other.
        self.w_qkv_paired = None
        rotary = self.position.rotary_tables() if self.position is not None and hasattr(self.position, "rotary_tables") else None
        if (fused.dtype == torch.bfloat16 and self.head_dim % 16 == 0 and rotary is not None
                and rotary[2] == self.head_dim):
            self.w_qkv_paired = placement.matrix(
                ops.pair_rows_for_rotation(fused, self.num_heads + self.num_kv_heads, self.head_dim))
        self.w_o = placement.place_matrix(get("o_proj.weight"))

    def refusals(self):
        if self.head_dim > ops.ATTENTION_MAX_HEAD_DIM:
            return [f"head_dim={self.head_dim}: the attention kernels take head sizes up to {ops.ATTENTION_MAX_HEAD_DIM}"]
        return []

    def tree_graph_safe(self) -> bool:
        # (the position encoding is no child with tensors of its own, but it runs inside forward)
        return super().tree_graph_safe() and (self.position is None or self.position.tree_graph_safe())

    def cache_spec(self) -> CacheSpec:
        return CacheSpec(kind="window" if self.window > 0 else "full", window=self.window,
                         paged={"k": (self.num_kv_heads, PAGE, self.head_dim),
                                "v": (self.num_kv_heads, self.head_dim, PAGE)})

    def decode_round(self) -> int:
        # the decode kernels have a workgroup per request, kv head and 16 query heads of it, and workgroups
        # go to the compute units in turn
        tiles = self.num_kv_heads * ((self.num_heads // self.num_kv_heads + 15) // 16)
        return max(1, ops.mfma.compute_units() // tiles)

    def decode_plan_hint(self, lens, plan_len, choices):
        # (only the bfloat16 kernels on the matrix cores cut their keys by a plan)
        if (self.w_qkv is None or self.w_qkv.dtype != torch.bfloat16 or self.head_dim > 128 or self.head_dim % 16
                or (choices is not None and not choices.fast_attention)):
            return None
        n = ops.mfma.decode_cut(lens, self.num_heads, self.num_kv_heads, self.head_dim, plan_len, choices)
        return None if n is None else (ops.mfma.cut_hint_name(self.num_heads, self.num_kv_heads, self.head_dim), n)

    def fuses_norm(self, h, norm, step):
        # A few rows (decoding): the q/k/v projection applies the norm itself.
        rms = norm.fused_rms()
        return (rms is not None and step.act_dtype == torch.bfloat16
                and ops.gemv_norm_supported(h, rms[0], self.w_qkv, h.shape[0], gated=False, choices=step.choices))

    def forward(self, x, step, cache, out, accumulate, write_cache=True, pre_norm=None):
        """pre_norm: the norm in front of this mixer when `fuses_norm` said yes; x is then the
        un-normed 32-bit stream and the projection applies pre_norm.fused_rms() itself."""
        T = x.shape[0]
        n_q, n_kv, hd = self.num_heads, self.num_kv_heads, self.head_dim
        tables = self.position.rotary_tables() if self.position is not None else None
        cos, sin, rot = tables if tables is not None else (None, None, 0)
        # an encoding that is no rotation by a table of angles transforms q and k itself
        applies = self.position is not None and tables is None
        if cos is not None and step.max_position >= cos.shape[0]:
            raise ValueError(f"position {step.max_position} is beyond the position table ({cos.shape[0]} rows)")
        block_table = step.block_tables[cache.group]
        k_cache, v_cache = cache.paged["k"], cache.paged["v"]
        act = step.act_dtype
        q = step.buffer("attn.q", (T, self.q_dim), act)
        rms = pre_norm.fused_rms() if pre_norm is not None else None
        sum_rows = ops.mfma.qkv_sum_max_rows(T == step.num_seqs and rot == hd and not applies, hd, step.choices)

        def project(weight, dst):
            if rms is not None:
                ops.gemv_norm(x, rms[0], rms[1], weight, dst)
            else:
                ops.gemm(x, weight, dst, choices=step.choices)
        if (write_cache and rms is not None and cos is not None and self.w_qkv_paired is not None
                and ops.gemv_norm_rope_supported(x, rms[0], self.w_qkv_paired, k_cache, T, hd, rot, step.choices)):
            # decoding: norm, projection, rotation and the cache write are one kernel
            ops.gemv_norm_rope(x, rms[0], rms[1], self.w_qkv_paired, step.positions, step.seq_idx,
                               block_table, cos, sin, q, k_cache, v_cache, n_q, n_kv, hd)
        elif (write_cache and rms is None and T > sum_rows and cos is not None
              and ops.gemm_qkv_rope_supported(x, self.w_qkv, k_cache, hd, rot, step.choices)):
            # many rows (prompts): rotation and the cache write are the projection's epilogue
            ops.gemm_qkv_rope(x, self.w_qkv, cos, sin, step.positions, step.seq_idx, block_table, q, k_cache, v_cache,
                              n_q, n_kv, hd)
        elif write_cache:
            adds = (rms is None and ops.mfma.GEMV_NORM_MAX_ROWS < T <= sum_rows
                    and x.dtype == torch.bfloat16 and self.w_qkv.dtype == torch.bfloat16
                    and (T * (self.q_dim + 2 * self.kv_dim)) % 4 == 0)
            # (the product that adds has a buffer that nothing else writes: what it is left holding is known)
            qkv = step.buffer("attn.qkv_sum" if adds else "attn.qkv", (T, self.q_dim + 2 * self.kv_dim), torch.float32)
            if adds:
                # a few dozen rows (decoding at larger batches): q/k/v has too few output tiles for the
                # chip, so the product is cut over k and adds its parts into a cleared buffer
                # (measured at 32 rows of the 3B sizes: 10.7 + clearing against 19.5 us). The buffer
                # is cleared for the step's first such layer; the rotation kernel leaves it zero for
                # the next one (a clearing kernel per layer took 4.6 us). The note of that is the
                # step's: every step, and every recording of one, clears for itself.
                if step.extra.get("attn.qkv_sum zero", (0, 0)) != (qkv.data_ptr(), qkv.numel()):
                    ops.clear(qkv)
                step.extra.pop("attn.qkv_sum zero", None)
                ops.gemm(x, self.w_qkv, qkv, accumulate=True, fixed_order=step.fixed_order, choices=step.choices)
            else:
                project(self.w_qkv, qkv)
            if applies:
                self.position.apply(qkv[:, :self.q_dim].view(T, n_q, hd),
                                    qkv[:, self.q_dim:self.q_dim + self.kv_dim].view(T, n_kv, hd), step.positions)
            if adds and not applies and rot == hd and T == step.num_seqs:
                # decoded tokens only: the attention kernel rotates, writes the cache and clears the rows itself
                o = step.buffer("attn.o", (T, self.q_dim), act)
                if ops.mfma.attention_decode_rope(qkv, cos, sin, k_cache, v_cache, o, step, block_table, n_q, n_kv, hd,
                                                  self.scale, self.window):
                    step.extra["attn.qkv_sum zero"] = (qkv.data_ptr(), qkv.numel())
                    ops.gemm(o, self.w_o, out, accumulate, fixed_order=step.fixed_order, choices=step.choices)
                    return
            ops.rope_kv_write(qkv, cos, sin, step.positions, step.seq_idx, block_table, q, k_cache, v_cache,
                              n_q, n_kv, hd, rot, write_cache=True, zero_input=adds)
            if adds:
                step.extra["attn.qkv_sum zero"] = (qkv.data_ptr(), qkv.numel())
        else:
            # A layer that reads another layer's cache projects queries only.
            q32 = step.buffer("attn.q32", (T, self.q_dim), torch.float32)
            project(self.w_qkv[:self.q_dim // 16] if ops.is_blocked(self.w_qkv) else self.w_qkv[:self.q_dim], q32)
            if applies:
                self.position.apply(q32.view(T, n_q, hd), None, step.positions)
            ops.rope_q_only(q32, cos, sin, step.positions, q, n_q, hd, rot)
        o = step.buffer("attn.o", (T, self.q_dim), act)
        ops.attention_project(q, k_cache, v_cache, o, step, block_table, n_q, n_kv, hd, self.scale, self.window,
                              self.w_o, out, accumulate)


register_part("mixer", "attention", Attention)
