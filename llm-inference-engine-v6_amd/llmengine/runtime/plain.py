"""Python faces of the plain C++ twins of the device kernels (csrc/host/plain_kernels.cpp).

Every function takes and returns 32-bit CPU tensors (int32 for ids and positions) and runs
one serial loop nest in the order of the reference's scalar kernels (src/kernels.cpp). The
engine never calls them: they are what the tests hold each device kernel against, beside the
tests' own plain Python implementation.
"""
from __future__ import annotations

import torch

from . import native


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to("cpu", torch.float32).contiguous()


def _i32(v) -> torch.Tensor:
    return torch.as_tensor(v, dtype=torch.int32, device="cpu").contiguous()


def _check(code: int, what: str) -> int:
    if code < 0:
        raise ValueError(f"{what}: refused by the plain kernel (code {code})")
    return code


def embed(table: torch.Tensor, tokens) -> torch.Tensor:
    table, tokens = _f32(table), _i32(tokens)
    V, H = table.shape
    out = torch.empty(tokens.numel(), H, dtype=torch.float32)
    _check(native.library().llme_plain_embed(table.data_ptr(), tokens.data_ptr(), tokens.numel(), V, H,
                                             out.data_ptr()), "embed")
    return out


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    x, w = _f32(x), _f32(w)
    T, H = x.shape
    out = torch.empty_like(x)
    _check(native.library().llme_plain_rmsnorm(x.data_ptr(), w.data_ptr(), T, H, float(eps), out.data_ptr()), "rmsnorm")
    return out


def linear(a: torch.Tensor, w: torch.Tensor, into: torch.Tensor | None = None) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed; added to `into` when given."""
    a, w = _f32(a), _f32(w)
    (M, K), N = a.shape, w.shape[0]
    if w.shape[1] != K:
        raise ValueError(f"linear: a is {tuple(a.shape)}, w is {tuple(w.shape)}")
    out = _f32(into).clone() if into is not None else torch.empty(M, N, dtype=torch.float32)
    _check(native.library().llme_plain_linear(a.data_ptr(), w.data_ptr(), M, N, K, out.data_ptr(),
                                              1 if into is not None else 0), "linear")
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    gate, up = _f32(gate), _f32(up)
    out = torch.empty_like(gate)
    _check(native.library().llme_plain_swiglu(gate.data_ptr(), up.data_ptr(), gate.numel(), out.data_ptr()), "swiglu")
    return out


def inv_freq(head_dim: int, theta: float, scaling=None) -> torch.Tensor:
    """scaling = (factor, low_freq_factor, high_freq_factor, original_max_position) or None."""
    out = torch.empty(head_dim // 2, dtype=torch.float32)
    f, lo, hi, orig = scaling if scaling is not None else (1.0, 1.0, 1.0, 0.0)
    _check(native.library().llme_plain_inv_freq(head_dim, float(theta), 0 if scaling is None else 1, float(f), float(lo),
                                                float(hi), float(orig), out.data_ptr()), "inv_freq")
    return out


def rope_tables(inv: torch.Tensor, positions, head_dim: int) -> tuple[torch.Tensor, torch.Tensor]:
    inv, positions = _f32(inv), _i32(positions)
    n = positions.numel()
    cos, sin = torch.empty(n, head_dim, dtype=torch.float32), torch.empty(n, head_dim, dtype=torch.float32)
    _check(native.library().llme_plain_rope_tables(inv.data_ptr(), positions.data_ptr(), n, head_dim, cos.data_ptr(),
                                                   sin.data_ptr()), "rope_tables")
    return cos, sin


def rope_apply(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [T, heads, head_dim], cos and sin [T, head_dim]."""
    out, cos, sin = _f32(x).clone(), _f32(cos), _f32(sin)
    T, heads, hd = out.shape
    _check(native.library().llme_plain_rope_apply(out.data_ptr(), cos.data_ptr(), sin.data_ptr(), T, heads, hd),
           "rope_apply")
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """q [T, n_q, hd]: the last T positions of a request whose keys and values so far are
    k, v [ctx + T, n_kv, hd]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    T, n_q, hd = q.shape
    total, n_kv, _ = k.shape
    if v.shape != k.shape or total < T:
        raise ValueError(f"attention: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    out = torch.empty_like(q)
    _check(native.library().llme_plain_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), T, total - T, n_q, n_kv, hd,
                                                 int(window), out.data_ptr()), "attention")
    return out


def argmax(row: torch.Tensor) -> int:
    row = _f32(row)
    return _check(native.library().llme_plain_argmax(row.data_ptr(), row.numel()), "argmax")


def sample(row: torch.Tensor, temperature: float, u: float) -> int:
    row = _f32(row)
    return _check(native.library().llme_plain_sample(row.data_ptr(), row.numel(), float(temperature), float(u)), "sample")


def llama_forward(cfg, weights: dict, tokens, positions=None, window: int = 0) -> torch.Tensor:
    """Logits [T, V] of one whole sequence through the plain C++ backend of the Llama decoder
    (csrc/host/plain_model.cpp): every tensor in 32-bit, serial loops, no cache. cfg: the typed
    configuration (config.llama.LlamaConfig); weights: checkpoint names -> tensors."""
    import ctypes
    tokens = _i32(tokens)
    T = tokens.numel()
    positions = _i32(range(T) if positions is None else positions)
    if positions.numel() != T:
        raise ValueError("llama_forward: one position per token")
    w = {k: _f32(v) for k, v in weights.items()}
    per_layer = ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight",
                 "self_attn.v_proj.weight", "self_attn.o_proj.weight", "post_attention_layernorm.weight",
                 "mlp.gate_proj.weight", "mlp.up_proj.weight", "mlp.down_proj.weight")
    L = cfg.num_hidden_layers
    pointers = (ctypes.c_void_p * (9 * L))(*[w[f"model.layers.{l}.{n}"].data_ptr() for l in range(L) for n in per_layer])
    sizes = _i32([L, cfg.hidden_size, cfg.intermediate_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                  cfg.head_dim, cfg.vocab_size, int(window)])
    sc = cfg.rope_scaling
    rope = torch.tensor([cfg.rope_theta, 0.0 if sc is None else 1.0] +
                        ([1.0, 1.0, 1.0, 0.0] if sc is None else
                         [sc.factor, sc.low_freq_factor, sc.high_freq_factor, float(sc.original_max_position_embeddings)]),
                        dtype=torch.float64)
    embed = w["model.embed_tokens.weight"]
    head = embed if cfg.tie_word_embeddings else w["lm_head.weight"]
    logits = torch.empty(T, cfg.vocab_size, dtype=torch.float32)
    _check(native.library().llme_plain_llama_forward(sizes.data_ptr(), rope.data_ptr(), float(cfg.rms_norm_eps),
                                                     embed.data_ptr(), w["model.norm.weight"].data_ptr(), head.data_ptr(),
                                                     pointers, tokens.data_ptr(), positions.data_ptr(), T,
                                                     logits.data_ptr()), "llama_forward")
    return logits
