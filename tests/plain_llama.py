"""A plain, slow implementation of the Llama decoder, written from the reference's
formulas: whole sequences, no cache, one function per part, torch on the CPU.

It shares no code with the engine under llm-inference-engine-v6_amd/: it reads
checkpoints with the safetensors library and computes with elementary tensor
operations. Every function cites the lines of the reference it follows
(paths relative to the reference's root). The reference was read, not run.

`dtype` is the arithmetic type (float64 by default: an oracle tighter than the
engine's 32-bit path; float32 reproduces the reference's own precision).
`rounder` optionally rounds activations where the bfloat16 engine stores them in
bfloat16 (normed activations, rotated q and k, v, attention output, gated
activation), so that the bfloat16 engine can be compared more tightly.
"""
from __future__ import annotations

import json
import math
import os

import torch


# ------------------------------------------------------------------------------------
# configuration: defaults of src/weights.cpp:59-96
def plain_config(cfg: dict) -> dict:
    n_q = cfg["num_attention_heads"]
    out = {
        "H": cfg["hidden_size"], "FF": cfg["intermediate_size"], "L": cfg["num_hidden_layers"],
        "n_q": n_q, "n_kv": cfg.get("num_key_value_heads", n_q),                       # weights.cpp:64
        "hd": cfg.get("head_dim") or cfg["hidden_size"] // n_q,                        # weights.cpp:65-68
        "V": cfg["vocab_size"], "max_pos": cfg["max_position_embeddings"],
        "eps": cfg.get("rms_norm_eps", 1e-5),                                          # weights.cpp:71
        "tie": cfg.get("tie_word_embeddings", False),                                  # weights.cpp:72
        "theta": cfg.get("rope_theta", 10000.0),                                       # weights.cpp:79
        "scaling": None,
    }
    block = None
    rp = cfg.get("rope_parameters")
    if rp is not None:                                                                 # weights.cpp:89-93
        out["theta"] = rp.get("rope_theta", out["theta"])
        if rp.get("rope_type", "default") == "llama3":
            block = rp
    elif cfg.get("rope_scaling") is not None:                                          # weights.cpp:94-95
        block = cfg["rope_scaling"]
    if block is not None:                                                              # weights.cpp:81-87
        out["scaling"] = (block.get("factor", 1.0), block.get("low_freq_factor", 1.0),
                          block.get("high_freq_factor", 1.0),
                          block.get("original_max_position_embeddings", 0))
    return out


def load_plain_model(model_dir: str, dtype=torch.float64):
    """(config dict, {name: tensor}) from a model folder, via the safetensors library."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    weights = {}
    for name in sorted(os.listdir(model_dir)):
        if name.endswith(".safetensors"):
            weights.update(load_file(os.path.join(model_dir, name)))
    return cfg, {k: v.to(dtype) for k, v in weights.items()}


# ------------------------------------------------------------------------------------
def plain_embed(table: torch.Tensor, tokens) -> torch.Tensor:
    """h = E[token, :], a row copy without scaling (src/kernels.cpp:59-66, src/engine.cpp:118)."""
    return torch.stack([table[int(t)] for t in tokens])


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """out = w * x * (1 / sqrt(sum(x^2) / dim + eps)) per row (src/kernels.cpp:18-24): the
    weight multiplies directly (no 1 + w), eps is inside the root."""
    sumsq = (x * x).sum(dim=-1, keepdim=True)
    inv_rms = 1.0 / torch.sqrt(sumsq / x.shape[-1] + eps)
    return (w * x) * inv_rms


def plain_linear_by_rows(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out[m, n] = sum_k a[m, k] * w[n, k], W stored [N, K]; no bias (src/kernels.cpp:33-57)."""
    out = torch.zeros(a.shape[0], w.shape[0], dtype=a.dtype)
    for n in range(w.shape[0]):
        out[:, n] = (a * w[n]).sum(dim=-1)
    return out


def plain_linear(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """The same sum as `plain_linear_by_rows` through the library's matrix product on the CPU
    (tests pin the two to each other): fast enough for layers of real width."""
    return a @ w.T


def plain_silu(x: torch.Tensor) -> torch.Tensor:
    """v / (1 + exp(-v)) (src/kernels.cpp:26-31)."""
    return x / (1.0 + torch.exp(-x))


def plain_inv_freq(head_dim: int, theta: float, scaling) -> list[float]:
    """Inverse frequencies in 64-bit, returned as the 32-bit values the reference stores
    (src/kernels.cpp:114-160). scaling = (factor, low_freq_factor, high_freq_factor, original)."""
    half = head_dim // 2
    inv = [1.0 / math.pow(float(theta), (2 * i) / float(head_dim)) for i in range(half)]   # kernels.cpp:126-131
    if scaling is not None:
        factor, low, high, orig = scaling
        low_wavelen = float(orig) / low                                    # kernels.cpp:134-137
        high_wavelen = float(orig) / high
        band = float(high) - low
        for i in range(half):
            fr = inv[i]
            wavelen = 2.0 * math.pi / fr                                   # kernels.cpp:145
            if wavelen > low_wavelen:
                inv[i] = fr / factor                                       # kernels.cpp:146-147
            elif wavelen < high_wavelen:
                pass                                                       # kernels.cpp:148-149
            else:
                smooth = (float(orig) / wavelen - low) / band              # kernels.cpp:151-153
                inv[i] = (1.0 - smooth) * fr / factor + smooth * fr
    return [float(torch.tensor(v, dtype=torch.float64).to(torch.float32)) for v in inv]   # kernels.cpp:157-158


def plain_rope_tables(inv_freq: list[float], positions, head_dim: int):
    """cos, sin [len(positions), head_dim]: angle = p * inv_freq[i] in 64-bit, stored in 32-bit,
    both halves of a row equal (src/kernels.cpp:162-187)."""
    half = head_dim // 2
    cos = torch.zeros(len(positions), head_dim, dtype=torch.float64)
    sin = torch.zeros(len(positions), head_dim, dtype=torch.float64)
    for r, p in enumerate(positions):
        for i in range(half):
            angle = float(p) * inv_freq[i]
            c = float(torch.tensor(math.cos(angle), dtype=torch.float64).to(torch.float32))
            s = float(torch.tensor(math.sin(angle), dtype=torch.float64).to(torch.float32))
            cos[r, i] = cos[r, i + half] = c
            sin[r, i] = sin[r, i + half] = s
    return cos, sin


def plain_apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [T, heads, hd], cos/sin [T, hd]. Pairs are (i, i + hd/2):
    x[i] <- a cos[i] - b sin[i]; x[i + h] <- b cos[i + h] + a sin[i + h] (src/kernels.cpp:189-203)."""
    half = x.shape[-1] // 2
    out = torch.empty_like(x)
    c, s = cos.to(x.dtype)[:, None, :], sin.to(x.dtype)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    out[..., :half] = a * c[..., :half] - b * s[..., :half]
    out[..., half:] = b * c[..., half:] + a * s[..., half:]
    return out


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0) -> torch.Tensor:
    """q [T, n_q, hd], k and v [T, n_kv, hd] -> [T, n_q, hd]. For the token at position p and
    query head h: kv head = h / (n_q / n_kv); s_t = (q . K[t]) / sqrt(hd) for t <= p; stable softmax;
    out = sum_t p_t V[t] (src/kernels.cpp:413-474; the token loop of src/engine.cpp:186-189 makes
    the mask: only keys up to the own position exist). window > 0: only keys t > p - window."""
    T, n_q, hd = q.shape
    n_kv = k.shape[1]
    group = n_q // n_kv                                                      # kernels.cpp:421
    scale = 1.0 / math.sqrt(float(hd))                                       # kernels.cpp:422
    out = torch.zeros_like(q)
    for h in range(n_q):
        kv_h = h // group                                                    # kernels.cpp:441
        for p in range(T):
            lo = max(0, p - window + 1) if window > 0 else 0
            scores = (k[lo:p + 1, kv_h] * q[p, h]).sum(dim=-1) * scale       # kernels.cpp:446-455
            e = torch.exp(scores - scores.max())                             # kernels.cpp:458-462
            probs = e * (1.0 / e.sum())                                      # kernels.cpp:463-464
            out[p, h] = (probs[:, None] * v[lo:p + 1, kv_h]).sum(dim=0)      # kernels.cpp:467-474
    return out


def plain_mlp(x: torch.Tensor, w_gate, w_up, w_down, rounder=None) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)) (src/engine.cpp:213-217)."""
    act = plain_silu(plain_linear(x, w_gate)) * plain_linear(x, w_up)
    if rounder:
        act = rounder(act)
    return plain_linear(act, w_down)


def _identity(x):
    return x


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(x.dtype)


def plain_forward(cfg: dict, weights: dict, tokens, dtype=torch.float64, rounder=None, positions=None,
                  schedule=None, window: int = 0, rows=None) -> torch.Tensor:
    """Logits [T, V] at every position of one sequence, or at the positions `rows` only
    (src/engine.cpp:105-261 per token, applied to the whole sequence at once). `positions` shifts the sequence (default 0..T-1). `schedule`:
    list of (layer, cache id, writes) in running order (default: each layer once, own cache);
    a call that does not write reads the keys and values of the cache id's writer."""
    c = plain_config(cfg)
    rnd = rounder or _identity
    w = {k: t.to(dtype) for k, t in weights.items()}
    T = len(tokens)
    positions = list(range(T)) if positions is None else list(positions)
    inv_freq = plain_inv_freq(c["hd"], c["theta"], c["scaling"])
    cos, sin = plain_rope_tables(inv_freq, positions, c["hd"])
    h = plain_embed(w["model.embed_tokens.weight"], tokens)                           # engine.cpp:118
    schedule = schedule or [(l, l, True) for l in range(c["L"])]
    kv_store = {}
    for layer, cache_id, writes in schedule:
        p = f"model.layers.{layer}."
        x = rnd(plain_rmsnorm(h, w[p + "input_layernorm.weight"], c["eps"]))          # engine.cpp:137
        q = plain_linear(x, w[p + "self_attn.q_proj.weight"]).view(T, c["n_q"], c["hd"])    # engine.cpp:142
        q = rnd(plain_apply_rope(q, cos, sin))                                        # engine.cpp:163-166
        if writes:
            k = plain_linear(x, w[p + "self_attn.k_proj.weight"]).view(T, c["n_kv"], c["hd"])   # engine.cpp:143
            v = plain_linear(x, w[p + "self_attn.v_proj.weight"]).view(T, c["n_kv"], c["hd"])   # engine.cpp:144
            k = rnd(plain_apply_rope(k, cos, sin))                                    # engine.cpp:167-170
            kv_store[cache_id] = (k, rnd(v))
        k, v = kv_store[cache_id]
        attn = rnd(plain_attention(q, k, v, window)).reshape(T, c["n_q"] * c["hd"])   # engine.cpp:186-189
        h = h + plain_linear(attn, w[p + "self_attn.o_proj.weight"])                  # engine.cpp:193,206
        x = rnd(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], c["eps"]))  # engine.cpp:208
        h = h + plain_mlp(x, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                          w[p + "mlp.down_proj.weight"], rounder)                     # engine.cpp:213-239
    if rows is not None:
        h = h[list(rows)]
    x = rnd(plain_rmsnorm(h, w["model.norm.weight"], c["eps"]))                       # engine.cpp:243
    head = w["model.embed_tokens.weight"] if c["tie"] else w["lm_head.weight"]        # model.cpp:185-195
    return plain_linear(x, head)                                                      # engine.cpp:247


def plain_argmax(row: torch.Tensor) -> int:
    """First index of the maximum, strict > (src/engine.cpp:52-58)."""
    best, arg = row[0], 0
    for i in range(1, row.shape[0]):
        if row[i] > best:
            best, arg = row[i], i
    return arg


def plain_generate(cfg: dict, weights: dict, prompt, max_new_tokens: int, eos=(), dtype=torch.float64,
                   choose=None):
    """Greedy generation by running the whole sequence again for every token
    (src/engine.cpp:753-773: EOS is not appended; 'stop' or 'length')."""
    ids = list(prompt)
    finish = "length"
    for i in range(max_new_tokens):
        logits = plain_forward(cfg, weights, ids, dtype)[-1]
        nxt = choose(logits, i) if choose else plain_argmax(logits)
        if nxt in eos:
            finish = "stop"
            break
        ids.append(int(nxt))
    return ids, finish


def plain_sample_bounds(row: torch.Tensor, temperature: float):
    """Cumulative probabilities of softmax(row / T) in ascending id order: token i is drawn
    when the uniform number falls in [cum[i-1], cum[i])."""
    z = row.to(torch.float64) / temperature
    p = torch.exp(z - z.max())
    p = p / p.sum()
    return torch.cumsum(p, dim=0)
