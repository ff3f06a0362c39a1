"""Python faces of the HIP kernels: each checks its operands on the host (device,
layout, type, shape, the limits the kernel assumes) and then launches on the
current HIP stream. Nothing here computes on the host and nothing falls back to
another library: a refused size raises `KernelError`.
"""
from __future__ import annotations

import torch

from .lib import BF16, F32, KernelError, check, code, entry, ptr, require, stream  # noqa: F401

_FLOATS = (torch.float32, torch.bfloat16)


from .choices import DEFAULT, KernelChoices, choices_of  # noqa: E402,F401

# The choices of operations that are called without a step (kernels on their own).
policy = DEFAULT


# --- weight layouts ------------------------------------------------------------------
# A weight matrix [N, K] (y = x W^T) is a 2-d tensor, row-major, or a 5-d tensor
# [N / 16, K / 32, 4, 16, 8] in the blocked layout of the matrix kernels: block (i, j) holds rows
# 16 i .. 16 i + 15 and k = 32 j .. 32 j + 31 as [4 q][16 r][8], element (r, 8 q + e) of the block at
# [q][r][e], which is the order in which a wavefront's 64 lanes hold a matrix-instruction operand.
# A wavefront then loads an operand as 1 KB of consecutive addresses. The tensor's rank tells the
# layout; row slices in steps of 16 rows are slices of the first dimension.
def is_blocked(w: torch.Tensor) -> bool:
    return w.dim() == 5


def weight_shape(w: torch.Tensor) -> tuple[int, int]:
    """(N, K) of a weight matrix in either layout."""
    if w.dim() == 5:
        if tuple(w.shape[2:]) != (4, 16, 8):
            raise KernelError(f"a blocked weight has blocks of [4, 16, 8], not {tuple(w.shape[2:])}")
        return w.shape[0] * 16, w.shape[1] * 32
    if w.dim() != 2:
        raise KernelError(f"a weight matrix is [N, K] or blocked [N / 16, K / 32, 4, 16, 8], not {tuple(w.shape)}")
    return w.shape[0], w.shape[1]


def can_block(w: torch.Tensor) -> bool:
    return (w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[0] % 16 == 0 and w.shape[1] % 32 == 0
            and w.is_contiguous())


def block_weight(w: torch.Tensor) -> torch.Tensor:
    """The blocked copy of a row-major bfloat16 matrix whose N is a multiple of 16 and K of 32."""
    if not can_block(w):
        raise KernelError(f"block_weight: needs bfloat16 [N, K] with N % 16 == 0 and K % 32 == 0, got "
                          f"{w.dtype} {tuple(w.shape)}")
    N, K = w.shape
    return w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()


def unblock_weight(w: torch.Tensor) -> torch.Tensor:
    """The row-major copy of a blocked matrix."""
    N, K = weight_shape(w)
    return w.permute(0, 3, 1, 2, 4).reshape(N, K).contiguous()


def _require_weight(w: torch.Tensor, name: str, dtypes, K: int | None = None) -> tuple[int, int]:
    require(w, name, dtypes)
    N, Kw = weight_shape(w)
    if K is not None and Kw != K:
        raise KernelError(f"{name}: expected K = {K}, got a matrix of [{N}, {Kw}]")
    return N, Kw


# --- embedding ---------------------------------------------------------------------
def embed_gather(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, :] = table[tokens[t], :] widened to 32-bit (the table row-major or blocked)."""
    V, H = _require_weight(table, "table", _FLOATS)
    T = tokens.shape[0]
    require(tokens, "tokens", torch.int32, (T,))
    require(out, "out", torch.float32, (T, H))
    check(entry("llme_embed_gather")(ptr(table), code(table.dtype), ptr(tokens), ptr(out), T, H,
                                     1 if is_blocked(table) else 0, stream()), "embed_gather")


# --- norm --------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
            rows: torch.Tensor | None = None) -> None:
    """out[r] = weight * x[rows[r] or r] / sqrt(mean(x^2) + eps); x is 32-bit."""
    require(x, "x", torch.float32, (None, None))
    H = x.shape[1]
    require(weight, "weight", _FLOATS, (H,))
    R = x.shape[0] if rows is None else rows.shape[0]
    if rows is not None:
        require(rows, "rows", torch.int32, (R,))
    require(out, "out", _FLOATS, (R, H))
    check(entry("llme_rmsnorm")(ptr(x), ptr(weight), code(weight.dtype), ptr(out), code(out.dtype),
                                ptr(rows), R, H, float(eps), stream()), "rmsnorm")


# --- feed-forward activation ------------------------------------------------------
def swiglu(gu: torch.Tensor, out: torch.Tensor, group: int) -> None:
    """out[t, j] = silu(gate_j) * up_j from gu [T, 2 FF] laid out in alternating groups."""
    require(out, "out", _FLOATS, (None, None))
    T, FF = out.shape
    require(gu, "gu", _FLOATS, (T, 2 * FF))
    if group <= 0 or FF % group != 0:
        raise KernelError(f"swiglu: group {group} does not divide the width {FF}")
    if gu.dtype == torch.bfloat16 and out.dtype != torch.bfloat16:
        raise KernelError("swiglu: bfloat16 input needs bfloat16 output")
    check(entry("llme_swiglu")(ptr(gu), code(gu.dtype), ptr(out), code(out.dtype), T, FF, group, stream()),
          "swiglu")


# --- rotary encoding + cache write --------------------------------------------------
def rope_kv_write(qkv: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                  positions: torch.Tensor, seq_idx: torch.Tensor, block_table: torch.Tensor,
                  q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                  n_q: int, n_kv: int, head_dim: int, rotary_dim: int, write_cache: bool = True,
                  max_position: int | None = None, zero_input: bool = False) -> None:
    """Rotates q and k heads of qkv [T, (n_q + 2 n_kv) hd] (32-bit) by the tables' rows
    at `positions`, writes q to q_out and k, v into the pages named by the block table.
    k_cache [pages, n_kv, page, hd]; v_cache [pages, n_kv, hd, page]. zero_input: qkv is all
    zeros afterwards (for a product that adds its parts into it)."""
    T = qkv.shape[0]
    require(qkv, "qkv", torch.float32, (T, (n_q + 2 * n_kv) * head_dim))
    require(positions, "positions", torch.int32, (T,))
    require(seq_idx, "seq_idx", torch.int32, (T,))
    require(block_table, "block_table", torch.int32, (None, None))
    require(q_out, "q_out", _FLOATS, (T, n_q * head_dim))
    require(k_cache, "k_cache", _FLOATS, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", k_cache.dtype, (k_cache.shape[0], n_kv, head_dim, page))
    if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim:
        raise KernelError(f"rope: rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
    if (cos is None) != (sin is None):
        raise KernelError("rope: cos and sin tables come together")
    if cos is not None:
        require(cos, "cos", torch.float32, (None, rotary_dim // 2))
        require(sin, "sin", torch.float32, tuple(cos.shape))
    check(entry("llme_rope_kv_write")(
        ptr(qkv), ptr(cos), ptr(sin), ptr(positions), ptr(seq_idx), ptr(block_table), block_table.shape[1],
        ptr(q_out), code(q_out.dtype), ptr(k_cache), ptr(v_cache), code(k_cache.dtype), T, n_q, n_kv,
        head_dim, rotary_dim if cos is not None else 0, page, 1 if write_cache else 0,
        1 if zero_input and write_cache else 0, stream()),
        "rope_kv_write")
    if zero_input and not write_cache:
        clear(qkv)


def rope_q_only(q32: torch.Tensor, cos: torch.Tensor | None, sin: torch.Tensor | None,
                positions: torch.Tensor, q_out: torch.Tensor, n_q: int, head_dim: int, rotary_dim: int) -> None:
    """Rotates query heads only (a layer that reads keys and values another layer cached)."""
    T = q32.shape[0]
    require(q32, "q32", torch.float32, (T, n_q * head_dim))
    require(positions, "positions", torch.int32, (T,))
    require(q_out, "q_out", _FLOATS, (T, n_q * head_dim))
    if cos is not None:
        require(cos, "cos", torch.float32, (None, rotary_dim // 2))
        require(sin, "sin", torch.float32, tuple(cos.shape))
    check(entry("llme_rope_kv_write")(
        ptr(q32), ptr(cos), ptr(sin), ptr(positions), None, None, 0, ptr(q_out), code(q_out.dtype), None, None,
        code(q_out.dtype), T, n_q, 0, head_dim, rotary_dim if cos is not None else 0, 1, 0, 0, stream()),
        "rope_q_only")


# --- matrix product ------------------------------------------------------------------
def gemm_generic(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> None:
    require(a, "a", _FLOATS, (None, None))
    M, K = a.shape
    N, _ = _require_weight(w, "w", _FLOATS, K)
    require(out, "out", _FLOATS, (M, N))
    check(entry("llme_gemm_generic")(ptr(a), code(a.dtype), ptr(w), code(w.dtype), ptr(out), code(out.dtype),
                                     M, N, K, 1 if accumulate else 0, 1 if is_blocked(w) else 0, stream()),
          "gemm_generic")


def clear(t: torch.Tensor) -> None:
    """Zeros a 32-bit buffer (for a product cut over k, whose parts add into it)."""
    require(t, "buffer", torch.float32)
    if t.numel() % 4 or t.data_ptr() % 16:
        raise KernelError("clear: a multiple of 4 values at a 16-byte aligned address")
    check(entry("llme_clear_f32")(ptr(t), t.numel(), stream()), "clear")


_fast_gemm = None       # set by ops/mfma.py when the MFMA kernels are present


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False,
         fixed_order: bool = False, choices: KernelChoices | None = None) -> None:
    """out[m, n] (+)= sum_k a[m, k] w[n, k]; 32-bit accumulation whatever the types. A sum that
    adds into `out` may be cut over k into parts that several workgroups add with atomics, in
    whatever order they finish: the result then differs from run to run in its last bits.
    fixed_order forbids that cut (every output element is summed by one workgroup in one order)."""
    if ((choices or DEFAULT).fast_gemm and _fast_gemm is not None
            and _fast_gemm(a, w, out, accumulate, fixed_order, choices)):
        return
    gemm_generic(a, w, out, accumulate)


# --- attention -----------------------------------------------------------------------
ATTENTION_MAX_HEAD_DIM = 256        # (a lane of attention_generic holds head_dim / 64 values of a row)


def attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                      positions: torch.Tensor, seq_idx: torch.Tensor, block_table: torch.Tensor,
                      n_q: int, n_kv: int, head_dim: int, scale: float, window: int = 0) -> None:
    T = q.shape[0]
    require(q, "q", _FLOATS, (T, n_q * head_dim))
    require(out, "out", q.dtype, (T, n_q * head_dim))
    require(k_cache, "k_cache", _FLOATS, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", k_cache.dtype, (k_cache.shape[0], n_kv, head_dim, page))
    require(positions, "positions", torch.int32, (T,))
    require(seq_idx, "seq_idx", torch.int32, (T,))
    require(block_table, "block_table", torch.int32, (None, None))
    if head_dim > ATTENTION_MAX_HEAD_DIM:
        raise KernelError(f"attention: head_dim {head_dim} is beyond the kernel's limit of {ATTENTION_MAX_HEAD_DIM}")
    if n_q % n_kv:
        raise KernelError(f"attention: {n_q} query heads do not divide into {n_kv} key/value heads")
    check(entry("llme_attention_generic")(
        ptr(q), code(q.dtype), ptr(k_cache), ptr(v_cache), code(k_cache.dtype), ptr(out), ptr(positions),
        ptr(seq_idx), ptr(block_table), block_table.shape[1], T, n_q, n_kv, head_dim, page, float(scale),
        int(window), stream()), "attention_generic")


# set by ops/mfma.py when the MFMA kernels are present
_fast_attention = None
_fast_attention_project = None


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, step,
              block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int, scale: float,
              window: int = 0) -> None:
    """Attention of every token of the step over its request's pages. `step` carries
    positions, request index per token and, on the host, how the batch is cut."""
    if choices_of(step).fast_attention and _fast_attention is not None and _fast_attention(
            q, k_cache, v_cache, out, step, block_table, n_q, n_kv, head_dim, scale, window):
        return
    attention_generic(q, k_cache, v_cache, out, step.positions, step.seq_idx, block_table, n_q, n_kv,
                      head_dim, scale, window)


def attention_project(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, o: torch.Tensor, step,
                      block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int, scale: float, window: int,
                      w_o: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
    """attention (as above, into o) and the output projection behind it: out (+)= o w_o^T. Where a
    step of a few decoded tokens cuts its keys into splits, the splits' join and the projection are
    one kernel, and o is not written."""
    # (only a step of up to 16 decoded tokens is asked about: steps launched kernel by kernel count their calls)
    choices = choices_of(step)
    if (q.shape[0] <= 16 and choices.fast_attention and choices.fast_gemm and _fast_attention_project is not None
            and _fast_attention_project(q, k_cache, v_cache, o, step, block_table, n_q, n_kv, head_dim, scale, window,
                                        w_o, out, accumulate)):
        return
    attention(q, k_cache, v_cache, o, step, block_table, n_q, n_kv, head_dim, scale, window)
    gemm(o, w_o, out, accumulate, fixed_order=step.fixed_order, choices=choices)


# --- sampling ------------------------------------------------------------------------
# The two-stage argmax and the sampler keep per-part results in scratch memory. Calls on one
# stream run one after the other and share a scratch per (device, stream); a caller whose launches
# are recorded into a graph brings a scratch of its own (`sampling_scratch`), which then lives as
# long as the recording does: the shared one is replaced when a later call needs a larger one.
_shared_scratch: dict = {}


def sampling_scratch(device, rows: int, vocab: int):
    """Scratch for argmax / sample calls of up to `rows` rows of `vocab` columns."""
    n = max(1, rows * entry("llme_argmax_parts")(vocab))
    return (torch.empty(n, dtype=torch.float32, device=device), torch.empty(n, dtype=torch.int32, device=device),
            torch.empty(n, dtype=torch.float32, device=device))


def _scratch_for(logits: torch.Tensor, scratch):
    R, V = logits.shape
    need = R * entry("llme_argmax_parts")(V)
    if scratch is not None:
        if len(scratch) != 3 or any(t.numel() < need or t.device != logits.device for t in scratch):
            raise KernelError(f"the sampling scratch is too small for {R} rows of {V} columns")
        return scratch
    key = (logits.device, stream())
    have = _shared_scratch.get(key)
    if have is None or have[0].numel() < need:
        if len(_shared_scratch) >= 64:
            _shared_scratch.clear()
        n = max(need, 4096)
        have = _shared_scratch[key] = (torch.empty(n, dtype=torch.float32, device=logits.device),
                                       torch.empty(n, dtype=torch.int32, device=logits.device),
                                       torch.empty(n, dtype=torch.float32, device=logits.device))
    return have


def argmax(logits: torch.Tensor, out: torch.Tensor, scratch=None) -> None:
    """out[r] = first index of the maximum of logits[r, :]."""
    require(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    require(out, "out", torch.int32, (R,))
    argmax_into(logits, ptr(out), scratch)


def argmax_into(logits: torch.Tensor, out_ptr: int, scratch=None, also_ptr: int = 0, slot_ptr: int = 0) -> None:
    """argmax with the result (one int32 per row) written to an address the device can reach:
    device memory, or pinned host memory, which the device sees at the same address. also_ptr: a
    second place for the same result. slot_ptr: an int32 in device memory, 0 or 1: the result goes to
    out_ptr + 4 * slot * rows (out then holds two results in turn)."""
    require(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    val, idx, _ = _scratch_for(logits, scratch)
    if also_ptr or slot_ptr:
        check(entry("llme_argmax_to")(ptr(logits), out_ptr, also_ptr or None, slot_ptr or None, ptr(val), ptr(idx), R, V,
                                      stream()), "argmax")
    else:
        check(entry("llme_argmax")(ptr(logits), out_ptr, ptr(val), ptr(idx), R, V, stream()), "argmax")


def sample_into(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor, out_ptr: int, scratch=None,
                also_ptr: int = 0, slot_ptr: int = 0) -> None:
    """sample with the result written as argmax_into writes it: to out_ptr + 4 * slot * rows (device
    memory, or pinned host memory), and to also_ptr where given."""
    require(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    require(temperature, "temperature", torch.float32, (R,))
    require(uniform, "uniform", torch.float32, (R,))
    val, idx, sums = _scratch_for(logits, scratch)
    check(entry("llme_sample_to")(ptr(logits), ptr(temperature), ptr(uniform), out_ptr, also_ptr or None, slot_ptr or None,
                                  ptr(val), ptr(idx), ptr(sums), R, V, stream()), "sample")


def sample(logits: torch.Tensor, temperature: torch.Tensor, uniform: torch.Tensor, out: torch.Tensor,
           scratch=None) -> None:
    require(logits, "logits", torch.float32, (None, None))
    R, V = logits.shape
    require(temperature, "temperature", torch.float32, (R,))
    require(uniform, "uniform", torch.float32, (R,))
    require(out, "out", torch.int32, (R,))
    val, idx, sums = _scratch_for(logits, scratch)
    check(entry("llme_sample")(ptr(logits), ptr(temperature), ptr(uniform), ptr(out), ptr(val), ptr(idx), ptr(sums),
                               R, V, stream()), "sample")
