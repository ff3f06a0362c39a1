"""The MFMA (matrix core) kernels: bfloat16 matrix products and, in a later section,
attention. Importing this module makes `ops.gemm` and `ops.attention` choose them where
operand types and sizes fit; what they refuse goes to the plain-precision kernels."""
from __future__ import annotations

import ctypes

import torch

from . import kernels
from .choices import DEFAULT, KernelChoices, choices_of
from .lib import check, declare, entry, ptr, require, stream

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float

declare("llme_gemm_bf16", [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _vp])


def gemm_bf16_supported(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool) -> bool:
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and out.dtype in (torch.float32, torch.bfloat16)
            and not (accumulate and out.dtype != torch.float32)
            and w.dim() in (2, 5) and a.shape[1] % 8 == 0 and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0
            and out.data_ptr() % 16 == 0)


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, accumulate: bool = False, *,
              gated: bool = False, waves: int = 0, ksplit: int = 0, tile: int = 0, force_tile: bool = False,
              direct: int = -1, _supported: bool = False) -> None:
    """bfloat16 a [M, K] and w [N, K] -> out [M, N] (float32 or bfloat16), 32-bit accumulation.
    K must be a multiple of 8. gated: w holds gate and up rows interleaved in groups of 16 and
    out is bfloat16 [M, N / 2] = silu(gate) * up. waves / ksplit / tile (64, 128, 128096, 128064, 96128, 96064) /
    force_tile override the launch choices (tests and measurements); direct: whether the product may
    use the 256 x 256 tile kernel whose slabs go from memory straight into LDS, which needs a blocked w
    (-1: where it pays, 0: never, 1: it must, with tile 256256)."""
    require(a, "a", torch.bfloat16, (None, None))
    M, K = a.shape
    N, _ = kernels._require_weight(w, "w", torch.bfloat16, K)
    if gated:
        require(out, "out", torch.bfloat16, (M, N // 2))
        if N % 32 or accumulate:
            raise kernels.KernelError("gemm_bf16: a gated product needs a multiple of 32 weight rows and no accumulation")
    else:
        require(out, "out", (torch.float32, torch.bfloat16), (M, N))
    if not _supported and not gemm_bf16_supported(a, w, out, accumulate):     # (the dispatcher has asked already)
        raise kernels.KernelError(f"gemm_bf16: K={K} must be a multiple of 8, pointers 16-byte aligned, and "
                                  "accumulation needs a float32 output")
    if force_tile and not tile:
        tile = 128
    check(entry("llme_gemm_bf16")(ptr(a), ptr(w), ptr(out), 0 if out.dtype == torch.float32 else 1, M, N, K,
                                  1 if accumulate else 0, 1 if gated else 0, waves, ksplit, tile,
                                  1 if kernels.is_blocked(w) else 0, int(direct), stream()),
          "gemm_bf16")


def gemm_gated(x: torch.Tensor, w_gate_up: torch.Tensor, out: torch.Tensor, group: int, scratch,
               choices: KernelChoices | None = None) -> None:
    """out [T, FF] = silu(x Wg^T) * (x Wu^T), the gate and up rows interleaved in groups of `group`
    rows of w_gate_up [2 FF, K]. One MFMA kernel where the types and sizes fit it; otherwise the
    product into a 32-bit scratch [T, 2 FF] (scratch(shape, dtype) provides it) and the
    activation kernel."""
    T, FF = out.shape
    if ((choices or DEFAULT).fast_gemm and group == 16 and out.dtype == torch.bfloat16 and (2 * FF) % 32 == 0
            and x.dtype == torch.bfloat16 and gemm_bf16_supported(x, w_gate_up, out, False)):
        r = tail_rows(T, choices)
        if r:
            gemm_bf16(x[:T - r], w_gate_up, out[:T - r], gated=True, _supported=True)
            gemm_bf16(x[T - r:], w_gate_up, out[T - r:], gated=True, _supported=True)
            return
        gemm_bf16(x, w_gate_up, out, gated=True, _supported=True)
        return
    gu = scratch((T, 2 * FF), torch.float32)
    kernels.gemm(x, w_gate_up, gu, choices=choices)
    kernels.swiglu(gu, out, group)


declare("llme_gemm_bf16_qkv_rope", [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp])


def gemm_qkv_rope_supported(x: torch.Tensor, w_qkv: torch.Tensor, k_cache: torch.Tensor, head_dim: int,
                            rotary_dim: int, choices: KernelChoices | None = None) -> bool:
    """Whether a step may take gemm_qkv_rope: the kernel takes the operands, and the choices allow it."""
    return (choices or DEFAULT).fast_gemm and _gemm_qkv_rope_fits(x, w_qkv, k_cache, head_dim, rotary_dim)


def _gemm_qkv_rope_fits(x, w_qkv, k_cache, head_dim: int, rotary_dim: int) -> bool:
    return (x.dtype == torch.bfloat16 and w_qkv.dtype == torch.bfloat16
            and k_cache.dtype == torch.bfloat16 and head_dim in (16, 32, 64, 128) and rotary_dim == head_dim
            and w_qkv.dim() in (2, 5) and x.shape[1] % 8 == 0 and x.data_ptr() % 16 == 0 and w_qkv.data_ptr() % 16 == 0)


def gemm_qkv_rope(x: torch.Tensor, w_qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                  seq_idx: torch.Tensor, block_table: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, n_q: int, n_kv: int, head_dim: int, tile: int = 0) -> None:
    """The q/k/v projection of a step's rows with rotation and cache write in the product's epilogue:
    x [T, K] bfloat16 (normed), w_qkv [(n_q + 2 n_kv) hd, K] bfloat16 (row-major or blocked); q heads
    and k heads are rotated at the rows' positions, q goes to q_out [T, n_q hd], k and v into the
    rows' pages. The 32-bit q/k/v rows that the separate kernels pass between them never exist.
    Full rotation, head size 16, 32, 64 or 128. tile: 0 (chosen), 64, 96064, 128064, 96128 or 128."""
    require(x, "x", torch.bfloat16, (None, None))
    T, K = x.shape
    n_rows, _ = kernels._require_weight(w_qkv, "w_qkv", torch.bfloat16, K)
    if n_rows != (n_q + 2 * n_kv) * head_dim:
        raise kernels.KernelError(f"gemm_qkv_rope: w_qkv has {n_rows} rows, the heads need {(n_q + 2 * n_kv) * head_dim}")
    require(positions, "positions", torch.int32, (T,))
    require(seq_idx, "seq_idx", torch.int32, (T,))
    require(block_table, "block_table", torch.int32, (None, None))
    require(cos, "cos", torch.float32, (None, head_dim // 2))
    require(sin, "sin", torch.float32, tuple(cos.shape))
    require(q_out, "q_out", torch.bfloat16, (T, n_q * head_dim))
    require(k_cache, "k_cache", torch.bfloat16, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", torch.bfloat16, (k_cache.shape[0], n_kv, head_dim, page))
    if not _gemm_qkv_rope_fits(x, w_qkv, k_cache, head_dim, head_dim):
        raise kernels.KernelError(f"gemm_qkv_rope: head size {head_dim} (16, 32, 64 or 128), K={K} (multiple of 8) or the "
                                  "operand types are not supported")
    check(entry("llme_gemm_bf16_qkv_rope")(
        ptr(x), ptr(w_qkv), T, K, 1 if kernels.is_blocked(w_qkv) else 0, ptr(cos), ptr(sin), ptr(positions), ptr(seq_idx),
        ptr(block_table), block_table.shape[1], ptr(q_out), ptr(k_cache), ptr(v_cache), n_q, n_kv, head_dim, page,
        int(tile), stream()), "gemm_qkv_rope")


TAIL_ROWS_ROUND = 1024              # rows that the tile kernels cover in full rounds of workgroups (tail_rows)


def tail_rows(M: int, choices: KernelChoices | None = None) -> int:
    """Rows at the end of a product of M rows that a launch of their own takes (0: none). The tile kernels
    cover whole multiples of 1,024 rows in full rounds of workgroups over the chip at the widths of the Llama
    sizes; a few rows more start another round that is almost empty. Those few rows (a step's decoded tokens
    behind a prompt portion of 1,024 or 2,048) then cost less as a small product of their own, although it
    reads the weights once more. Measured on whole prompts (ms, one launch / two): 1B sizes 1,040 tokens
    3.69 / 3.42, 2,080 tokens 6.20 / 5.69; 8B sizes 20.5 / 18.4 and 35.0 / 33.1; 3B sizes (whose width of 3,072 fills
    no round exactly) 9.14 / 9.14 and 15.7 / 15.1. Anywhere else two launches lose (1B sizes, 1,160 tokens 3.83 /
    4.24; 1,550 tokens 4.76 / 4.97)."""
    ch = choices or DEFAULT
    r = M % TAIL_ROWS_ROUND
    return r if ch.tail_rows_apart and M > TAIL_ROWS_ROUND and 0 < r <= ch.tail_rows_most else 0


def _fast_gemm(a, w, out, accumulate, fixed_order=False, choices: KernelChoices | None = None) -> bool:
    if a.dim() != 2 or w.dim() not in (2, 5) or not gemm_bf16_supported(a, w, out, accumulate):
        return False
    r = tail_rows(a.shape[0], choices) if accumulate else 0
    if r:                                                   # (sums into the residual stream; see tail_rows)
        m, ks = a.shape[0] - r, 1 if fixed_order else 0
        gemm_bf16(a[:m], w, out[:m], True, ksplit=ks, _supported=True)
        gemm_bf16(a[m:], w, out[m:], True, ksplit=ks, _supported=True)
        return True
    # (ksplit 1: the entry point cuts nothing over k, so no partial sums meet in atomics)
    gemm_bf16(a, w, out, accumulate, ksplit=1 if fixed_order and accumulate else 0, _supported=True)
    return True


kernels._fast_gemm = _fast_gemm


# --- attention ---------------------------------------------------------------------------
declare("llme_attention_bf16_rows", [_i, _i, _i, _i])
declare("llme_attention_bf16_splits_prefill", [_i, _i, _i, _i])
declare("llme_attention_bf16", [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i,
                                _i, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp, _i, _vp])


def attention_tuning(rows: int = 0, shared: int = -1, read_once: int = -1, half_rows: bool = False) -> int:
    """Overrides of the attention kernels' launch choices for one call (tests, measurements), as
    the entry points take them; 0 leaves every choice to the entry point. rows: rows per work item
    of the prefill kernel without LDS (16, 32, 64; 0: by head size). shared: the prefill kernel that
    shares K and V through LDS: -1 where it takes the sizes, 0 never, 1 wherever it can, 2 / 3 with
    one / two wavefronts per tile whatever the number of items. read_once: the decode kernel's
    cache hint on keys and values: -1 the entry point chooses, 0 off, 1 on. half_rows: work items of
    half the rows in the kernel that shares K and V (plan_attention sets it by itself for steps with
    few items; the choice prefill_half_rows False keeps it from that)."""
    if rows not in (0, 16, 32, 64) or not -1 <= shared <= 3 or not -1 <= read_once <= 1:
        raise kernels.KernelError(f"attention_tuning: rows {rows}, shared {shared}, read_once {read_once}")
    return rows | (shared + 1) << 8 | (read_once + 1) << 12 | (TUNING_HALF_ROWS if half_rows else 0)


TUNING_HALF_ROWS = 1 << 15

_work_queues: dict = {}


def work_queue(device: torch.device) -> torch.Tensor:
    """Two zeroed integers for the prefill kernel's work counter, one pair per device and
    stream: launches on one stream run one after the other and leave them zero."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream())
    q = _work_queues.get(key)
    if q is None:
        q = _work_queues[key] = torch.zeros(2, dtype=torch.int32, device=device)
    return q


_compute_units = 0


def compute_units() -> int:
    """Compute units of the current device (asked once)."""
    global _compute_units
    if _compute_units <= 0:
        _compute_units = max(1, int(entry("llme_compute_units")()))
    return _compute_units

MIN_SPLIT = 128                     # keys per split at least: one 32-key block per wavefront
MAX_SPLITS = 64                     # the join kernel's limit


def attention_bf16_supported(q, k_cache, head_dim: int) -> bool:
    return (q.dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and head_dim % 16 == 0
            and head_dim <= 128 and k_cache.shape[2] % 16 == 0 and q.data_ptr() % 16 == 0
            and k_cache.data_ptr() % 16 == 0)


def plan_attention(new_lens, ctx_lens, n_q: int, n_kv: int, head_dim: int, plan_len: int | None = None,
                   tuning: int = 0, choices: KernelChoices | None = None, cut: int | None = None) -> dict:
    """Launch sizes for a step, from how its batch is cut (host-side numbers only). plan_len:
    plan the decode splits for requests of up to this many tokens, whatever their length now
    (a recorded step is replayed while the requests grow). tuning: see attention_tuning. choices:
    the sizes at which the plan changes its shape. cut: what decode_cut said for this step, where the caller
    has asked already (a recorded step is kept under it)."""
    ch = choices or DEFAULT
    rows = entry("llme_attention_bf16_rows")(head_dim, n_q, n_kv, tuning)
    if rows <= 0:
        raise kernels.KernelError(f"plan_attention: tuning {tuning} is not one that attention_tuning makes")
    decode = [c + 1 for n, c in zip(new_lens, ctx_lens) if n == 1]
    groups = sum((n + rows - 1) // rows for n in new_lens if n >= 2)
    plan = {"n_decode": len(decode), "groups": groups, "split_len": 32, "nsplit": 1, "prefill_splits": 1,
            "prefill_run": 1, "tuning": tuning}
    if groups and entry("llme_attention_bf16_splits_prefill")(head_dim, n_q, n_kv, tuning):
        group = n_q // n_kv
        items = groups * (n_q // (4 if group % 4 == 0 else 2 if group % 2 == 0 else 1))
        # few rows over long contexts: too few work items for the chip, each with many keys
        keys = max(c + n for n, c in zip(new_lens, ctx_lens) if n >= 2)
        splits = 1
        if items <= (ch.prefill_cut_items or 3 * compute_units() // 4):
            # (items wanted: two per compute unit; three where the step has more than half a compute unit's number
            # already, which two would cut in two or not at all)
            wanted = ch.prefill_items_wanted or (2 if 2 * items <= compute_units() else 3) * compute_units()
            splits = max(1, min(wanted // items, keys // ch.prefill_min_run, ch.prefill_max_splits))
            if splits < ch.prefill_min_splits:
                splits = 1                                 # (two runs win less than their join costs)
            if items * 4 > compute_units() and keys * head_dim < ch.prefill_cut_keys_per_item * 64 * items:
                splits = 1                                 # (many items with keys that are not long: whole keys, half rows)
            stretches = (keys + 63) // 64
            run = (stretches + splits - 1) // splits       # stretches of 64 keys per run
        if splits > 1:
            plan["prefill_splits"], plan["prefill_run"] = splits, run
        elif (ch.prefill_half_rows and not tuning & TUNING_HALF_ROWS
              and items <= (3 if head_dim == 64 else 1) * compute_units()):
            # few items whose keys are not cut (short prompts, portions early in a prompt): work items of
            # half the rows, until the items of whole rows number one workgroup less per compute unit than
            # LDS lets it hold (measurements in attention_prefill.hip). Where the keys are cut the items are
            # many already, and half rows were no faster (256 tokens behind 16,128: 2.75 against 2.66 ms a step).
            tuning |= TUNING_HALF_ROWS
        if tuning & TUNING_HALF_ROWS:
            rows = entry("llme_attention_bf16_rows")(head_dim, n_q, n_kv, tuning)
            plan["groups"] = sum((n + rows - 1) // rows for n in new_lens if n >= 2)
            plan["tuning"] = tuning
    if decode:
        longest = max(decode) if plan_len is None else max(plan_len, max(decode))
        pairs = len(decode) * n_kv * ((n_q // n_kv + 15) // 16)
        nsplit = max(1, min((ch.decode_blocks_wanted or compute_units()) // pairs, (longest + MIN_SPLIT - 1) // MIN_SPLIT, MAX_SPLITS))
        if not groups:
            # (a step of decoded tokens only, many of them: by where the pieces land)
            n = cut if cut is not None else decode_cut(decode, n_q, n_kv, head_dim, plan_len, ch)
            if n is not None:
                nsplit = max(1, min(n, (longest + MIN_SPLIT - 1) // MIN_SPLIT, MAX_SPLITS))
        split_len = ((longest + nsplit - 1) // nsplit + 31) // 32 * 32
        plan["split_len"] = split_len
        plan["nsplit"] = (longest + split_len - 1) // split_len
    return plan


def decode_cut(lens, n_q: int, n_kv: int, head_dim: int, plan_len: int | None = None,
               choices: KernelChoices | None = None) -> int | None:
    """Into how many splits a step of single decoded tokens cuts its keys (lens: the keys each request sees,
    in the step's order): the host runtime's estimate (csrc/host/decode_plan.cpp) from where the pieces land
    on the compute units. Asked where a workgroup per request, kv head and 16 query heads is more than half
    the compute units, so that filling the units once would leave the keys whole, and where filling them once
    takes 2 to 6 splits, which one or two more may beat when the requests differ in length (the short ones'
    last pieces are empty). None otherwise (few workgroups: plan_attention cuts to one workgroup per unit)."""
    ch = choices or DEFAULT
    units = ch.decode_blocks_wanted or compute_units()
    tiles = n_kv * ((n_q // n_kv + 15) // 16)
    S = len(lens)
    if S == 0 or ch.decode_cut_most <= 1:
        return None
    longest = max(max(lens), plan_len or 0)
    first = max(1, min(units // (S * tiles), (longest + MIN_SPLIT - 1) // MIN_SPLIT, MAX_SPLITS))
    if first > 6:
        return None
    most = ch.decode_cut_most if first == 1 else min(first + 2, MAX_SPLITS)
    rotates = (first == 1 and ch.decode_rope and GEMV_NORM_MAX_ROWS < S <= qkv_sum_max_rows(True, head_dim, ch)
               and (head_dim == 64 or (head_dim == 128 and S * tiles <= compute_units())))
    apart_us = 0.0
    if first == 1:
        apart_us = (ch.decode_cut_join_us if S > GEMV_NORM_MAX_ROWS else 0.0) + (ch.decode_cut_rope_us if rotates else 0.0)
    from ..runtime import native
    n = native.library().llme_decode_cut((ctypes.c_int * S)(*lens), S, tiles, units, head_dim, longest, first, most,
                                         ch.decode_cut_tbs, ch.decode_cut_key_ns, ch.decode_cut_lone_ns,
                                         ch.decode_cut_piece_us, apart_us, ch.decode_cut_each_us, ch.decode_cut_gain)
    if n < 1:
        raise kernels.KernelError(f"decode_cut: the host runtime refused its arguments (code {n})")
    return n


def cut_hint_name(n_q: int, n_kv: int, head_dim: int) -> tuple:
    """The name under which a recorded step is told its decode_cut (step.plan_hints)."""
    return ("attention_cut", n_q, n_kv, head_dim)


def _step_plan(step, n_q: int, n_kv: int, head_dim: int) -> dict:
    """The step's attention plan for these head counts, made once per step."""
    key = ("attention_plan", n_q, n_kv, head_dim)
    plan = step.extra.get(key)
    if plan is None:
        cut = (getattr(step, "plan_hints", None) or {}).get(cut_hint_name(n_q, n_kv, head_dim))
        plan = step.extra[key] = plan_attention(step.new_lens, step.ctx_lens, n_q, n_kv, head_dim, step.plan_len,
                                                choices=choices_of(step), cut=cut)
    return plan


def attention_bf16(q, k_cache, v_cache, out, q_start, ctx_len, block_table, n_q: int, n_kv: int, head_dim: int,
                   scale: float, window: int, plan: dict, part_o=None, part_ml=None, pre_part_o=None,
                   pre_part_ml=None) -> None:
    """Attention of a step's tokens over bfloat16 pages. q_start [S + 1], ctx_len [S] int32 on
    the device; plan from plan_attention; part_o / part_ml: float32 scratch for split decoding,
    pre_part_o / pre_part_ml: for prompt portions whose keys are cut (plan["prefill_splits"] > 1)."""
    T = q.shape[0]
    S = ctx_len.shape[0]
    require(q, "q", torch.bfloat16, (T, n_q * head_dim))
    require(out, "out", torch.bfloat16, (T, n_q * head_dim))
    require(k_cache, "k_cache", torch.bfloat16, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", torch.bfloat16, (k_cache.shape[0], n_kv, head_dim, page))
    require(q_start, "q_start", torch.int32, (S + 1,))
    require(ctx_len, "ctx_len", torch.int32, (S,))
    require(block_table, "block_table", torch.int32, (S, None))
    if not attention_bf16_supported(q, k_cache, head_dim):
        raise kernels.KernelError(f"attention_bf16: head size {head_dim} must be a multiple of 16 up to 128 and "
                                  f"the page size {page} a multiple of 16")
    if n_q % n_kv:
        raise kernels.KernelError(f"attention: {n_q} query heads do not divide into {n_kv} key/value heads")
    if plan["n_decode"] and plan["nsplit"] > 1:
        require(part_o, "part_o", torch.float32)
        require(part_ml, "part_ml", torch.float32)
        if part_o.numel() < S * n_q * plan["nsplit"] * head_dim or part_ml.numel() < S * n_q * plan["nsplit"] * 2:
            raise kernels.KernelError("attention_bf16: the scratch for split decoding is too small")
    pre_splits = plan.get("prefill_splits", 1) if plan["groups"] else 1
    if pre_splits > 1:
        require(pre_part_o, "pre_part_o", torch.float32)
        require(pre_part_ml, "pre_part_ml", torch.float32)
        if pre_part_o.numel() < T * n_q * pre_splits * head_dim or pre_part_ml.numel() < T * n_q * pre_splits * 2:
            raise kernels.KernelError("attention_bf16: the scratch for prompt portions with cut keys is too small")
    check(entry("llme_attention_bf16")(
        ptr(q), ptr(k_cache), ptr(v_cache), ptr(out), ptr(part_o), ptr(part_ml), ptr(q_start), ptr(ctx_len),
        ptr(block_table), block_table.shape[1], S, n_q, n_kv, head_dim, page, float(scale), int(window),
        plan["n_decode"], plan["split_len"], plan["nsplit"], plan["groups"],
        ptr(work_queue(q.device)) if plan["groups"] else None, T, pre_splits, max(1, int(plan.get("prefill_run", 1))),
        ptr(pre_part_o) if pre_splits > 1 else None, ptr(pre_part_ml) if pre_splits > 1 else None,
        int(plan.get("tuning", 0)), stream()),
        "attention_bf16")


def _fast_attention(q, k_cache, v_cache, out, step, block_table, n_q, n_kv, head_dim, scale, window) -> bool:
    if not attention_bf16_supported(q, k_cache, head_dim) or out.dtype != torch.bfloat16:
        return False
    plan = _step_plan(step, n_q, n_kv, head_dim)
    part_o = part_ml = None
    if plan["n_decode"] and plan["nsplit"] > 1:
        S = step.num_seqs
        part_o = step.buffer("attn.part_o", (S * n_q * plan["nsplit"] * head_dim,), torch.float32)
        part_ml = step.buffer("attn.part_ml", (S * n_q * plan["nsplit"] * 2,), torch.float32)
    pre_part_o = pre_part_ml = None
    if plan["groups"] and plan["prefill_splits"] > 1:
        T = q.shape[0]
        pre_part_o = step.buffer("attn.pre_part_o", (T * n_q * plan["prefill_splits"] * head_dim,), torch.float32)
        pre_part_ml = step.buffer("attn.pre_part_ml", (T * n_q * plan["prefill_splits"] * 2,), torch.float32)
    attention_bf16(q, k_cache, v_cache, out, step.q_start, step.ctx_len, block_table, n_q, n_kv, head_dim, scale,
                   window, plan, part_o, part_ml, pre_part_o, pre_part_ml)
    return True


kernels._fast_attention = _fast_attention

declare("llme_attention_join_project_supported", [_i, _i, _i, _i, _i])
declare("llme_attention_join_project_pays", [_i, _i, _i, _i, _i])
declare("llme_attention_join_project", [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp])
TUNING_NO_JOIN = 1 << 14            # the decode kernel leaves its splits unjoined (see attention_mfma.hip)


def attention_join_project(part_o, part_ml, w_o, out, n_rows: int, n_q: int, head_dim: int, nsplit: int) -> None:
    """out [n_rows, N] float32 += join(part_o, part_ml) w_o^T: the join of the decode kernel's key splits
    (part_o [n_rows, n_q, nsplit, head_dim], part_ml [.., 2], as llme_attention_bf16 leaves them with
    TUNING_NO_JOIN for requests of one token each) and the output projection, w_o blocked bfloat16."""
    require(part_o, "part_o", torch.float32)
    require(part_ml, "part_ml", torch.float32)
    N, _ = kernels._require_weight(w_o, "w_o", torch.bfloat16, n_q * head_dim)
    require(out, "out", torch.float32, (n_rows, N))
    if (not kernels.is_blocked(w_o) or part_o.numel() < n_rows * n_q * nsplit * head_dim
            or part_ml.numel() < n_rows * n_q * nsplit * 2
            or not entry("llme_attention_join_project_supported")(n_rows, n_q, head_dim, nsplit, N)):
        raise kernels.KernelError(f"attention_join_project: {n_rows} rows (at most 16), {n_q} heads of {head_dim}, "
                                  f"{nsplit} splits or the projection's layout are not supported")
    check(entry("llme_attention_join_project")(ptr(part_o), ptr(part_ml), ptr(w_o), ptr(out), n_rows, n_q, head_dim,
                                               nsplit, N, stream()), "attention_join_project")


def _fast_attention_project(q, k_cache, v_cache, o, step, block_table, n_q, n_kv, head_dim, scale, window, w_o, out,
                            accumulate) -> bool:
    """A step of up to 16 decoded tokens whose keys are cut into splits: the splits stay unjoined and
    one kernel joins them and projects. Everything else: not taken (the caller runs the two apart)."""
    T = q.shape[0]
    if (not choices_of(step).join_project or not accumulate or step.fixed_order or T > 16 or T != step.num_seqs
            or out.dtype != torch.float32 or w_o.dtype != torch.bfloat16 or not kernels.is_blocked(w_o)
            or not attention_bf16_supported(q, k_cache, head_dim) or o.dtype != torch.bfloat16):
        return False
    plan = _step_plan(step, n_q, n_kv, head_dim)
    N, K = kernels.weight_shape(w_o)
    if (plan["n_decode"] != T or plan["groups"] or plan["nsplit"] <= 1 or K != n_q * head_dim
            or not entry("llme_attention_join_project_pays")(T, n_q, head_dim, plan["nsplit"], N)):
        return False
    part_o = step.buffer("attn.part_o", (T * n_q * plan["nsplit"] * head_dim,), torch.float32)
    part_ml = step.buffer("attn.part_ml", (T * n_q * plan["nsplit"] * 2,), torch.float32)
    attention_bf16(q, k_cache, v_cache, o, step.q_start, step.ctx_len, block_table, n_q, n_kv, head_dim, scale, window,
                   dict(plan, tuning=int(plan.get("tuning", 0)) | TUNING_NO_JOIN), part_o, part_ml)
    attention_join_project(part_o, part_ml, w_o, out, T, n_q, head_dim, plan["nsplit"])
    return True


kernels._fast_attention_project = _fast_attention_project

declare("llme_attention_decode_rope_bf16", [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i,
                                            _i, _vp])


def attention_decode_rope(qkv, cos, sin, k_cache, v_cache, out, step, block_table, n_q: int, n_kv: int, head_dim: int,
                          scale: float, window: int) -> bool:
    """A step of single decoded tokens whose q/k/v rows [S, (n_q + 2 n_kv) head_dim] are still 32-bit and
    unrotated: rotation, the cache write at each request's position, attention over the pages into out
    [S, n_q head_dim] and the clearing of qkv, in the attention kernel (one workgroup per request and kv
    head, the keys in a single split). False, and nothing done, where the step or the sizes are not such."""
    T = qkv.shape[0]
    ch = choices_of(step)
    if (not ch.decode_rope or not ch.fast_attention or T != step.num_seqs or head_dim not in (64, 128)
            or cos is None or cos.shape[1] * 2 != head_dim or n_q % n_kv or n_q // n_kv > 16
            or qkv.dtype != torch.float32 or out.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16
            or k_cache.shape[2] % 16 or qkv.data_ptr() % 16 or cos.data_ptr() % 16 or sin.data_ptr() % 16
            or k_cache.data_ptr() % 16):
        return False
    plan = _step_plan(step, n_q, n_kv, head_dim)
    if plan["n_decode"] != T or plan["groups"] or plan["nsplit"] != 1:
        return False
    # (measured, ms a decode step at a context of 2,048, apart / inside: 1B sizes 1.238 / 1.203 at 17 requests,
    # 1.340 / 1.297 at 32, 1.758 / 1.724 at 64; 3B 2.950 / 2.889, 3.350 / 3.288, 4.84 / 4.88; 8B 4.369 / 4.298,
    # 4.876 / 4.810, 6.84 / 6.88: with heads of 128 and more workgroups than compute units it does not pay)
    if head_dim == 128 and T * n_kv > compute_units():
        return False
    S = T
    require(qkv, "qkv", torch.float32, (S, (n_q + 2 * n_kv) * head_dim))
    require(cos, "cos", torch.float32, (None, head_dim // 2))
    require(sin, "sin", torch.float32, tuple(cos.shape))
    require(out, "out", torch.bfloat16, (S, n_q * head_dim))
    require(k_cache, "k_cache", torch.bfloat16, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", torch.bfloat16, (k_cache.shape[0], n_kv, head_dim, page))
    require(block_table, "block_table", torch.int32, (S, None))
    check(entry("llme_attention_decode_rope_bf16")(
        ptr(qkv), ptr(cos), ptr(sin), ptr(k_cache), ptr(v_cache), ptr(out), ptr(step.q_start), ptr(step.ctx_len),
        ptr(block_table), block_table.shape[1], S, n_q, n_kv, head_dim, page, float(scale), int(window),
        plan["split_len"], stream()), "attention_decode_rope")
    return True


# --- projections fused with the norm in front of them (decoding) ---------------------------
declare("llme_gemv_norm", [_vp, _vp, _vp, _i, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp])

GEMV_NORM_MAX_ROWS = 16
# Steps of more rows than that and of at most this many cut their q/k/v product over k and add the parts
# into a cleared 32-bit buffer (too few output tiles for the chip otherwise); steps of more rows rotate
# and write the cache in the product's epilogue.
QKV_SUM_MAX_ROWS = 64


def qkv_sum_max_rows(decoded_only: bool, head_dim: int, choices: KernelChoices | None = None) -> int:
    """The most rows of a step whose q/k/v product is cut over k and added into a cleared buffer. A step of
    single decoded tokens keeps that way further: with heads of 64 (choices.qkv_sum_rows_decoding) the
    attention kernel then rotates and writes the cache itself (attention_decode_rope); with heads of 128
    (choices.qkv_sum_rows_decoding_128) the rotation kernel does, and the product's tiles of 96 or 128 rows
    with the rotation in their epilogue are the slower way until then."""
    ch = choices or DEFAULT
    if decoded_only and head_dim == 64 and ch.decode_rope:
        return max(QKV_SUM_MAX_ROWS, ch.qkv_sum_rows_decoding)
    if decoded_only and head_dim == 128:
        return max(QKV_SUM_MAX_ROWS, ch.qkv_sum_rows_decoding_128)
    return QKV_SUM_MAX_ROWS


def gemv_norm_supported(h: torch.Tensor, norm_weight: torch.Tensor, w: torch.Tensor, rows_out: int,
                        gated: bool, choices: KernelChoices | None = None) -> bool:
    """Whether a step may take gemv_norm: the kernel takes the operands, and the choices allow it."""
    return (choices or DEFAULT).fast_gemm and _gemv_norm_fits(h, norm_weight, w, rows_out, gated)


def _gemv_norm_fits(h, norm_weight, w, rows_out: int, gated: bool) -> bool:
    K = h.shape[1]
    if w.dim() not in (2, 5):
        return False
    n_rows, k_w = kernels.weight_shape(w)
    n_out = n_rows // 2 if gated else n_rows
    return (h.dtype == torch.float32 and w.dtype == torch.bfloat16
            and norm_weight.dtype in (torch.float32, torch.bfloat16) and 0 < rows_out <= GEMV_NORM_MAX_ROWS
            and K % 8 == 0 and 16 * (K + 8) * 2 <= 132 * 1024 and k_w == K
            and (not gated or n_out % 16 == 0) and w.data_ptr() % 16 == 0 and h.data_ptr() % 16 == 0
            and norm_weight.data_ptr() % 16 == 0)


def gemv_norm(h: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
              gated: bool = False, rows: torch.Tensor | None = None, tiles_per_round: int = 0,
              grid: int = 0) -> None:
    """out = (rmsnorm(h[rows]) with norm_weight) @ w^T for up to 16 rows of the 32-bit h; gated:
    w holds gate and up rows interleaved in groups of 16 and out = silu(gate) * up in bfloat16."""
    require(h, "h", torch.float32, (None, None))
    K = h.shape[1]
    M = h.shape[0] if rows is None else rows.shape[0]
    if rows is not None:
        require(rows, "rows", torch.int32, (M,))
    require(norm_weight, "norm_weight", (torch.float32, torch.bfloat16), (K,))
    n_rows, _ = kernels._require_weight(w, "w", torch.bfloat16, K)
    N = n_rows // 2 if gated else n_rows
    require(out, "out", torch.bfloat16 if gated else torch.float32, (M, N))
    if not _gemv_norm_fits(h, norm_weight, w, M, gated):
        raise kernels.KernelError(f"gemv_norm: {M} rows (at most 16), K={K} (multiple of 8, 16 rows must fit "
                                  "into LDS) or the operand types are not supported")
    check(entry("llme_gemv_norm")(ptr(h), ptr(rows), ptr(norm_weight), 0 if norm_weight.dtype == torch.float32 else 1,
                                  float(eps), ptr(w), ptr(out), M, N, K, 1 if gated else 0, tiles_per_round, grid,
                                  1 if kernels.is_blocked(w) else 0, stream()),
          "gemv_norm")


declare("llme_gemv_norm_rope", [_vp, _vp, _i, _f, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp,
                                _i, _i, _i, _i, _i, _i, _i, _i, _vp])


def gemv_norm_rope_supported(h, norm_weight, w_qkv, k_cache, n_tokens: int, head_dim: int, rotary_dim: int,
                             choices: KernelChoices | None = None) -> bool:
    return (gemv_norm_supported(h, norm_weight, w_qkv, n_tokens, gated=False, choices=choices) and rotary_dim == head_dim
            and head_dim % 16 == 0 and k_cache.dtype == torch.bfloat16)


def pair_rows_for_rotation(w_qkv: torch.Tensor, n_rotated_heads: int, head_dim: int) -> torch.Tensor:
    """The row order gemv_norm_rope wants of a row-major q/k/v matrix: within each of the first
    n_rotated_heads heads (the q and k heads), dims 0 .. 7, then their rotation partners
    hd/2 .. hd/2 + 7, then 8 .. 15, hd/2 + 8 .. hd/2 + 15 and so on; the other rows (v) as they
    are. head_dim must be a multiple of 16."""
    if w_qkv.dim() != 2 or head_dim % 16 or n_rotated_heads * head_dim > w_qkv.shape[0]:
        raise kernels.KernelError(f"pair_rows_for_rotation: a row-major matrix of whole heads of a multiple of 16 dims, "
                                  f"got {tuple(w_qkv.shape)} for {n_rotated_heads} heads of {head_dim}")
    half = head_dim // 2
    within = torch.arange(head_dim).view(2, half // 8, 8).permute(1, 0, 2).reshape(-1)     # [j][half][8]
    order = (torch.arange(n_rotated_heads)[:, None] * head_dim + within[None, :]).reshape(-1)
    rest = torch.arange(n_rotated_heads * head_dim, w_qkv.shape[0])
    return w_qkv[torch.cat([order, rest]).to(w_qkv.device)].contiguous()


def gemv_norm_rope(h: torch.Tensor, norm_weight: torch.Tensor, eps: float, w_qkv: torch.Tensor,
                   positions: torch.Tensor, seq_idx: torch.Tensor, block_table: torch.Tensor, cos: torch.Tensor,
                   sin: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   n_q: int, n_kv: int, head_dim: int, grid: int = 0) -> None:
    """For up to 16 rows: rmsnorm(h) @ w_qkv^T, q and k heads rotated at the rows' positions, q
    written to q_out (bfloat16) and k, v into the rows' cache pages. w_qkv is the q/k/v matrix with
    the rows of its q and k heads in the order of pair_rows_for_rotation (row-major or blocked);
    what is written has the usual order of dims. Full rotation, head size a multiple of 16."""
    require(h, "h", torch.float32, (None, None))
    M, K = h.shape
    require(norm_weight, "norm_weight", (torch.float32, torch.bfloat16), (K,))
    n_rows, _ = kernels._require_weight(w_qkv, "w_qkv", torch.bfloat16, K)
    if n_rows != (n_q + 2 * n_kv) * head_dim:
        raise kernels.KernelError(f"gemv_norm_rope: w_qkv has {n_rows} rows, the heads need {(n_q + 2 * n_kv) * head_dim}")
    require(positions, "positions", torch.int32, (M,))
    require(seq_idx, "seq_idx", torch.int32, (M,))
    require(block_table, "block_table", torch.int32, (None, None))
    require(cos, "cos", torch.float32, (None, head_dim // 2))
    require(sin, "sin", torch.float32, tuple(cos.shape))
    if cos.data_ptr() % 16 or sin.data_ptr() % 16:
        raise kernels.KernelError("gemv_norm_rope: the rotation tables must be 16-byte aligned")
    require(q_out, "q_out", torch.bfloat16, (M, n_q * head_dim))
    require(k_cache, "k_cache", torch.bfloat16, (None, n_kv, None, head_dim))
    page = k_cache.shape[2]
    require(v_cache, "v_cache", torch.bfloat16, (k_cache.shape[0], n_kv, head_dim, page))
    if not (_gemv_norm_fits(h, norm_weight, w_qkv, M, False) and head_dim % 16 == 0 and k_cache.dtype == torch.bfloat16):
        raise kernels.KernelError(f"gemv_norm_rope: {M} rows (at most 16), head size {head_dim} (multiple of 16) or "
                                  "the operand types are not supported")
    check(entry("llme_gemv_norm_rope")(
        ptr(h), ptr(norm_weight), 0 if norm_weight.dtype == torch.float32 else 1, float(eps), ptr(w_qkv),
        ptr(positions), ptr(seq_idx), ptr(block_table), block_table.shape[1], ptr(cos), ptr(sin), ptr(q_out),
        ptr(k_cache), ptr(v_cache), M, K, n_q, n_kv, head_dim, page, grid, 1 if kernels.is_blocked(w_qkv) else 0,
        stream()), "gemv_norm_rope")
