"""The step function: one batch of (request, its next tokens) through the model.

The reference has three forward entry points: one token of one sequence, one
token of each of B sequences, or a whole sequence token by token
(src/engine.cpp:273-282,488-493,694-716). Here they are one call. A step is a flat
batch of T tokens from several requests; each request brings n >= 1 consecutive
tokens (a whole prompt, a portion of one, or one decoded token) that continue what
its cache holds. The step runs only these tokens, writes their keys and values into
the request's pages, and returns 32-bit logits at the wanted places.
"""
from __future__ import annotations

import ctypes
import gc

from dataclasses import dataclass, field
from typing import Sequence

import torch

from .. import ops

from ..cache import CacheManager, CacheStorage, plan_groups
from ..models.model import DecoderModel


class CapacityError(RuntimeError):
    """The page pool cannot hold the tokens of a step."""


class StepCommittedError(RuntimeError):
    """A step ran and the cache holds its tokens, but what came after it failed (the choice of the
    next tokens, their copy to the host): running the same step again would cache its tokens twice."""


@dataclass
class StepEntry:
    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()        # places among `tokens` whose logits are wanted


def step_layout(mgr: CacheManager, entries: Sequence[StepEntry], page: int, max_blocks: int | None = None):
    """Where a step's integer arrays lie in its one buffer: tokens, positions, request index per
    token, first row of every request (S + 1), tokens cached before the step, slots, one block
    table per group (rows of max_blocks entries; by default as many as the longest request needs),
    the wanted rows. Returns (new_lens, ctx_lens, max_blocks, offsets, sizes, total, T, R, keys,
    wanted)."""
    S = len(entries)
    new_lens = [len(e.tokens) for e in entries]
    keys = (ctypes.c_int64 * S)(*[mgr.key_of(e.request_id) for e in entries])
    lengths = (ctypes.c_long * S)()
    if mgr._lib.llme_cm_lengths(mgr.handle, S, keys, lengths) != 0:
        raise RuntimeError("a request of the step is not live")
    ctx_lens = list(lengths)
    T = sum(new_lens)
    if max_blocks is None:
        max_blocks = max(1, max((c + n + page - 1) // page for c, n in zip(ctx_lens, new_lens)))
    wanted: list[int] = []
    row = 0
    for e, n in zip(entries, new_lens):
        if e.want:
            wanted += [row + int(w) for w in e.want]
        row += n
    R = len(wanted)
    sizes = [T, T, T, S + 1, S, S] + [S * max_blocks] * len(mgr.groups) + [R]
    offsets = [0]
    for s in sizes:
        offsets.append(offsets[-1] + s)
    return new_lens, ctx_lens, max_blocks, offsets, sizes, offsets[-1], T, R, keys, wanted


def fill_step_arrays(mgr: CacheManager, entries: Sequence[StepEntry], layout, h) -> tuple[list[int], int]:
    """Writes the arrays of `step_layout` into the int32 numpy buffer h: the tokens and the wanted
    rows here, everything that the cache manager knows (positions, request indices, first rows,
    lengths, slots and the block tables' rows) by the manager in one call. Returns the requests'
    slots and the step's highest position."""
    new_lens, _, max_blocks, offsets, _, total, _, R, keys, wanted = layout
    if h.shape[0] < total:
        raise RuntimeError("the buffer for the step's integer arrays is too small")
    S = len(entries)
    pos = offsets[0]
    for e, n in zip(entries, new_lens):
        h[pos:pos + n] = e.tokens
        pos += n
    base = h.ctypes.data
    top = mgr._lib.llme_cm_fill_step(mgr.handle, S, keys, (ctypes.c_int * S)(*new_lens), max_blocks,
                                     base + 4 * offsets[1], base + 4 * offsets[2], base + 4 * offsets[3],
                                     base + 4 * offsets[4], base + 4 * offsets[5], base + 4 * offsets[6])
    if top < 0:
        raise RuntimeError(f"the cache manager could not describe the step (code {top})")
    if R:
        h[offsets[-2]:offsets[-1]] = wanted
    return h[offsets[5]:offsets[6]].tolist(), int(top)


class Workspace:
    """Scratch buffers by name, grown on demand and kept, so that steps of the same
    size reuse the same device addresses."""

    def __init__(self, device: torch.device):
        self.device = device
        self._buffers: dict[tuple[str, torch.dtype], torch.Tensor] = {}
        self.keep_replaced = False      # set once a recorded graph holds addresses of these buffers
        self._replaced: list[torch.Tensor] = []
        # buffers that were first asked for (or outgrown) while a graph was being recorded: their memory then
        # belongs to that recording's own pool (see `made_while_recording`)
        self._recorded: dict[tuple[str, torch.dtype], int] = {}
        # the shaped views handed out, by (name, dtype, shape): a step asks for the same ones layer after layer
        self._views: dict[tuple, torch.Tensor] = {}

    def get(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        n = 1
        for d in shape:
            n *= int(d)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < n:
            if buf is not None and self.keep_replaced:
                self._replaced.append(buf)          # a recorded graph may still read and write it
            if torch.cuda.is_current_stream_capturing():
                self._recorded[key] = max(n, 1)
            buf = torch.empty(max(n, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self._views = {k: v for k, v in self._views.items() if k[:2] != key}
        if len(self._views) >= 4096:
            self._views.clear()
        view = self._views[(name, dtype, shape)] = buf[:n].view(shape)
        return view

    def made_while_recording(self) -> bool:
        """Call outside any recording. True if the last recording made buffers: they are replaced by
        buffers of the same sizes made in the ordinary way, and the recording, which holds the old
        addresses, must be thrown away and made again."""
        if not self._recorded:
            return False
        for key, n in self._recorded.items():
            self._buffers[key] = torch.empty(n, dtype=key[1], device=self.device)
        self._views = {k: v for k, v in self._views.items() if k[:2] not in self._recorded}
        self._recorded = {}
        return True


@dataclass
class StepContext:
    """What the parts see of a step. Device tensors are int32."""
    num_tokens: int
    num_seqs: int
    tokens: torch.Tensor            # [T] token ids
    positions: torch.Tensor         # [T] position of each token in its request
    seq_idx: torch.Tensor           # [T] row of the token's request in the per-request arrays
    q_start: torch.Tensor           # [S + 1] first row of each request's tokens in the batch
    ctx_len: torch.Tensor           # [S] tokens cached before this step
    slots: torch.Tensor             # [S] state slot of each request
    block_tables: dict[str, torch.Tensor]      # group -> [S, max_blocks]
    act_dtype: torch.dtype
    workspace: Workspace
    # host copies, for kernels' launch decisions and checks
    new_lens: list[int] = field(default_factory=list)
    ctx_lens: list[int] = field(default_factory=list)
    slot_list: list[int] = field(default_factory=list)
    max_position: int = 0
    # When a step is recorded as a HIP graph and replayed for later steps of the same shape,
    # launch sizes must not follow the momentary lengths: kernels plan for requests of up to
    # `plan_len` tokens instead (None: plan from ctx_lens / new_lens).
    plan_len: int | None = None
    # Sums into the residual stream may be cut over k and added with atomics in whatever order the
    # workgroups finish (faster at few rows; the last bits then differ from run to run). True: every
    # sum has one fixed order, and a step gives the same bits every time it runs.
    fixed_order: bool = False
    extra: dict = field(default_factory=dict)          # per-step notes of kernels (launch plans)
    # a recorded step: what the parts said of their plans when the runner chose the recording (Mixer.decode_plan_hint)
    plan_hints: dict = field(default_factory=dict)
    choices: "ops.KernelChoices | None" = None          # which kernels the operations may choose (the runner's)

    def buffer(self, name: str, shape: tuple[int, ...], dtype: torch.dtype) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype)


class _Staging:
    """Pinned host buffers for the step's integer arrays, used in rotation; a buffer
    is rewritten only after the copy that read it has finished."""

    def __init__(self, count: int = 4):
        self._bufs: list[torch.Tensor | None] = [None] * count
        self._events: list[torch.cuda.Event | None] = [None] * count
        self._next = 0

    def take(self, n: int) -> tuple[torch.Tensor, int]:
        i = self._next
        self._next = (self._next + 1) % len(self._bufs)
        if self._events[i] is not None:
            self._events[i].synchronize()
        buf = self._bufs[i]
        if buf is None or buf.numel() < n:
            buf = torch.empty(max(n, 1024), dtype=torch.int32, pin_memory=True)
            self._bufs[i] = buf
        return buf, i

    def sent(self, i: int) -> None:
        ev = self._events[i] or torch.cuda.Event()
        ev.record()
        self._events[i] = ev


class CacheContext:
    """A page pool with its device memory, for one model: the cache manager's
    bookkeeping plus the tensors the pages live in."""

    def __init__(self, model: DecoderModel, num_pages, page_size: int, max_requests: int,
                 dtype: torch.dtype, device: torch.device):
        specs = model.cache_specs()
        groups = plan_groups(specs, num_pages)
        self.manager = CacheManager(groups, page_size, max_requests)
        self.storage = CacheStorage(specs, groups, page_size, max_requests, dtype, device)
        self.page_size = page_size
        self.max_requests = max_requests
        self.graphs: dict = {}          # recorded decode steps over this pool's tensors, by shape
        self.chain = None               # the last launch that chose its tokens: (recording, requests, its key), see launch_choosing
        self.hints_memo = None          # the parts' plan hints of the last decode step: (requests, width, hints, uses left, the choices)

    def admit(self, request_id) -> int:
        self.chain = None
        slot = self.manager.admit(request_id)
        self.storage.clear_slot(slot)
        return slot

    def slot_admitted(self, slot: int) -> None:
        """A request was admitted by the host runtime itself (the scheduler): its state starts empty."""
        self.chain = None
        self.storage.clear_slot(slot)

    def release(self, request_id) -> None:
        self.chain = None
        self.manager.release(request_id)


class _DecodeRecord:
    """A recorded decode step: the graph, where its logits appear, and the integer arrays it
    reads (a device buffer with a pinned host mirror in the layout of `_build_context` for
    S requests of one token each). Between replays only what changed is rewritten on the host:
    tokens and lengths every step, a block-table entry when a request gets a new page,
    everything when other requests take part."""

    def __init__(self, graph, logits, meta: torch.Tensor, S: int, width: int, groups: list[str],
                 tok_host: torch.Tensor | None = None, draws: bool = False):
        self.graph, self.logits, self.meta = graph, logits, meta
        # a recording that samples reads a temperature and a uniform draw per request from behind the
        # integer arrays (2 S floats that the host sends up with them)
        self.draws = 2 * S if draws else 0
        # pinned, 2 S: where a recording that chooses leaves the chosen tokens, in its two halves in turn (the
        # half is named by the integer behind the arrays), so that a step can be launched before the
        # tokens of the one before it have been read; the same tokens also land in the token array
        # itself, where the next replay finds them without the host
        self.tok_host = tok_host
        self.tok_events = [torch.cuda.Event(), torch.cuda.Event()] if tok_host is not None else None
        self.slot = 1                           # the half the last launch used
        self.launches = [0, 0]                  # launches into each half so far
        self.S, self.width, self.groups = S, width, groups
        sizes = [S, S, S, S + 1, S, S] + [S * width] * len(groups) + [S]
        self.offsets = [0]
        for n in sizes:
            self.offsets.append(self.offsets[-1] + n)
        self.total = self.offsets[-1]
        self.host = torch.zeros(self.total + 1 + self.draws, dtype=torch.int32, pin_memory=True)   # (+ the half's number, the draws)
        self.np = h = self.host.numpy()
        self.np_draws = self.host.view(torch.float32).numpy()[self.total + 1:]
        o, G = self.offsets, len(groups)
        h[o[2]:o[3]] = range(S)                 # request index of each token
        h[o[3]:o[4]] = range(S + 1)             # first row of each request
        h[o[6 + G]:o[7 + G]] = range(S)         # wanted rows
        self.key_list: list[int] | None = None
        self.keys = None
        self.done = (ctypes.c_int * max(G * S, 1))()        # per group and request: table entries written so far
        self.serials = (ctypes.c_int64 * S)()               # which admission of its key sits in each place
        self.event: torch.cuda.Event | None = None
        self.scratch = None

    def refresh(self, mgr: CacheManager, entries: Sequence[StepEntry] | None, keys=None, slot: int = 0,
                tokens: Sequence[int] | None = None, temperature: float = 0.0,
                uniforms: Sequence[float] | None = None) -> None:
        """The step's tokens come in `entries` or in `tokens`; with neither they are the ones the last
        replay chose and left in the device's array. Everything else is rewritten as always.
        temperature, uniforms: for a recording that samples, the step's temperature and draws."""
        if self.event is not None:
            self.event.synchronize()            # the last copy has read the host mirror
        S, width, o, h = self.S, self.width, self.offsets, self.np
        if keys is not None:                    # the caller has them as an array already
            self.keys, self.key_list = keys, None
        else:
            keys = [mgr.key_of(e.request_id) for e in entries]
            if keys != self.key_list:
                self.key_list = keys
                self.keys = (ctypes.c_int64 * S)(*keys)
        if entries is not None:
            tokens = [e.tokens[0] for e in entries]
        if tokens is not None:
            h[o[0]:o[1]] = tokens
        h[self.total] = slot
        if self.draws:
            if uniforms is None or len(uniforms) != S:
                raise ValueError("a recording that samples needs a draw per request")
            self.np_draws[:S] = temperature
            self.np_draws[S:] = uniforms
        # lengths (tokens cached before this step), slots and the block-table entries that are new,
        # straight from the C++ manager into the pinned mirror
        base = h.ctypes.data
        rc = mgr._lib.llme_cm_fill_decode(mgr.handle, S, self.keys, width, base + 4 * o[4], base + 4 * o[5],
                                          base + 4 * o[6], self.done, self.serials)
        if rc != 0:
            raise RuntimeError(f"a request of the recorded step is not live (code {rc})")
        h[o[1]:o[2]] = h[o[4]:o[5]]             # the new token's position
        first = 0 if tokens is not None else o[1]
        self.meta[first:self.total + 1 + self.draws].copy_(self.host[first:], non_blocking=True)
        if self.event is None:
            self.event = torch.cuda.Event()
        self.event.record()


class PendingTokens:
    """A launched step that chooses its tokens itself, which have not been fetched yet."""

    def __init__(self, rec: _DecodeRecord, slot: int, launch: int):
        self.rec, self.slot, self.launch = rec, slot, launch


class ModelRunner:
    """A loaded model on a device plus the scratch memory its steps use."""

    GRAPH_BLOCK_BUCKET = 64         # block-table widths of recorded steps are multiples of this
    GRAPH_LIMIT = 192               # recorded steps kept per page pool; the least recently used one goes first

    def __init__(self, model: DecoderModel, dtype: torch.dtype, device: torch.device, use_graphs: bool = True,
                 deterministic: bool = False, choices: "ops.KernelChoices | None" = None):
        self.model = model
        # what the operations may choose for this runner's steps (a copy of its own: see ops/choices.py)
        self.choices = choices if choices is not None else ops.KernelChoices()
        self.deterministic = bool(deterministic)
        self.dtype = dtype
        self.device = device
        self.workspace = Workspace(device)
        self._staging = _Staging()
        self._meta_dev: torch.Tensor | None = None
        self.use_graphs = bool(use_graphs) and model.tree_graph_safe()
        self.graph_replays = 0

    def new_cache(self, num_pages, page_size: int, max_requests: int) -> CacheContext:
        return CacheContext(self.model, num_pages, page_size, max_requests, self.dtype, self.device)

    # ------------------------------------------------------------------------------
    def step(self, cache: CacheContext, entries: Sequence[StepEntry], max_position: int | None = None
             ) -> torch.Tensor | None:
        """Runs one step. Every entry's request must be admitted to `cache`. Pages for
        all entries are reserved first (CapacityError, with nothing changed, if the
        pools are short); then the tokens run as one batch; then the requests are
        that much longer. Returns logits [sum(len(want)), vocab] on the device, in
        the order of the entries and of their `want` lists, or None. The tensor is scratch
        memory of this runner (or of the recorded step that was replayed): it holds these
        logits until the runner's next step, which writes its own into the same place; a
        caller that needs them longer copies them."""
        mgr = cache.manager
        if not entries:
            return None
        cache.chain = None                      # (a later launch that chooses takes its tokens from the host again)
        vocab = self.model.vocab_size
        seen = set()
        for e in entries:
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.request_id!r}: a step entry needs at least one token")
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} appears twice in one step")
            seen.add(e.request_id)
            if min(e.tokens) < 0 or max(e.tokens) >= vocab:         # (the passing case without a loop in Python)
                bad = next(t for t in e.tokens if not 0 <= int(t) < vocab)
                raise ValueError(f"token id {bad} out of range [0, {vocab})")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is not among "
                                     f"{len(e.tokens)} tokens")
            end = mgr.length(e.request_id) + len(e.tokens)
            if max_position is not None and end > max_position:
                raise ValueError(f"request {e.request_id!r}: {end} tokens exceed the position limit "
                                 f"{max_position}")
        # pages for every entry, or none
        if not mgr.reserve_batch([(e.request_id, len(e.tokens)) for e in entries]):
            need = {g: sum(mgr.pages_needed(e.request_id, len(e.tokens))[g] for e in entries) for g in mgr.groups}
            raise CapacityError(f"the step needs {need} more pages, free are "
                                f"{({g: mgr.free_pages(g) for g in mgr.groups})}")

        if self.use_graphs and all(len(e.tokens) == 1 and len(e.want) == 1 and e.want[0] == 0 for e in entries):
            logits = self._decode_step_graphed(cache, entries)
        else:
            ctx, logit_rows = self._build_context(cache, entries)
            logits = self.model.forward(ctx, cache.storage.layers, logit_rows)
        for e in entries:
            mgr.commit(e.request_id, len(e.tokens))
        return logits

    # ------------------------------------------------------------------------------
    def _decode_step_graphed(self, cache: CacheContext, entries: Sequence[StepEntry]) -> torch.Tensor:
        """A step of single decoded tokens, all wanting logits: the launch sequence depends
        only on the number of requests and on the width of the block tables, so it is
        recorded once as a HIP graph and replayed; only the integer arrays change."""
        mgr = cache.manager
        lengths = [mgr.length(e.request_id) for e in entries]
        hints = self._decode_hints(cache, lengths)
        rec = self._decode_record(cache, entries, max(lengths), choose=None, hints=hints)
        rec.refresh(mgr, entries)
        rec.graph.replay()
        self.graph_replays += 1
        return rec.logits

    def _decode_width(self, cache: CacheContext, longest: int) -> int:
        need = (longest + cache.page_size) // cache.page_size
        bucket = self.GRAPH_BLOCK_BUCKET
        return (need + bucket - 1) // bucket * bucket

    HINTS_REUSED = 32               # steps of the same requests that go by the hints of the first

    def _decode_hints(self, cache: CacheContext, lengths: Sequence[int], ids: Sequence | None = None) -> tuple:
        """What the parts' launch plans make of these lengths (tokens cached before the step), for a step
        recorded at the width of block table that the longest needs. With ids: what they made of them a few
        steps ago, while the same requests go on in the same order at the same width (each has grown by one
        per step, which changes no plan much; asking costs the host some 15 us a step)."""
        width = self._decode_width(cache, max(lengths))
        memo = cache.hints_memo
        chosen = self.choices.key()
        if (ids is not None and memo is not None and memo[1] == width and memo[3] > 0 and memo[0] == ids
                and memo[4] == chosen):
            cache.hints_memo = (memo[0], width, memo[2], memo[3] - 1, chosen)
            return memo[2]
        hints = self.model.decode_plan_hints([int(n) + 1 for n in lengths], width * cache.page_size, self.choices)
        if ids is not None:
            cache.hints_memo = (list(ids), width, hints, self.HINTS_REUSED, chosen)
        return hints

    def _decode_key(self, cache: CacheContext, S: int, longest: int, choose: str | None, hints: tuple = ()):
        # (a recording holds the launches that the choices of its time led to, and those that the parts
        # planned from the requests' lengths: hints)
        return (S, self._decode_width(cache, longest), choose, self.choices.key(), hints)

    def _decode_record(self, cache: CacheContext, entries: Sequence[StepEntry] | None, longest: int,
                       choose: str | None, S: int | None = None, hints: tuple = ()):
        """The recording for this many requests and this width of block tables. choose None: it ends
        at the logits. "greedy": the argmax is behind the model, its result written into pinned host
        memory. "sampled": the sampling kernels instead, with a temperature and a uniform draw per
        request that the host sends up with the integer arrays. Made at its first use (which needs
        the entries)."""
        page = cache.page_size
        mgr = cache.manager
        S = len(entries) if S is None else S
        key = self._decode_key(cache, S, longest, choose, hints)
        width = key[1]
        rec = cache.graphs.pop(key, None)
        if rec is not None:
            cache.graphs[key] = rec                      # (most recently used last)
        if rec is None:
            if entries is None:
                raise RuntimeError("a step that takes its tokens from the step before has no recording to run in")
            while len(cache.graphs) >= self.GRAPH_LIMIT:
                del cache.graphs[next(iter(cache.graphs))]
            # The step is recorded without having run: a part's step need not be repeatable (a mixer that
            # advances a state would count the token twice), and the first replay is its first run.
            # The recorded step reads its integer arrays from a buffer of its own.
            ops.load_kernels()                          # (no code object is loaded inside a recording)
            groups = len(mgr.groups)
            total = 7 * S + 1 + groups * S * width
            meta = torch.zeros(total + 1 + 2 * S + 64, dtype=torch.int32, device=self.device)
            ctx, logit_rows = self._build_context(cache, entries, max_blocks=width, plan_len=width * page, dev=meta)
            ctx.plan_hints = dict(hints)
            tok_host = scratch = temp_dev = uni_dev = None
            if choose == "sampled":
                temp_dev = meta[total + 1:total + 1 + S].view(torch.float32)
                uni_dev = meta[total + 1 + S:total + 1 + 2 * S].view(torch.float32)
            if choose:
                # pinned host memory is mapped into the device's address space: the kernel writes
                # the tokens where the host reads them, without a copy of its own; the argmax's
                # scratch belongs to the recording (the one that plain calls share may be replaced)
                tok_host = torch.zeros(2 * S, dtype=torch.int32, pin_memory=True)
                scratch = ops.sampling_scratch(self.device, S, self.model.vocab_size)
            torch.cuda.synchronize(self.device)
            self.workspace.keep_replaced = True
            # Scratch buffers that the step is the first to ask for are made while it is recorded and
            # belong to the recording's own memory pool, which later steps of other kinds must not be
            # handed: they are made again outside, and the step is recorded once more with those.
            # No garbage collection while launches are recorded: a collection that finds an engine nobody
            # holds any more destroys its recordings and frees their memory, which the runtime refuses
            # while a stream is being recorded (the process then ends in the destructor's error).
            collecting = gc.isenabled()
            gc.disable()
            try:
                for attempt in range(3):
                    ctx.extra.clear()                   # (notes of the pass before: launch plans, what was left cleared)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        logits = self.model.forward(ctx, cache.storage.layers, logit_rows)
                        if choose == "sampled":
                            ops.sample_into(logits, temp_dev, uni_dev, tok_host.data_ptr(), scratch,
                                            also_ptr=meta.data_ptr(), slot_ptr=meta.data_ptr() + 4 * total)
                        elif choose:
                            ops.argmax_into(logits, tok_host.data_ptr(), scratch, also_ptr=meta.data_ptr(),
                                            slot_ptr=meta.data_ptr() + 4 * total)
                    if not self.workspace.made_while_recording():
                        break
                    del graph, logits
                else:
                    raise RuntimeError("a decode step asks for new scratch buffers every time it is recorded")
            finally:
                if collecting:
                    gc.enable()
            cache.graphs[key] = rec = _DecodeRecord(graph, logits, meta, S, width, list(mgr.groups), tok_host,
                                                    draws=choose == "sampled")
            rec.scratch = scratch                       # (kept alive: the graph holds its addresses)
        return rec

    def step_choosing(self, cache: CacheContext, entries: Sequence[StepEntry], max_position: int | None = None,
                    temperature: float = 0.0, uniforms: Sequence[float] | None = None) -> list[int] | None:
        """The next token of every entry, greedy or (temperature > 0, a uniform draw per entry in
        `uniforms`) sampled, for a step of single decoded tokens that all want one: bookkeeping in two
        calls into the host runtime, the choice inside the recorded graph, its result read from pinned
        memory. None if the step is not of that kind (then `step` and a sampler do it)."""
        if not self.use_graphs or not entries or (temperature > 0 and uniforms is None):
            return None
        ids = []
        for e in entries:
            if len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0:
                return None
            ids.append(e.request_id)
        pending = self.launch_choosing(cache, ids, [int(e.tokens[0]) for e in entries], max_position,
                                     temperature=temperature, uniforms=uniforms)
        try:
            return self.chosen_tokens(pending)
        except BaseException as e:
            raise StepCommittedError(f"the step ran, but its tokens could not be fetched: {e}") from e

    def launch_choosing(self, cache: CacheContext, ids: Sequence, tokens: Sequence[int] | None,
                      max_position: int | None = None, temperature: float = 0.0,
                      uniforms: Sequence[float] | None = None) -> "PendingTokens | None":
        """Launches a step of one token for each of the live requests `ids` whose choices (greedy, or
        sampled at `temperature` with the draws `uniforms`, one per request) `chosen_tokens` fetches
        later. tokens None: every request's token is the one that the launch
        before this one chose for it, taken where that step's argmax left it on the device, so that
        this step can be launched before the host has seen those tokens (the host's work for a step,
        some 40 us, then runs beside the device's instead of in front of it). That needs the launch
        before to have been of the same requests in the same recording; where it was not (the first
        step, or the block tables have outgrown the recording), None is returned and nothing is
        done: the caller fetches the tokens and passes them. At most one launch may be waiting for
        its `chosen_tokens` when another is made."""
        S = len(ids)
        if len(set(ids)) != S:
            raise ValueError("a request appears twice in one step")
        choose = "sampled" if temperature and temperature > 0 else "greedy"
        if choose == "sampled" and (uniforms is None or len(uniforms) != S):
            raise ValueError("sampling needs a uniform draw per request")
        if tokens is not None:
            vocab = self.model.vocab_size
            if len(tokens) != S:
                raise ValueError(f"{len(tokens)} tokens for {S} requests")
            for t in tokens:
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"token id {t} out of range [0, {vocab})")
        mgr = cache.manager
        keys = (ctypes.c_int64 * S)(*[mgr.key_of(r) for r in ids])
        lengths = (ctypes.c_int * S)()
        if tokens is None:
            # (asked before anything changes: a chain that cannot go on leaves the manager as it was)
            last = cache.chain
            if last is None or last[1] != list(ids):
                return None
            longest = max(mgr.length(r) for r in ids)
            # (the chain keeps the plan it began with: every request has grown by one since)
            if (self._decode_key(cache, S, longest, choose, last[2][-1]) != last[2]
                    or cache.graphs.get(last[2]) is not last[0]):
                return None
        # lengths, the position limit and the pages in one call; a call that fails has changed nothing
        rc = mgr._lib.llme_cm_decode_begin(mgr.handle, S, keys, lengths, int(max_position or 0))
        if rc < 0:
            raise RuntimeError(f"a request of the step is not live (code {rc})")
        longest = max(lengths)
        if rc == 2:
            raise ValueError(f"{longest + 1} tokens exceed the position limit {max_position}")
        if rc == 0:
            need = {g: sum(mgr.pages_needed(r, 1)[g] for r in ids) for g in mgr.groups}
            raise CapacityError(f"the step needs {need} more pages, free are "
                                f"{({g: mgr.free_pages(g) for g in mgr.groups})}")
        hints = cache.chain[2][-1] if tokens is None else self._decode_hints(cache, lengths, list(ids))
        key = self._decode_key(cache, S, longest, choose, hints)
        if key in cache.graphs or tokens is None:
            rec = self._decode_record(cache, None, longest, choose, S=S, hints=hints)
        else:                                   # (a new recording is made from entries)
            rec = self._decode_record(cache, [StepEntry(r, [t], [0]) for r, t in zip(ids, tokens)], longest, choose,
                                      hints=hints)
        slot = 1 - rec.slot
        rec.refresh(mgr, None, keys, slot=slot, tokens=tokens, temperature=float(temperature or 0.0), uniforms=uniforms)
        rec.graph.replay()
        rec.tok_events[slot].record()
        rec.slot = slot
        rec.launches[slot] += 1                 # (what an older launch left in this half is gone)
        self.graph_replays += 1
        mgr._lib.llme_cm_commit_batch(mgr.handle, S, keys, 1)
        cache.chain = (rec, list(ids), key)
        return PendingTokens(rec, slot, rec.launches[slot])

    def chosen_tokens(self, pending: "PendingTokens") -> list[int]:
        """The tokens a launched step chose (waits for it). They can be fetched until the launch
        after the next one, which uses the same half of the recording's token buffer."""
        rec, slot = pending.rec, pending.slot
        if rec.launches[slot] != pending.launch:
            raise RuntimeError("the tokens of this launch have been overwritten: two later steps were launched "
                               "before they were fetched")
        rec.tok_events[slot].synchronize()
        return rec.tok_host[slot * rec.S:(slot + 1) * rec.S].tolist()

    # ------------------------------------------------------------------------------
    def _build_context(self, cache: CacheContext, entries: Sequence[StepEntry], max_blocks: int | None = None,
                       plan_len: int | None = None, dev: torch.Tensor | None = None):
        mgr = cache.manager
        S = len(entries)
        groups = list(mgr.groups)
        layout = step_layout(mgr, entries, cache.page_size, max_blocks)
        new_lens, ctx_lens, max_blocks, offsets, sizes, total, T, R = layout[:8]
        host, idx = self._staging.take(total)
        slot_list, top = fill_step_arrays(mgr, entries, layout, host.numpy())

        if dev is None:
            if self._meta_dev is None or self._meta_dev.numel() < total:
                self._meta_dev = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
            dev = self._meta_dev
        elif dev.numel() < total:
            raise RuntimeError("the recorded step's integer buffer is too small for this step")
        dev[:total].copy_(host[:total], non_blocking=True)
        self._staging.sent(idx)

        def view(k: int, shape=None):
            t = dev[offsets[k]:offsets[k + 1]]
            return t if shape is None else t.view(shape)

        ctx = StepContext(
            num_tokens=T, num_seqs=S, tokens=view(0), positions=view(1), seq_idx=view(2), q_start=view(3),
            ctx_len=view(4), slots=view(5),
            block_tables={g: view(6 + gi, (S, max_blocks)) for gi, g in enumerate(groups)},
            act_dtype=self.dtype, workspace=self.workspace, new_lens=new_lens, ctx_lens=ctx_lens,
            slot_list=slot_list, max_position=top,
            plan_len=plan_len, fixed_order=self.deterministic, choices=self.choices)
        logit_rows = view(len(sizes) - 1) if R else None
        return ctx, logit_rows
