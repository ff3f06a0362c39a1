"""Continuous batching above the step function.

State machine, knobs and finish reasons are the reference's
`ContinuousBatchScheduler` (src/scheduler.cpp:136-319): requests wait in a FIFO,
are admitted while fewer than `max_concurrent` are live (no page check at
admission), prefill under one token budget per step shared in admission order,
then decode one token per step; a sequence ends with "stop" (an EOS id was
sampled; it is not appended), "length" (`max_new_tokens` reached, or 0 asked) or
"capacity" (the page pool cannot hold its next tokens; what it generated so far is
kept; nothing is preempted or recomputed). Results come back in enqueue order.
One more reason, "error", has no counterpart there: a step ran, but the choice of
its next tokens failed afterwards; its sequences cannot go on and keep what they had.

What differs from the reference: a step is ONE mixed batch. Prompt portions and
the single tokens of decoding requests go through the model together, and because
pages are reserved before the batch runs, running out of pages is decided here, on
the host, in the reference's order (prompt portions take pages first, then
decoding requests). A request whose prompt ends in step k decodes first in step
k + 1 (the reference does both in step k); token streams are the same. Pages of a
finished request go back at the end of the step in which it finished, which is
when the reference's next step would find them.
"""
from __future__ import annotations

import ctypes
import weakref
from dataclasses import dataclass
from typing import Protocol, Sequence

from ..runtime import native
from .step import StepCommittedError, StepEntry

_REASONS = {1: "stop", 2: "length", 3: "capacity", 4: "error"}


def rounds_order(n: int, per_round: int) -> list[int]:
    """For n items ranked by size (rank 0 the largest) that are dealt out to per_round places in turn
    (item at position p goes to place p % per_round): the rank to put at each position so that the places'
    sums come out even. The ranks are cut into rounds of per_round; the last round, which may be short and so
    lands on the first places, stands in its own order, the round before it reversed, and so on in turns: a
    place that got the smallest of one round gets the largest of the next."""
    if per_round <= 0 or n <= per_round:
        return list(range(n))
    rounds = [list(range(a, min(a + per_round, n))) for a in range(0, n, per_round)]
    for back, ranks in enumerate(reversed(rounds)):
        if back % 2 == 1:
            ranks.reverse()
    return [rank for ranks in rounds for rank in ranks]


@dataclass
class SequenceResult:
    seq_id: int
    prompt_len: int
    token_ids: list[int]
    finish_reason: str

    def __repr__(self) -> str:
        return f"<SequenceResult seq_id={self.seq_id} finish={self.finish_reason} len={len(self.token_ids)}>"


class StepBackend(Protocol):
    """What the scheduler needs of an engine."""
    vocab_size: int
    max_pos: int
    eos_token_ids: Sequence[int]

    def open_cache(self, block_manager, max_requests: int): ...           # -> object with .manager (a CacheManager)
    def run_step(self, cache, entries: list[StepEntry], draws: list[tuple[int, int]],
                 temperature: float, seed: int) -> list[int]: ...          # next token per wanted row


class ContinuousBatchScheduler:
    """The decisions are made in C++ (csrc/host/scheduler.cpp: admission, the step's batch under
    the token budget, what happens when pages run out, who finishes and why); this class checks
    the requests, carries each planned batch to the engine's step function and brings the
    sampled tokens back. The cache the engine opens must have a `manager` that is the C++ cache
    manager's face; if it has a `slot_admitted(slot)` method, it is told the slot of every
    request that is admitted (to clear its fixed-size state)."""

    def __init__(self, engine: StepBackend, block_manager, max_concurrent: int = 64,
                 max_prefill_tokens_per_step: int = 256, temperature: float = 0.0, seed: int = 0):
        if max_concurrent <= 0:
            raise ValueError("ContinuousBatchScheduler: max_concurrent must be >= 1")
        if max_prefill_tokens_per_step <= 0:
            raise ValueError("ContinuousBatchScheduler: max_prefill_tokens_per_step must be >= 1")
        if temperature < 0:
            raise ValueError("ContinuousBatchScheduler: temperature must be >= 0")
        self.engine = engine
        self.block_manager = block_manager
        self.max_concurrent = int(max_concurrent)
        self._budget = int(max_prefill_tokens_per_step)
        self.temperature = float(temperature)
        self.seed = int(seed)
        # Sequence ids are the requests' keys in the cache manager, and every scheduler counts from
        # 0: two schedulers over one block manager would take each other's keys, and a second one
        # that asks for more slots would have the pool replaced under the first.
        other = getattr(block_manager, "_scheduler", None)
        other = other() if other is not None else None
        if other is not None and not other.idle:
            raise ValueError("ContinuousBatchScheduler: this block manager already serves a scheduler with "
                             "requests in flight; give every scheduler a BlockManager of its own")
        self._cache = engine.open_cache(block_manager, self.max_concurrent)
        try:
            block_manager._scheduler = weakref.ref(self)
        except AttributeError:
            pass                                        # (a stand-in manager without attributes)
        self._lib = native.library()
        self._h = self._lib.llme_sched_create(self._cache.manager.handle, self.max_concurrent, self._budget)
        if not self._h:
            raise ValueError("ContinuousBatchScheduler: the scheduler refused its sizes")
        # an engine whose decode kernel deals a step's requests out to the compute units in turn says after
        # how many it has been round once (rounds_order)
        self._lib.llme_sched_set_decode_round(self._h, max(0, int(getattr(engine, "decode_round", 0) or 0)))
        # and an engine whose products run a few rows more than a multiple of some number of rows in launches
        # of their own says which (rows, most): the step's last prompt portion then leaves those few for the
        # next step
        rows, over = getattr(engine, "step_rows_round", None) or (0, 0)
        if rows > 0 and 0 < over < rows:
            self._lib.llme_sched_set_row_round(self._h, int(rows), int(over))
        n = self.max_concurrent
        self._admitted = (ctypes.c_int * n)()
        self._entry_seq = (ctypes.c_int64 * n)()
        self._entry_count = (ctypes.c_int * n)()
        self._entry_want = (ctypes.c_int * n)()
        self._entry_gen = (ctypes.c_long * n)()
        self._tokens = None
        self._size_tokens()
        self.steps = 0

    def __del__(self):
        if getattr(self, "_h", None):
            self._lib.llme_sched_destroy(self._h)
            self._h = None

    def _size_tokens(self) -> None:
        self._tokens_cap = self._budget + self.max_concurrent
        self._tokens = (ctypes.c_int * self._tokens_cap)()

    # ---- knobs ----
    @property
    def budget(self) -> int:
        return self._budget

    @budget.setter
    def budget(self, value: int) -> None:
        if value <= 0:
            raise ValueError("ContinuousBatchScheduler: max_prefill_tokens_per_step must be >= 1")
        self._budget = int(value)
        self._lib.llme_sched_set_budget(self._h, self._budget)
        self._size_tokens()

    # ---- requests ----
    def enqueue(self, prompt: Sequence[int], max_new_tokens: int) -> int:
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("enqueue: prompt is empty")
        if max_new_tokens < 0:
            raise ValueError("enqueue: max_new_tokens negative")
        V = self.engine.vocab_size
        for t in prompt:
            if t < 0 or t >= V:
                raise ValueError(f"enqueue: token id {t} out of range [0, {V})")
        if len(prompt) + int(max_new_tokens) > self.engine.max_pos:
            raise ValueError("enqueue: prompt + max_new_tokens exceeds RoPE max_pos")
        arr = (ctypes.c_int * len(prompt))(*prompt)
        return int(self._lib.llme_sched_enqueue(self._h, arr, len(prompt), int(max_new_tokens)))

    @property
    def idle(self) -> bool:
        return bool(self._lib.llme_sched_idle(self._h))

    @property
    def results(self) -> list[SequenceResult]:
        out = []
        seq_id, plen, ntok, reason = ctypes.c_int64(), ctypes.c_long(), ctypes.c_long(), ctypes.c_int()
        for i in range(self._lib.llme_sched_num_results(self._h)):
            self._lib.llme_sched_result_info(self._h, i, ctypes.byref(seq_id), ctypes.byref(plen), ctypes.byref(ntok),
                                             ctypes.byref(reason))
            toks = (ctypes.c_int * max(ntok.value, 1))()
            self._lib.llme_sched_result_tokens(self._h, i, toks)
            out.append(SequenceResult(int(seq_id.value), int(plen.value), list(toks[:ntok.value]),
                                      _REASONS.get(reason.value, "")))
        return out

    def clear_results(self) -> None:
        self._lib.llme_sched_clear_results(self._h)

    # ---- one step ----
    def step(self) -> bool:
        n_admitted = ctypes.c_int()
        E = self._lib.llme_sched_plan(self._h, ctypes.byref(n_admitted), self._admitted, self._entry_seq,
                                      self._entry_count, self._entry_want, self._entry_gen, self._tokens,
                                      self._tokens_cap)
        if E < 0:
            why = {-1: "a sequence id of this scheduler is already live in the cache (another user of the same "
                       "block manager holds that key)",
                   -2: f"the cache it was given has fewer slots than max_concurrent = {self.max_concurrent}",
                   -6: "the step before was neither completed nor aborted, or the batch does not fit its buffers"}
            raise RuntimeError(f"the scheduler could not plan a step (code {E}): {why.get(E, 'host runtime error')}")
        told = getattr(self._cache, "slot_admitted", None)
        if told is not None:
            for i in range(n_admitted.value):
                told(self._admitted[i])
        entries: list[StepEntry] = []
        draws: list[tuple[int, int]] = []
        pos = 0
        for i in range(E):
            n, seq_id = self._entry_count[i], int(self._entry_seq[i])
            want = [n - 1] if self._entry_want[i] else []
            entries.append(StepEntry(seq_id, self._tokens[pos:pos + n], want))
            if want:
                draws.append((seq_id, int(self._entry_gen[i])))
            pos += n
        sampled: list[int] = []
        if entries:
            try:
                sampled = self.engine.run_step(self._cache, entries, draws, self.temperature, self.seed)
                if len(sampled) != len(draws):
                    raise StepCommittedError(f"the step returned {len(sampled)} tokens for {len(draws)} wanted rows")
            except StepCommittedError:
                # the batch ran and the cache holds its tokens, but the next tokens never arrived: no
                # sequence of the batch can go on, each ends with "error" and keeps what it had
                self._lib.llme_sched_fail(self._h)
                raise
            except BaseException:
                # the batch did not run: the prompts stay where they were and the next step offers
                # the same portions again (the step function changes nothing when it fails before
                # it commits)
                self._lib.llme_sched_abort(self._h)
                raise
            self.steps += 1
        eos = [int(t) for t in self.engine.eos_token_ids]
        rc = self._lib.llme_sched_complete(self._h, (ctypes.c_int * max(len(sampled), 1))(*[int(t) for t in sampled]),
                                           len(sampled), (ctypes.c_int * max(len(eos), 1))(*eos), len(eos))
        if rc < 0:
            raise RuntimeError(f"the scheduler could not take the step's tokens (code {rc})")
        return not self.idle

    def run_until_idle(self) -> None:
        while self.step():
            pass
