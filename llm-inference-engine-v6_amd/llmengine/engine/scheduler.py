"""Continuous batching above the step function.

State machine, knobs and finish reasons are the reference's
`ContinuousBatchScheduler` (src/scheduler.cpp:136-319): requests wait in a FIFO,
are admitted while fewer than `max_concurrent` are live (no page check at
admission), prefill under one token budget per step shared in admission order,
then decode one token per step; a sequence ends with "stop" (an EOS id was
sampled; it is not appended), "length" (`max_new_tokens` reached, or 0 asked) or
"capacity" (the page pool cannot hold its next tokens; what it generated so far is
kept; nothing is preempted or recomputed). Results come back in enqueue order.

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

from collections import deque
from dataclasses import dataclass, field
from typing import Protocol, Sequence

from .step import StepEntry

WAITING, PREFILLING, RUNNING, FINISHED = "WAITING", "PREFILLING", "RUNNING", "FINISHED"


@dataclass
class SequenceResult:
    seq_id: int
    prompt_len: int
    token_ids: list[int]
    finish_reason: str

    def __repr__(self) -> str:
        return f"<SequenceResult seq_id={self.seq_id} finish={self.finish_reason} len={len(self.token_ids)}>"


@dataclass
class Sequence_:
    seq_id: int
    token_ids: list[int]
    prompt_len: int
    max_new_tokens: int
    state: str = WAITING
    prefill_cursor: int = 0
    finish_reason: str = ""

    @property
    def generated(self) -> int:
        return len(self.token_ids) - self.prompt_len


class StepBackend(Protocol):
    """What the scheduler needs of an engine."""
    vocab_size: int
    max_pos: int
    eos_token_ids: Sequence[int]

    def open_cache(self, block_manager, max_requests: int): ...           # -> object with .manager, .admit, .release
    def run_step(self, cache, entries: list[StepEntry], draws: list[tuple[int, int]],
                 temperature: float, seed: int) -> list[int]: ...          # next token per wanted row


class ContinuousBatchScheduler:
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
        self._cache = engine.open_cache(block_manager, self.max_concurrent)
        self._waiting: deque[Sequence_] = deque()
        self._prefilling: list[Sequence_] = []
        self._running: list[Sequence_] = []
        self._results: list[SequenceResult] = []
        self._next_id = 0
        self.steps = 0

    # ---- knobs ----
    @property
    def budget(self) -> int:
        return self._budget

    @budget.setter
    def budget(self, value: int) -> None:
        if value <= 0:
            raise ValueError("ContinuousBatchScheduler: max_prefill_tokens_per_step must be >= 1")
        self._budget = int(value)

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
        seq = Sequence_(self._next_id, prompt, len(prompt), int(max_new_tokens))
        self._next_id += 1
        self._waiting.append(seq)
        return seq.seq_id

    @property
    def idle(self) -> bool:
        return not (self._waiting or self._prefilling or self._running)

    @property
    def results(self) -> list[SequenceResult]:
        return sorted(self._results, key=lambda r: r.seq_id)

    def clear_results(self) -> None:
        self._results.clear()

    # ---- one step ----
    def _finish(self, seq: Sequence_, reason: str) -> None:
        seq.state = FINISHED
        seq.finish_reason = reason

    def _retire(self) -> None:
        for lst in (self._prefilling, self._running):
            keep = []
            for seq in lst:
                if seq.state == FINISHED:
                    self._cache.release(seq.seq_id)
                    self._results.append(SequenceResult(seq.seq_id, seq.prompt_len, list(seq.token_ids),
                                                        seq.finish_reason))
                else:
                    keep.append(seq)
            lst[:] = keep

    def _accept(self, seq: Sequence_, token: int) -> None:
        """A sampled token arrives for a sequence (src/scheduler.cpp:208-227,271-282)."""
        if token in self._eos:
            self._finish(seq, "stop")
            return
        seq.token_ids.append(int(token))
        if seq.generated >= seq.max_new_tokens:
            self._finish(seq, "length")

    def step(self) -> bool:
        self._eos = set(self.engine.eos_token_ids)
        mgr = self._cache.manager
        # admission: no page check, as in the reference
        while self._waiting and len(self._prefilling) + len(self._running) < self.max_concurrent:
            seq = self._waiting.popleft()
            seq.state = PREFILLING
            self._cache.admit(seq.seq_id)
            self._prefilling.append(seq)

        entries: list[StepEntry] = []
        owners: list[Sequence_] = []            # sequence of each wanted row
        draws: list[tuple[int, int]] = []
        pending = {g: 0 for g in mgr.groups}

        def take_pages(seq: Sequence_, n: int) -> bool:
            if not mgr.can_reserve(seq.seq_id, n, pending):
                return False
            for g, k in mgr.pages_needed(seq.seq_id, n).items():
                pending[g] += k
            return True

        # prompt portions under the step's token budget, in admission order
        budget = self._budget
        prompt_ends: list[Sequence_] = []
        for seq in self._prefilling:
            if budget <= 0:
                break
            n = min(budget, seq.prompt_len - seq.prefill_cursor)
            if n <= 0:
                continue
            if not take_pages(seq, n):
                self._finish(seq, "capacity")
                continue
            ends = seq.prefill_cursor + n == seq.prompt_len
            want = [n - 1] if ends and seq.max_new_tokens > 0 else []
            entries.append(StepEntry(seq.seq_id, seq.token_ids[seq.prefill_cursor:seq.prefill_cursor + n], want))
            if want:
                owners.append(seq)
                draws.append((seq.seq_id, 0))
            if ends:
                prompt_ends.append(seq)
            seq.prefill_cursor += n
            budget -= n
        # one token for every decoding request
        for seq in self._running:
            if seq.state != RUNNING:
                continue
            if not take_pages(seq, 1):
                self._finish(seq, "capacity")
                continue
            entries.append(StepEntry(seq.seq_id, [seq.token_ids[-1]], [0]))
            owners.append(seq)
            draws.append((seq.seq_id, seq.generated))

        if entries:
            tokens = self.engine.run_step(self._cache, entries, draws, self.temperature, self.seed)
            if len(tokens) != len(owners):
                raise RuntimeError(f"the step returned {len(tokens)} tokens for {len(owners)} wanted rows")
            for seq, tok in zip(owners, tokens):
                self._accept(seq, tok)
            self.steps += 1

        for seq in prompt_ends:
            if seq.state == FINISHED:
                continue
            if seq.max_new_tokens == 0:
                self._finish(seq, "length")         # nothing is sampled (src/scheduler.cpp:203-207)
            else:
                seq.state = RUNNING
                self._prefilling.remove(seq)
                self._running.append(seq)
        self._retire()
        return not self.idle

    def run_until_idle(self) -> None:
        while self.step():
            pass
