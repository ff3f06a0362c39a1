"""The scheduler's decisions (no GPU), against a stand-in engine whose next token is a
function of the whole history that was fed to it: any token fed twice, skipped, or out of
order changes the stream. Cases follow the reference's tests/test_scheduler.py."""
import pytest

from llmengine.cache import CacheManager, GroupSpec
from llmengine.engine.scheduler import ContinuousBatchScheduler

V = 97


def next_token(history):
    return (sum((i + 1) * t for i, t in enumerate(history)) * 31 + len(history)) % V


def single_generate(prompt, max_new, eos=()):
    ids, finish = list(prompt), "length"
    for _ in range(max_new):
        t = next_token(ids)
        if t in eos:
            finish = "stop"
            break
        ids.append(t)
    return ids, finish


class FakeCache:
    def __init__(self, pages, page_size, max_requests):
        self.manager = CacheManager([GroupSpec("full", "full", 0, pages)], page_size, max_requests)

    def admit(self, rid):
        return self.manager.admit(rid)

    def release(self, rid):
        self.manager.release(rid)


class FakeBlocks:
    def __init__(self, num_blocks, block_size):
        self.num_blocks, self.block_size = num_blocks, block_size
        self.cache = None

    @property
    def free_blocks(self):
        return self.cache.manager.free_pages() if self.cache else self.num_blocks


class FakeEngine:
    def __init__(self, eos=(), max_pos=512):
        self.vocab_size, self.max_pos, self.eos_token_ids = V, max_pos, tuple(eos)
        self.history = {}
        self.batches = []           # per step: list of (request, n tokens)

    def open_cache(self, blocks, max_requests):
        blocks.cache = FakeCache(blocks.num_blocks, blocks.block_size, max_requests)
        return blocks.cache

    def run_step(self, cache, entries, draws, temperature, seed):
        out = []
        self.batches.append([(e.request_id, len(e.tokens)) for e in entries])
        for e in entries:
            assert cache.manager.reserve(e.request_id, len(e.tokens)), "the scheduler promised pages"
            h = self.history.setdefault(e.request_id, [])
            assert cache.manager.length(e.request_id) == len(h)
            for i, t in enumerate(e.tokens):
                h.append(t)
                if i in e.want:
                    out.append(next_token(h))
            cache.manager.commit(e.request_id, len(e.tokens))
        assert len(draws) == len(out)
        return out


def run(prompts, max_new, blocks=(64, 4), **kw):
    eng = FakeEngine(eos=kw.pop("eos", ()))
    bm = FakeBlocks(*blocks)
    s = ContinuousBatchScheduler(eng, bm, **kw)
    for p, n in zip(prompts, max_new if isinstance(max_new, list) else [max_new] * len(prompts)):
        s.enqueue(p, n)
    s.run_until_idle()
    return s, eng, bm


def test_streams_equal_single_sequence():
    prompts = [[1], [2, 3, 4], [5, 6, 7, 8, 9, 10, 11], [12, 13]]       # tests/test_scheduler.py:97-124
    s, eng, bm = run(prompts, 12)
    for r, p in zip(s.results, prompts):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 12)
        assert r.prompt_len == len(p)
    assert bm.free_blocks == bm.num_blocks and s.idle
    assert [r.seq_id for r in s.results] == [0, 1, 2, 3]


def test_one_mixed_batch_per_step():
    s, eng, _ = run([[1, 2, 3], list(range(20, 50))], 6, max_prefill_tokens_per_step=8)
    mixed = [b for b in eng.batches if any(n > 1 for _, n in b) and any(n == 1 and rid == 0 for rid, n in b)]
    assert mixed, "a prompt portion and a decoded token never shared a step"
    for b in eng.batches:
        assert sum(n for rid, n in b if not (n == 1 and len(eng.history[rid]) > 3 and rid == 0)) <= 8 + 1
    for r, p in zip(s.results, [[1, 2, 3], list(range(20, 50))]):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 6)


def test_budget_is_shared_in_admission_order_and_excludes_decoding():
    prompts = [list(range(1, 6)), list(range(1, 4)), list(range(1, 10))]
    s, eng, _ = run(prompts, 3, max_prefill_tokens_per_step=7)
    assert eng.batches[0] == [(0, 5), (1, 2)]                    # first takes what it needs, next the rest
    assert eng.batches[1][:2] == [(1, 1), (2, 6)]                # then decoding tokens ride along, uncounted
    assert (0, 1) in eng.batches[1]
    for b in eng.batches:
        decoding = sum(1 for rid, n in b if n == 1 and len(eng.history[rid]) > len(prompts[rid]))
        assert sum(n for _, n in b) - decoding <= 7


def test_decoding_requests_stand_longest_first_and_pages_go_in_admission_order():
    """A step's decoded tokens come in the order of the requests' lengths (the decode kernels deal the
    requests out in turn); the streams are the same, and when pages run out it is still the request that
    came later which ends."""
    prompts = [[1, 2], list(range(1, 12)), [3, 4, 5, 6], list(range(2, 9))]
    s, eng, _ = run(prompts, 5)
    seen = 0
    for b in eng.batches:
        decoding = [rid for rid, n in b if n == 1 and len(eng.history[rid]) > len(prompts[rid])]
        if len(decoding) == 4:
            assert decoding == [1, 3, 2, 0]
            seen += 1
    assert seen >= 3
    for r, p in zip(s.results, prompts):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 5)
    # 8 pages of 4, two requests that need their next page in the same steps (3 + t and 7 + t tokens): when one
    # page is left, the request that came first takes it, though the other is longer and stands in front
    s, eng, bm = run([[1, 2, 3], list(range(1, 8))], 12, blocks=(8, 4))
    assert [r.finish_reason for r in s.results] == ["length", "capacity"]
    assert s.results[0].token_ids == single_generate([1, 2, 3], 12)[0]
    assert bm.free_blocks == bm.num_blocks


def test_rounds_order_pairs_long_with_short():
    from llmengine.engine.scheduler import rounds_order
    assert rounds_order(3, 4) == [0, 1, 2] and rounds_order(4, 4) == [0, 1, 2, 3] and rounds_order(5, 0) == list(range(5))
    assert rounds_order(7, 4) == [3, 2, 1, 0, 4, 5, 6]
    assert rounds_order(10, 4) == [0, 1, 2, 3, 7, 6, 5, 4, 8, 9]
    for n, per in [(44, 32), (64, 32), (72, 32), (9, 2), (100, 7)]:
        order = rounds_order(n, per)
        assert sorted(order) == list(range(n))
        sizes = [1000 - 7 * r for r in range(n)]                      # rank 0 the largest
        places = [sum(sizes[order[p]] for p in range(j, n, per)) for j in range(per)]
        plain = [sum(sizes[p] for p in range(j, n, per)) for j in range(per)]
        assert max(places) <= max(plain) and max(places) - min(places) <= max(plain) - min(plain)


def test_the_engine_names_the_round_and_the_scheduler_orders_by_it():
    """An engine that says after how many requests its decode kernel has been round the compute units once gets
    its decoding requests in rounds_order of their lengths; the streams do not change."""
    from llmengine.engine.scheduler import rounds_order
    prompts = [list(range(1, 2 + 2 * i)) for i in range(7)]           # lengths 1, 3, .. 13: request 6 the longest
    eng = FakeEngine()
    eng.decode_round = 3
    s = ContinuousBatchScheduler(eng, FakeBlocks(64, 4))
    for p in prompts:
        s.enqueue(p, 6)
    s.run_until_idle()
    by_length = [6, 5, 4, 3, 2, 1, 0]
    seen = 0
    for b in eng.batches:
        decoding = [rid for rid, n in b if n == 1 and len(eng.history[rid]) > len(prompts[rid])]
        if len(decoding) == 7:
            assert decoding == [by_length[r] for r in rounds_order(7, 3)]
            seen += 1
    assert seen >= 3
    for r, p in zip(s.results, prompts):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 6)


def test_a_few_rows_past_a_round_are_left_for_the_next_step():
    """An engine whose products run a few rows past a multiple of some number apart (step_rows_round): the
    portion that uses the budget up gives those few tokens back; streams, and everything else, stay."""
    prompts = [[1, 2, 3], [4, 5], list(range(1, 60))]
    eng = FakeEngine()
    eng.step_rows_round = (16, 4)
    s = ContinuousBatchScheduler(eng, FakeBlocks(64, 4), max_prefill_tokens_per_step=16)
    for p in prompts:
        s.enqueue(p, 8)
    s.run_until_idle()
    # step 0: 3 + 2 + 11 prompt tokens, nobody decodes yet: 16 rows. step 1: 16 prompt tokens + 2 decoding = 18 rows,
    # two more than a round: the portion is 14. then 16 rows every step while the long prompt lasts
    assert eng.batches[0] == [(0, 3), (1, 2), (2, 11)]
    assert eng.batches[1][0] == (2, 14) and sorted(eng.batches[1][1:]) == [(0, 1), (1, 1)]
    assert eng.batches[2][0] == (2, 14) and eng.batches[3][0] == (2, 14)
    assert eng.batches[4][0] == (2, 6)                      # the prompt's end is never cut short
    for r, p in zip(s.results, prompts):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 8)
    # what a portion gives back does not go to the prompt behind it
    eng = FakeEngine()
    eng.step_rows_round = (16, 4)
    s = ContinuousBatchScheduler(eng, FakeBlocks(128, 4), max_prefill_tokens_per_step=16)
    two = [[1, 2, 3], list(range(1, 50)), list(range(2, 40))]
    for p in two:
        s.enqueue(p, 4)
    s.run_until_idle()
    assert eng.batches[0] == [(0, 3), (1, 13)] and eng.batches[1][:1] == [(1, 15)] and (2, 1) not in eng.batches[1]
    assert sum(n for _, n in eng.batches[1]) == 16
    for r, p in zip(s.results, two):
        assert (r.token_ids, r.finish_reason) == single_generate(p, 4)
    # without the hint, and where the rows past the round are more than the engine runs apart: the whole budget
    eng = FakeEngine()
    s = ContinuousBatchScheduler(eng, FakeBlocks(64, 4), max_prefill_tokens_per_step=16)
    for p in prompts:
        s.enqueue(p, 8)
    s.run_until_idle()
    assert eng.batches[1][0] == (2, 16)
    eng = FakeEngine()
    eng.step_rows_round = (16, 1)
    s = ContinuousBatchScheduler(eng, FakeBlocks(64, 4), max_prefill_tokens_per_step=16)
    for p in prompts:
        s.enqueue(p, 8)
    s.run_until_idle()
    assert eng.batches[1][0] == (2, 16)


@pytest.mark.parametrize("max_new", [0, 1, 2, 5])               # tests/test_scheduler.py:220-280
def test_exact_counts(max_new):
    s, _, bm = run([[4, 5, 6]], max_new)
    r = s.results[0]
    assert len(r.token_ids) == 3 + max_new and r.finish_reason == "length"
    assert bm.free_blocks == bm.num_blocks


def test_small_budget_long_prompt():
    s, eng, _ = run([list(range(1, 21))], 4, max_prefill_tokens_per_step=2)   # tests/test_scheduler.py:312-331
    r = s.results[0]
    assert len(r.token_ids) == 24 and r.finish_reason == "length"
    assert [n for b in eng.batches[:10] for _, n in b] == [2] * 10


def test_eos_stops_and_is_not_appended():
    prompt = [3, 1, 4]
    stream, _ = single_generate(prompt, 8)
    eos = stream[5]                                               # the third generated token
    s, _, _ = run([prompt], 8, eos=(eos,))
    r = s.results[0]
    first = stream[3:].index(eos)
    assert r.finish_reason == "stop" and r.token_ids == stream[:3 + first]


def test_capacity_termination():
    # 4 pages of 4 tokens, two requests of 4 + 12 tokens: tests/test_scheduler.py:285-307
    s, eng, bm = run([[1, 2, 3, 4], [5, 6, 7, 8]], 12, blocks=(4, 4), max_concurrent=2,
                     max_prefill_tokens_per_step=4)
    reasons = [r.finish_reason for r in s.results]
    assert "capacity" in reasons
    for r, p in zip(s.results, [[1, 2, 3, 4], [5, 6, 7, 8]]):
        full, _ = single_generate(p, 12)
        assert r.token_ids == full[:len(r.token_ids)]            # what was generated is kept and right
        assert len(r.token_ids) >= 4
    assert bm.free_blocks == 4
    # a prompt that can never fit ends with capacity and the queue goes on
    s2, _, bm2 = run([list(range(1, 30)), [1, 2]], 2, blocks=(2, 4))
    assert [r.finish_reason for r in s2.results] == ["capacity", "length"]
    assert s2.results[0].token_ids == list(range(1, 30)) and bm2.free_blocks == 2


def test_freed_pages_serve_waiting_requests():
    prompts = [[i + 1] * 6 for i in range(6)]
    s, _, bm = run(prompts, 5, blocks=(6, 4), max_concurrent=2)
    assert [r.finish_reason for r in s.results] == ["length"] * 6
    for r, p in zip(s.results, prompts):
        assert r.token_ids == single_generate(p, 5)[0]
    assert bm.free_blocks == 6


def test_invalid_knobs_and_requests():
    eng, bm = FakeEngine(max_pos=16), FakeBlocks(8, 4)
    for kw in ({"max_concurrent": 0}, {"max_prefill_tokens_per_step": 0}, {"temperature": -1.0}):
        with pytest.raises(ValueError):
            ContinuousBatchScheduler(eng, bm, **kw)
    s = ContinuousBatchScheduler(eng, bm)
    with pytest.raises(ValueError):
        s.budget = 0
    s.budget = 3
    assert s.budget == 3
    for prompt, n in (([], 1), ([1], -1), ([V], 1), ([-1], 1), ([1] * 10, 7)):
        with pytest.raises(ValueError):
            s.enqueue(prompt, n)
    assert s.idle and not s.step()
    s.enqueue([1] * 10, 6)                                        # exactly max_pos is allowed
    s.run_until_idle()
    assert len(s.results[0].token_ids) == 16
    s.clear_results()
    assert s.results == []


def test_a_failing_step_changes_nothing():
    """The model run raises once, in a step that carries prompt portions and decoded tokens: the
    scheduler forgets the batch, the prompts stay where they were, and the streams that come out
    afterwards are those of an undisturbed run (a prompt that had moved on would skip tokens)."""
    prompts = [[1, 2, 3], list(range(20, 50)), list(range(5, 25)), [9]]

    class Failing(FakeEngine):
        def __init__(self, fail_at):
            super().__init__()
            self.fail_at, self.calls = fail_at, 0

        def run_step(self, cache, entries, draws, temperature, seed):
            self.calls += 1
            if self.calls == self.fail_at:
                raise RuntimeError("the step failed")
            return super().run_step(cache, entries, draws, temperature, seed)

    for fail_at in (1, 2, 3, 5):
        eng, bm = Failing(fail_at), FakeBlocks(64, 4)
        s = ContinuousBatchScheduler(eng, bm, max_concurrent=3, max_prefill_tokens_per_step=8)
        for p in prompts:
            s.enqueue(p, 7)
        failures = 0
        while True:
            try:
                if not s.step():
                    break
            except RuntimeError as e:
                assert "the step failed" in str(e)
                failures += 1
        assert failures == 1
        for r, p in zip(s.results, prompts):
            assert (r.token_ids, r.finish_reason) == single_generate(p, 7), (fail_at, r.seq_id)
        assert bm.free_blocks == bm.num_blocks and s.idle
        bm.cache.manager.check()


def test_one_scheduler_per_block_manager():
    eng, bm = FakeEngine(), FakeBlocks(64, 4)
    first = ContinuousBatchScheduler(eng, bm, max_concurrent=2)
    first.enqueue([1, 2, 3], 4)
    first.step()
    with pytest.raises(ValueError, match="BlockManager of its own"):
        ContinuousBatchScheduler(eng, bm, max_concurrent=4)
    first.run_until_idle()
    eng.history.clear()                                               # (the stand-in keys its histories by sequence id)
    second = ContinuousBatchScheduler(eng, bm, max_concurrent=4)      # the first is idle: the manager is free again
    second.enqueue([4, 5], 3)
    second.run_until_idle()
    assert second.results[0].token_ids[:2] == [4, 5]


def test_a_step_that_fails_after_it_ran_ends_its_sequences():
    """The batch runs and the cache holds its tokens, but the choice of the next tokens fails: the
    sequences of that batch cannot go on (offering the same tokens again would cache them twice).
    Each ends with "error" and the tokens it had, its pages go back, and requests that were not in
    the batch are served as if nothing had happened."""
    from llmengine import StepCommittedError
    prompts = [[1, 2, 3], list(range(20, 50)), list(range(5, 25)), [9], [4, 4, 4, 4]]

    class FailsBehind(FakeEngine):
        def __init__(self, fail_at):
            super().__init__()
            self.fail_at, self.calls, self.lost = fail_at, 0, []

        def run_step(self, cache, entries, draws, temperature, seed):
            out = super().run_step(cache, entries, draws, temperature, seed)
            self.calls += 1
            if self.calls == self.fail_at:
                self.lost = [e.request_id for e in entries]
                raise StepCommittedError("the tokens were not chosen")
            return out

    for fail_at in (1, 2, 4, 6):
        eng, bm = FailsBehind(fail_at), FakeBlocks(64, 4)
        s = ContinuousBatchScheduler(eng, bm, max_concurrent=3, max_prefill_tokens_per_step=8)
        for p in prompts:
            s.enqueue(p, 7)
        failures = 0
        while True:
            try:
                if not s.step():
                    break
            except StepCommittedError:
                failures += 1
        assert failures == 1 and eng.lost
        for r, p in zip(s.results, prompts):
            whole = single_generate(p, 7)
            if r.seq_id in eng.lost:
                assert r.finish_reason == "error"
                assert r.token_ids == whole[0][:len(r.token_ids)] and len(r.token_ids) >= len(p)
            else:
                assert (r.token_ids, r.finish_reason) == whole, (fail_at, r.seq_id)
        assert bm.free_blocks == bm.num_blocks and s.idle
        bm.cache.manager.check()
