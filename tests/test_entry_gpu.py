"""Generation through the entry points on the GPU: `Engine.generate`, the scheduler with
greedy and temperature sampling, the command line and bin/trace_run, compared with the plain
implementation; input validation; the tied head; calls from several threads."""
import json
import os
import subprocess
import sys
import threading

import numpy as np
import pytest
import torch

import replay
from plain_llama import (bf16_round, load_plain_model, plain_forward, plain_generate, plain_sample_bounds)
from tiny_models import A_INIT, B_INIT, TINY_A, TINY_B, make_model_dir, random_tokens

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dir_a(tmp_path_factory):
    return make_model_dir(tmp_path_factory.mktemp("A"), TINY_A, A_INIT, torch.bfloat16)


@pytest.fixture(scope="module")
def dir_b(tmp_path_factory):
    return make_model_dir(tmp_path_factory.mktemp("B"), TINY_B, B_INIT, torch.bfloat16)


def test_greedy_generate_equals_plain(dir_a):
    """Tiny A: prompts of 5, 11 and 17 tokens, 8 greedy tokens each, 32-bit: token for token."""
    from llmengine import Engine
    cfg, w = load_plain_model(dir_a)
    engine = Engine(dir_a, "fp32", block_size=4)
    for i, n in enumerate((5, 11, 17)):
        prompt = random_tokens(n, 256, 40 + i)
        assert engine.generate(prompt, 8) == plain_generate(cfg, w, prompt, 8)
    assert engine.generate([1, 2, 3], 0) == ([1, 2, 3], "length")
    assert engine.dtype == "fp32" and engine.max_pos == 128 and engine.cfg.hidden_size == 64


@pytest.mark.parametrize("chunk", [2, 7, 16])
def test_prompts_longer_than_a_prefill_step(dir_a, chunk):
    """max_prefill_tokens_per_step below the prompt's length: `generate` and `forward_logits` feed
    the prompt in portions of that many tokens (the last one shorter), and nothing changes."""
    from llmengine import Engine
    cfg, w = load_plain_model(dir_a)
    engine = Engine(dir_a, "fp32", block_size=4, max_prefill_tokens_per_step=chunk)
    steps = []
    step = engine.step
    engine.step = lambda cache, entries: (steps.append([len(e.tokens) for e in entries]), step(cache, entries))[1]
    for i, n in enumerate((5, 33, 40)):
        prompt = random_tokens(n, 256, 60 + i)
        steps.clear()
        assert engine.generate(prompt, 6) == plain_generate(cfg, w, prompt, 6)
        # (the five decode steps behind the prompt are launched by the runner itself, from recorded graphs)
        assert steps == [[chunk]] * (n // chunk) + ([[n % chunk]] if n % chunk else [])
    ids = random_tokens(41, 256, 70)
    steps.clear()
    got = engine.forward_logits(ids)
    assert steps == [[chunk]] * (41 // chunk) + ([[41 % chunk]] if 41 % chunk else [])
    ref = plain_forward(cfg, w, ids).numpy()
    assert got.shape == ref.shape and np.abs(got - ref).max() / np.abs(ref).max() < 1e-5


def test_bf16_generate_is_greedy_under_its_own_rounding(dir_b):
    """In bfloat16 a near-tie may fall the other way; every chosen token must still be a
    maximum of the plain logits up to the bfloat16 tolerance."""
    from llmengine import Engine
    cfg, w = load_plain_model(dir_b)
    engine = Engine(dir_b, "bf16", block_size=8)
    prompt = random_tokens(9, 384, 3)
    ids, finish = engine.generate(prompt, 12)
    assert finish == "length" and len(ids) == 21 and ids[:9] == prompt
    ref = plain_forward(cfg, w, ids, rounder=bf16_round)
    for i in range(9, 21):
        row = ref[i - 1]
        assert row[ids[i]] >= row.max() - 2e-2 * row.abs().max(), i


def test_eos_and_limits(tmp_path, dir_a):
    from llmengine import Engine
    cfg, w = load_plain_model(dir_a)
    prompt = [9, 8, 7, 6]
    stream, _ = plain_generate(cfg, w, prompt, 6)
    eos = stream[6]                                              # the third generated token
    d = str(tmp_path / "eos")
    os.makedirs(d)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(dict(TINY_A, eos_token_id=[eos, 255]), f)
    os.symlink(os.path.join(dir_a, "model.safetensors"), os.path.join(d, "model.safetensors"))
    engine = Engine(d, "fp32")
    ids, finish = engine.generate(prompt, 6)
    assert finish == "stop" and ids == stream[:4 + stream[4:].index(eos)]      # EOS is not appended
    with pytest.raises(ValueError):
        engine.generate([], 3)
    with pytest.raises(ValueError):
        engine.generate([1], -1)
    with pytest.raises(ValueError):
        engine.generate([256], 1)
    with pytest.raises(ValueError):
        engine.generate([-1], 1)
    with pytest.raises(RuntimeError, match="max_pos"):
        engine.generate([1] * 100, 29)
    with pytest.raises(RuntimeError, match="max_pos"):
        engine.generate([1], 2 ** 31 - 1)
    assert len(engine.generate([1] * 100, 28)[0]) == 128        # exactly max_pos fits


def test_requests_are_checked_before_weights(tmp_path):
    """A checkpoint that lacks a tensor: bad requests are still refused as bad requests, and a good
    request gets the loader's error with the tensor's name (tests/test_input_validation.py:104-136)."""
    from llmengine import Engine, WeightError
    from llmengine.weights import random_state, write_state_dict
    w = dict(random_state(TINY_A, 0, torch.bfloat16))
    del w["model.layers.1.mlp.down_proj.weight"]
    d = str(tmp_path)
    write_state_dict(os.path.join(d, "model.safetensors"), w)
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(TINY_A, f)
    engine = Engine(d, "fp32")
    assert engine.has_weight("lm_head.weight") and not engine.has_weight("model.layers.1.mlp.down_proj.weight")
    with pytest.raises(ValueError):
        engine.generate([999], 1)
    with pytest.raises(WeightError, match="missing weight: model.layers.1.mlp.down_proj.weight"):
        engine.generate([1], 1)


def test_tied_head_shares_the_embedding_on_the_device(dir_a, dir_b):
    from llmengine import Engine
    a, b = Engine(dir_a, "bf16"), Engine(dir_b, "bf16")
    assert a.model.head.weight.data_ptr() == a.model.embedding.weight.data_ptr()
    assert b.model.head.weight.data_ptr() != b.model.embedding.weight.data_ptr()
    assert a.model.embedding.weight.dtype == torch.bfloat16 and a.model.embedding.weight.is_cuda


def _check_sampled(cfg, w, result, temperature, seed, tol):
    """Teacher-forced check of a sampled stream: every token's cumulative-probability interval
    under the plain logits contains the request's draw (within tol)."""
    from llmengine.sampling import uniform_draw
    ref = plain_forward(cfg, w, result.token_ids)
    for i in range(result.prompt_len, len(result.token_ids)):
        tok = result.token_ids[i]
        u = uniform_draw(seed, result.seq_id, i - result.prompt_len)
        cum = plain_sample_bounds(ref[i - 1], temperature)
        lo = cum[tok - 1].item() if tok > 0 else 0.0
        assert lo - tol <= u <= cum[tok].item() + tol, (result.seq_id, i, tok, u, lo, cum[tok].item())


def test_scheduler_temperature_workload(dir_b):
    """Tiny B's workload: prompts of 1, 9, 33 and 70 tokens, a 16-token prefill budget, 12 tokens
    each at temperature 0.8 with sampler seed 7, pages of 8."""
    from llmengine import BlockManager, ContinuousBatchScheduler, Engine
    cfg, w = load_plain_model(dir_b)
    engine = Engine(dir_b, "fp32")
    blocks = BlockManager(40, 8, 3, 1, 32)
    sched = ContinuousBatchScheduler(engine, blocks, max_concurrent=4, max_prefill_tokens_per_step=16,
                                     temperature=0.8, seed=7)
    prompts = [random_tokens(n, 384, 60 + n) for n in (1, 9, 33, 70)]
    for p in prompts:
        sched.enqueue(p, 12)
    sched.run_until_idle()
    assert blocks.free_blocks == 40
    for r, p in zip(sched.results, prompts):
        assert r.finish_reason == "length" and len(r.token_ids) == len(p) + 12 and r.token_ids[:len(p)] == p
        _check_sampled(cfg, w, r, 0.8, 7, 1e-4)
    # the same requests alone, in another order and batch: the same tokens (draws belong to requests)
    again = ContinuousBatchScheduler(engine, BlockManager(40, 8), max_concurrent=1,
                                     max_prefill_tokens_per_step=200, temperature=0.8, seed=7)
    for p in prompts:
        again.enqueue(p, 12)
    again.run_until_idle()
    assert [r.token_ids for r in again.results] == [r.token_ids for r in sched.results]


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_scheduler_greedy_equals_generate(dir_a, dtype):
    from llmengine import BlockManager, ContinuousBatchScheduler, Engine
    engine = Engine(dir_a, dtype, block_size=4)
    prompts = [[1], [2, 3, 4], list(range(5, 12)), [12, 13]] + [random_tokens(n, 256, n) for n in (20, 31)]
    alone = [engine.generate(p, 12) for p in prompts]
    blocks = BlockManager(64, 4, 2, 2, 16)
    sched = ContinuousBatchScheduler(engine, blocks, max_concurrent=3, max_prefill_tokens_per_step=6)
    for p in prompts:
        sched.enqueue(p, 12)
    sched.run_until_idle()
    if dtype == "fp32":
        assert [(r.token_ids, r.finish_reason) for r in sched.results] == alone
    else:
        # In bfloat16 a near-tie may fall the other way in a batch than alone (other kernels add in
        # another order), after which the streams differ: every token of every stream must be a
        # maximum of the plain logits of its own history, up to the bfloat16 tolerance.
        cfg, w = load_plain_model(dir_a)
        for r, p in zip(sched.results, prompts):
            assert r.token_ids[:len(p)] == p and len(r.token_ids) == len(p) + 12 and r.finish_reason == "length"
            ref = plain_forward(cfg, w, r.token_ids, rounder=bf16_round)
            for i in range(len(p), len(r.token_ids)):
                row = ref[i - 1]
                assert row[r.token_ids[i]] >= row.max() - 2e-2 * row.abs().max(), (r.seq_id, i)
    assert blocks.free_blocks == 64 and [r.seq_id for r in sched.results] == list(range(len(prompts)))


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_sampled_step_with_the_choice_in_the_recording(dir_b, dtype):
    """run_step at a temperature takes decode steps through a recording that ends in the sampling
    kernels, the temperature and the draws sent up with the step's integer arrays: the same tokens
    as the sampler chooses from the logits of an engine without recordings, with requests that come
    and go, two temperatures in turn through the same recording, and a greedy step between."""
    from llmengine import Engine, StepEntry
    from llmengine.sampling import Sampler
    engine, plain = Engine(dir_b, dtype), Engine(dir_b, dtype, use_graphs=False)
    prompts = {"x": random_tokens(19, 384, 1), "y": random_tokens(8, 384, 2), 7: random_tokens(33, 384, 3)}
    caches = [e.new_cache(12, 8, 3) for e in (engine, plain)]
    last = {}
    for rid, p in prompts.items():
        for c, e in zip(caches, (engine, plain)):
            c.admit(rid)
            lg = e.step(c, [StepEntry(rid, p, [len(p) - 1])])
        last[rid] = int(lg.argmax())
    number = {"x": 0, "y": 1, 7: 2}
    recordings = set()
    for turn in range(14):
        ids = list(last) if turn % 4 else list(last)[::-1]
        entries = [StepEntry(r, [last[r]], [0]) for r in ids]
        temperature = (0.7, 1.6, 0.0)[turn % 3]
        draws = [(number[r], turn) for r in ids]
        got = engine.run_step(caches[0], entries, draws, temperature, seed=11)
        want = Sampler(temperature, 11).choose(plain.step(caches[1], entries), draws)
        assert got == want, (turn, temperature)
        last = dict(zip(ids, got))
        recordings |= {k[:3] for k in caches[0].graphs}
        if turn == 6:
            for c in caches:
                c.release("y")
            del last["y"]
    assert engine.runner.graph_replays >= 14 and plain.runner.graph_replays == 0
    # one recording for each number of requests and kind of choice, whatever the temperature
    assert sorted(k[2] for k in recordings) == ["greedy", "greedy", "sampled", "sampled"]


def test_scheduler_at_a_temperature_with_many_live_requests(dir_a):
    """28 requests, up to 24 live, at temperature 1.1: the decode steps' recordings (of every number of
    live requests that occurs, each ending in the sampling kernels) choose the tokens that an engine
    without recordings samples from its logits, request by request, and every token lies in its
    draw's interval under the plain logits."""
    from llmengine import BlockManager, ContinuousBatchScheduler, Engine
    cfg, w = load_plain_model(dir_a)
    prompts = [random_tokens(3 + (7 * i) % 40, 256, 500 + i) for i in range(28)]
    news = [6 + (5 * i) % 17 for i in range(28)]
    streams = []
    for graphs in (True, False):
        engine = Engine(dir_a, "fp32", use_graphs=graphs)
        blocks = BlockManager(400, 8, 2, 2, 16)
        sched = ContinuousBatchScheduler(engine, blocks, max_concurrent=24, max_prefill_tokens_per_step=48,
                                         temperature=1.1, seed=13)
        for p, n in zip(prompts, news):
            sched.enqueue(p, n)
        sched.run_until_idle()
        assert blocks.free_blocks == 400
        streams.append([(r.seq_id, r.token_ids, r.finish_reason) for r in sched.results])
        if graphs:
            kinds = {k[2] for k in sched._cache.graphs}
            sizes = {k[0] for k in sched._cache.graphs}
            assert kinds == {"sampled"} and max(sizes) > 16 and len(sizes) > 3
            for r in sched.results:
                _check_sampled(cfg, w, r, 1.1, 13, 1e-4)
    assert streams[0] == streams[1]


def test_generate_at_a_temperature_is_the_same_with_and_without_recordings(dir_a, dir_b):
    """generate() launches each sampled step before it has fetched the token of the step before;
    the stream is the one an engine without recordings samples, and the one the plain logits allow."""
    from types import SimpleNamespace
    from llmengine import Engine
    for folder, vocab in ((dir_a, 256), (dir_b, 384)):
        cfg, w = load_plain_model(folder)
        for seed in (3, 4):
            kw = dict(temperature=0.9, sampler_seed=seed)
            prompt = random_tokens(11 + seed, vocab, seed)
            with_rec, finish = Engine(folder, "fp32", **kw).generate(prompt, 20)
            without, _ = Engine(folder, "fp32", use_graphs=False, **kw).generate(prompt, 20)
            assert with_rec == without and len(with_rec) > len(prompt)
            _check_sampled(cfg, w, SimpleNamespace(token_ids=with_rec, prompt_len=len(prompt), seq_id=0), 0.9, seed, 1e-4)


def test_greedy_step_with_the_argmax_in_the_recording(dir_b):
    """run_step at temperature 0 takes decode steps through a recording that ends in the argmax:
    same tokens as the logits' own argmax, a clear error when the pages run out, and requests
    that come and go between the steps."""
    from llmengine import CapacityError, Engine, StepEntry
    engine = Engine(dir_b, "bf16")
    a = Engine(dir_b, "bf16")
    prompts = {"x": random_tokens(19, 384, 1), "y": random_tokens(8, 384, 2), 7: random_tokens(33, 384, 3)}
    caches = [e.new_cache(12, 8, 3) for e in (engine, a)]
    last = {}
    for rid, p in prompts.items():
        for c, e in zip(caches, (engine, a)):
            c.admit(rid)
            lg = e.step(c, [StepEntry(rid, p, [len(p) - 1])])
        last[rid] = int(lg.argmax())
    for turn in range(12):
        ids = list(last) if turn % 4 else list(last)[::-1]
        entries = [StepEntry(r, [last[r]], [0]) for r in ids]
        got = engine.run_step(caches[0], entries, None)
        want = a.step(caches[1], entries).argmax(dim=1).tolist()
        assert got == want
        last = dict(zip(ids, got))
        if turn == 5:                                        # one leaves, the others go on
            for c in caches:
                c.release("y")
            del last["y"]
        if turn == 7:
            # a large argmax elsewhere replaces the scratch that plain calls share, and new tensors
            # take the freed memory: the recordings keep a scratch of their own and must not notice
            from llmengine import ops
            big = torch.randn(72, 128256, device="cuda:0")
            ops.argmax(big, torch.empty(72, dtype=torch.int32, device="cuda:0"))
            torch.cuda.synchronize()
            filler = [torch.full((4096,), float("nan"), device="cuda:0") for _ in range(64)]
    assert engine.runner.graph_replays >= 10
    with pytest.raises(CapacityError):                       # 12 pages of 8: the three requests outgrow them
        for _ in range(40):
            got = engine.run_step(caches[0], [StepEntry(r, [last[r]], [0]) for r in last], None)
            last = dict(zip(last, got))
    before = {r: caches[0].manager.length(r) for r in last}
    with pytest.raises(CapacityError):
        engine.run_step(caches[0], [StepEntry(r, [last[r]], [0]) for r in last], None)
    assert before == {r: caches[0].manager.length(r) for r in last}      # a refused step changes nothing
    # .. and so does one that would pass the position limit (256 here): nothing is reserved for anyone
    roomy = engine.new_cache(40, 8, 2)
    for rid, n in (("p", 255), ("q", 40)):
        roomy.admit(rid)
        engine.step(roomy, [StepEntry(rid, random_tokens(n, 384, n), [])])
    free = roomy.manager.free_pages("full")
    engine.run_step(roomy, [StepEntry("p", [1], [0]), StepEntry("q", [2], [0])], None)       # p is 256 long now
    assert roomy.manager.free_pages("full") == free - 1                  # (q began a page)
    with pytest.raises(ValueError, match="position limit"):
        engine.run_step(roomy, [StepEntry("p", [1], [0]), StepEntry("q", [2], [0])], None)
    assert roomy.manager.free_pages("full") == free - 1 and roomy.manager.length("q") == 41
    roomy.manager.check()


def test_scheduler_capacity_on_the_gpu(dir_a):
    from llmengine import BlockManager, ContinuousBatchScheduler, Engine
    engine = Engine(dir_a, "fp32")
    blocks = BlockManager(4, 4)
    sched = ContinuousBatchScheduler(engine, blocks, max_concurrent=2, max_prefill_tokens_per_step=4)
    prompts = [[1, 2, 3, 4], [5, 6, 7, 8]]
    for p in prompts:
        sched.enqueue(p, 12)
    sched.run_until_idle()
    assert "capacity" in [r.finish_reason for r in sched.results]
    for r, p in zip(sched.results, prompts):
        full, _ = engine.generate(p, 12)
        assert r.token_ids == full[:len(r.token_ids)]
    assert blocks.free_blocks == 4


def test_threads_get_the_serial_answers(dir_a):
    from llmengine import Engine
    engine = Engine(dir_a, "fp32")
    prompts = [random_tokens(6 + i, 256, 900 + i) for i in range(6)]
    serial = [engine.generate(p, 6) for p in prompts]
    got = [None] * len(prompts)

    def work(i):
        got[i] = engine.generate(prompts[i], 6)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(prompts))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert got == serial


def test_schedulers_beside_generate_on_one_engine(dir_b):
    """Two schedulers (each with a block manager of its own) step while two other threads call
    generate on the same engine, as in the reference's tests/test_engine_thread_safety.py:65-125:
    the runner's scratch memory, its recorded decode steps and the stream are shared, and every
    stream of tokens must be the serial one (32-bit: no near ties between the batched and the
    single steps)."""
    from llmengine import BlockManager, ContinuousBatchScheduler, Engine
    engine = Engine(dir_b, "fp32", block_size=8)
    assert engine.runner.use_graphs
    prompts = [random_tokens(5 + 4 * i, 384, 950 + i) for i in range(4)]
    serial = [engine.generate(p, 9) for p in prompts]
    errors, from_sched, from_gen = [], [None, None], [None, None]

    def run_sched(k):
        try:
            sched = ContinuousBatchScheduler(engine, BlockManager(24, 8), max_concurrent=3, max_prefill_tokens_per_step=6)
            for p in prompts:
                sched.enqueue(p, 9)
            sched.run_until_idle()
            from_sched[k] = [(r.token_ids, r.finish_reason) for r in sched.results]
        except Exception as e:          # noqa: BLE001
            errors.append(e)

    def run_gen(k):
        try:
            from_gen[k] = [engine.generate(p, 9) for _ in range(2) for p in prompts]
        except Exception as e:          # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=run_sched, args=(k,)) for k in range(2)]
    threads += [threading.Thread(target=run_gen, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert from_sched[0] == serial and from_sched[1] == serial
    assert from_gen[0] == serial + serial and from_gen[1] == serial + serial


def test_a_head_size_beyond_the_kernels_is_refused_when_the_model_is_built():
    from llmengine import Engine
    cfg = dict(TINY_A, head_dim=512, hidden_size=64)
    engine = Engine(None, "fp32", _config=cfg, _tensors={})
    with pytest.raises(ValueError, match=r"self_attn: head_dim=512.*up to 256"):
        engine.runner


def test_command_line(dir_a, tmp_path):
    from llmengine import Engine
    prompt = [5, 17, 3, 99]
    want = Engine(dir_a, "fp32").generate(prompt, 5)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmengine-cli"), "--model", dir_a,
                          "--dtype", "fp32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "5"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert (rec["token_ids"], rec["finish_reason"]) == want
    pf = tmp_path / "prompts.txt"
    pf.write_text("1 2 3\n7,8,9,10,11\n")
    cfgf = tmp_path / "cfg.json"
    cfgf.write_text(json.dumps(TINY_A))
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "llmengine-cli"), "--random", str(cfgf),
                          "--seed", "3", "--prompt-file", str(pf), "--max-new-tokens", "4", "--temperature", "0.7",
                          "--block-size", "4"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    recs = [json.loads(line) for line in out.stdout.strip().splitlines()]
    assert [len(r["token_ids"]) for r in recs] == [7, 9] and all(r["finish_reason"] == "length" for r in recs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dir_b, tmp_path, dtype):
    """bin/trace_run as a user calls it: a mixed trace over so few pages that they are used again."""
    reqs = {f"q{i}": random_tokens(n, 384, 300 + i) for i, n in enumerate((70, 40, 3, 55, 64, 18))}
    steps = replay.mixed(reqs, max_live=4, seed=2)
    peak = replay.trace_peak_tokens(steps, 64)
    out_dir = tmp_path / "out"
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", dir_b, "--dtype", dtype, "--out",
                        str(out_dir), "--max-tokens", str(peak)], input=text, capture_output=True, text=True,
                       timeout=600)
    assert p.returncode == 0, p.stderr[-3000:]
    assert p.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    cfg, w = load_plain_model(dir_b)
    plain = {rid: plain_forward(cfg, w, ids, rounder=bf16_round if dtype == "bfloat16" else None).numpy()
             for rid, ids in reqs.items()}
    tol = 1e-5 if dtype == "float32" else 2e-2
    pos = {rid: 0 for rid in reqs}
    for s in steps:
        want_rows = sum(len(e["want"]) for e in s["entries"])
        rows = np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(want_rows, 384)
        r = 0
        for e in s["entries"]:
            for wnt in e["want"]:
                ref = plain[e["id"]][pos[e["id"]] + wnt]
                assert np.abs(rows[r] - ref).max() / np.abs(ref).max() < tol, (s["step"], e["id"], wnt)
                r += 1
            pos[e["id"]] += len(e["tokens"])


def test_trace_run_random_config_index_and_repeatability(tmp_path):
    """bin/trace_run over a model made from a configuration and a seed, with pages that do not
    divide 64 and the index of (request, position) per row; run twice in bfloat16, the files are
    the same bits (the model is wide enough that serving would cut its sums over k)."""
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 1024,
           "intermediate_size": 2048, "num_hidden_layers": 2, "num_attention_heads": 16, "num_key_value_heads": 4,
           "head_dim": 64, "vocab_size": 320, "max_position_embeddings": 512, "rms_norm_eps": 1e-5,
           "rope_theta": 10000.0, "tie_word_embeddings": True}
    cfgf = tmp_path / "config.json"
    cfgf.write_text(json.dumps(cfg))
    reqs = {f"q{i}": random_tokens(n, 320, 700 + i) for i, n in enumerate((70, 40, 3, 55, 64))}
    steps = replay.mixed(reqs, max_live=4, seed=4)
    peak = replay.trace_peak_tokens(steps, 64)
    text = "\n".join(json.dumps(s) for s in steps) + "\n"
    outs = []
    for run in range(2):
        out_dir = tmp_path / f"out{run}"
        p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--random-config", str(cfgf), "--seed", "9",
                            "--dtype", "bfloat16", "--out", str(out_dir), "--max-tokens", str(peak), "--block-size",
                            "48", "--index"], input=text, capture_output=True, text=True, timeout=600)
        assert p.returncode == 0, p.stderr[-3000:]
        outs.append(out_dir)
    # the index names every row
    index = [json.loads(line) for line in (outs[0] / "index.jsonl").read_text().splitlines()]
    pos = {rid: 0 for rid in reqs}
    expected = []
    for s in steps:
        rows = [[e["id"], pos[e["id"]] + w] for e in s["entries"] for w in e["want"]]
        for e in s["entries"]:
            pos[e["id"]] += len(e["tokens"])
        if rows:
            expected.append({"step": s["step"], "rows": rows})
    assert index == expected
    for s in steps:
        a = np.fromfile(outs[0] / f"{s['step']}.f32", dtype="<f4")
        b = np.fromfile(outs[1] / f"{s['step']}.f32", dtype="<f4")
        assert a.size == 320 * sum(len(e["want"]) for e in s["entries"]) and np.array_equal(a, b), s["step"]
    # and the logits are the model's: the same weights through the plain implementation
    from llmengine.weights import random_state
    wide = {k: v.double() for k, v in random_state(cfg, 9, torch.bfloat16)}
    rid, ids = "q1", reqs["q1"]
    ref = plain_forward(cfg, wide, ids, rounder=bf16_round).numpy()
    pos = 0
    for s in steps:
        r = 0
        for e in s["entries"]:
            if e["id"] == rid:
                rows = np.fromfile(outs[0] / f"{s['step']}.f32", dtype="<f4").reshape(-1, 320)
                for w in e["want"]:
                    got = rows[r + e["want"].index(w)]
                    assert np.abs(got - ref[pos + w]).max() / np.abs(ref[pos + w]).max() < 2e-2
                pos += len(e["tokens"])
            r += len(e["want"])
