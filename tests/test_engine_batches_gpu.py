"""The engine at the batch sizes that serving and the benchmark run: 24 and 70 live requests,
prompts in portions beside decoded tokens, then dozens of decode steps of the whole batch,
requests ending and new ones taking their pages and slots; every logit row against the plain
implementation, in 32-bit and in bfloat16, once with decode steps replayed from recorded graphs
and once launched plainly. The reference's counterpart is its batched-decode test
(tests/test_scheduler.py:97-124: a ragged batch decodes as each sequence does alone).

Also here: bit-for-bit repeatability of the deterministic mode, and 32-bit logits that do not
depend on the page size or on which physical pages a request got
(tests/test_paged_kv.py:20-43: paged equals contiguous exactly)."""
import numpy as np
import pytest
import torch

import replay
from plain_llama import bf16_round, plain_forward
from tiny_models import A_INIT, B_INIT, TINY_A, TINY_B, random_tokens

pytestmark = pytest.mark.gpu

TOL = {"fp32": 1e-5, "bf16": 2e-2}

# one layer of the 1B width (the fused decode kernels at width 2,048, the tile products at
# 17 to 64 and more rows), with a small vocabulary so that the plain implementation stays quick
WIDE_1B = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 2048,
           "intermediate_size": 8192, "num_hidden_layers": 1, "num_attention_heads": 32,
           "num_key_value_heads": 8, "head_dim": 64, "vocab_size": 1000, "max_position_embeddings": 4096,
           "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "tie_word_embeddings": True,
           "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                            "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}}
WIDE_INIT = dict(seed=11, std=0.02, norm_mean=1.0, norm_std=0.05)

# one layer of the 3B and of the 8B sizes: products over k of 3,072 / 8,192 and 4,096 / 14,336 at 17 to 64
# and more rows, heads of 128 with three and four query heads to a key/value head
WIDE_3B = dict(WIDE_1B, hidden_size=3072, intermediate_size=8192, num_attention_heads=24, head_dim=128)
WIDE_8B = dict(WIDE_1B, hidden_size=4096, intermediate_size=14336, num_attention_heads=32, head_dim=128,
               tie_word_embeddings=False,
               rope_scaling=dict(WIDE_1B["rope_scaling"], factor=8.0))

MODELS = {"A": (TINY_A, A_INIT, 16), "B": (TINY_B, B_INIT, 16), "1b": (WIDE_1B, WIDE_INIT, 16),
          "3b": (WIDE_3B, dict(WIDE_INIT, seed=12), 16), "8b": (WIDE_8B, dict(WIDE_INIT, seed=13), 16)}


def batch_schedule(requests: dict, max_live: int, portion: int = 24, seed: int = 0) -> list[dict]:
    """Up to max_live requests at a time. A request's prompt (its first third) runs in portions of
    up to `portion` tokens beside the single tokens of the requests that are decoding; the rest is
    decoded one token a step with every live request taking part, so that most steps are decode
    steps of the whole batch. Finished requests make room for waiting ones at once."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: list[dict] = []
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, ids = waiting.pop(0)
            live.append({"id": rid, "ids": list(ids), "pos": 0, "prompt": max(2, len(ids) // 3)})
        entries, ended = [], []
        for r in live:
            if r["pos"] < r["prompt"]:
                n = min(int(rng.integers(2, portion + 1)), r["prompt"] - r["pos"])
            else:
                n = 1
            entries.append({"id": r["id"], "tokens": r["ids"][r["pos"]:r["pos"] + n], "want": list(range(n))})
            r["pos"] += n
            if r["pos"] == len(r["ids"]):
                ended.append(r["id"])
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [r for r in live if r["id"] not in ended]
    return steps


@pytest.fixture(scope="module")
def zoo():
    from llmengine.weights import random_state
    out = {}
    for name, (cfg, init, page) in MODELS.items():
        tensors = dict(random_state(cfg, init["seed"], torch.bfloat16, init["std"], init["norm_mean"], init["norm_std"]))
        out[name] = (cfg, tensors, page)
    return out


_PLAIN: dict = {}


def plain_rows(name, cfg, tensors, reqs, rows, dtype):
    key = (name, dtype, tuple(sorted((rid, len(ids)) for rid, ids in reqs.items())))
    if key not in _PLAIN:
        # (against bfloat16 the plain sums need no 64 bits: half the time at the real widths)
        arith = torch.float32 if dtype == "bf16" and cfg["hidden_size"] >= 2048 else torch.float64
        wide = {k: v.to(arith) for k, v in tensors.items()}
        rounder = bf16_round if dtype == "bf16" else None
        _PLAIN[key] = {rid: plain_forward(cfg, wide, ids, dtype=arith, rounder=rounder, rows=rows[rid]).double().numpy()
                       for rid, ids in reqs.items()}
    return _PLAIN[key]


def _requests(cfg, count, lo, hi, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": random_tokens(int(rng.integers(lo, hi + 1)), cfg["vocab_size"], 500 + i) for i in range(count)}


def _count_product_rows(monkeypatch):
    """Notes the number of rows of every bfloat16 product that is launched."""
    from llmengine.ops import mfma
    rows = []
    inner = mfma.gemm_bf16

    def noting(a, w, out, *args, **kw):
        rows.append(a.shape[0])
        return inner(a, w, out, *args, **kw)
    monkeypatch.setattr(mfma, "gemm_bf16", noting)
    return rows


@pytest.mark.parametrize("graphs", [True, False], ids=["recorded", "plain"])
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("name,max_live,count", [("A", 24, 40), ("B", 24, 40), ("A", 70, 100), ("B", 70, 100),
                                                 ("1b", 24, 36), ("1b", 70, 90), ("3b", 24, 30), ("3b", 70, 80),
                                                 ("8b", 24, 30), ("8b", 70, 80)])
def test_many_live_requests_match_plain(zoo, name, max_live, count, dtype, graphs, monkeypatch):
    from llmengine import Engine
    if name in ("3b", "8b") and not graphs:
        pytest.skip("the larger widths run with recorded decode steps only (the plain implementation's time)")
    cfg, tensors, page = zoo[name]
    if name in ("3b", "8b"):                                        # (the same requests under both numbers of live ones)
        reqs = dict(list(_requests(cfg, 80, 62, 76, seed=5).items())[:count])
    else:
        reqs = _requests(cfg, count, 62, 100, seed=max_live)        # 40 and more decoded tokens each
    steps = batch_schedule(reqs, max_live, seed=max_live)
    # all rows of the tiny models; of the wide ones the first two, the prompt's last and every decoded one
    if cfg["hidden_size"] >= 2048:
        rows = {rid: sorted({0, 1} | set(range(max(2, len(ids) // 3) - 1, len(ids)))) for rid, ids in reqs.items()}
        steps = replay.want_only(steps, rows)
    else:
        rows = {rid: list(range(len(ids))) for rid, ids in reqs.items()}
    plain = plain_rows(name, cfg, tensors, reqs, rows, dtype)
    product_rows = _count_product_rows(monkeypatch) if dtype == "bf16" else None
    engine = Engine(None, dtype, _config=cfg, _tensors=dict(tensors), block_size=page, use_graphs=graphs)
    pages = replay.trace_peak_tokens(steps, round_to=page) // page  # so few that finished requests' pages are used again
    cache = engine.new_cache(pages, page, max_requests=max_live)
    got = replay.run_trace(engine, cache, steps)
    sizes = [sum(len(e["tokens"]) for e in st["entries"]) for st in steps]
    decode_steps = [len(st["entries"]) for st in steps if all(len(e["tokens"]) == 1 for e in st["entries"])]
    assert max(decode_steps) == max_live and len([s for s in decode_steps if s > 16]) >= 38
    # a portion beside more than 16 decoded tokens
    assert any(sum(len(e["tokens"]) == 1 for e in st["entries"]) > 16 and any(len(e["tokens"]) > 1 for e in st["entries"])
               for st in steps)
    if max_live == 70:
        assert max(sizes) > 64 and any(16 < s <= 64 for s in sizes)
    if product_rows is not None:
        assert any(16 < m <= 64 for m in product_rows), "no product of 17 to 64 rows ran"
        if max_live == 70:
            assert any(m > 64 for m in product_rows), "no product of more than 64 rows ran"
    if graphs:
        assert engine.runner.graph_replays > 20
    else:
        assert engine.runner.graph_replays == 0
    for rid, ids in reqs.items():
        assert sorted(got[rid]) == rows[rid], rid
        for i, pos in enumerate(rows[rid]):
            ref = plain[rid][i]
            err = np.abs(got[rid][pos].astype(np.float64) - ref).max() / np.abs(ref).max()
            assert err < TOL[dtype], f"request {rid} position {pos} of {len(ids)}: relative error {err:.3e}"
    assert all(cache.manager.free_pages(g) == cache.manager.num_pages(g) for g in cache.manager.groups)
    del engine
    torch.cuda.empty_cache()


# --- the same bits every time --------------------------------------------------------------
# A model wide enough that sums into the residual stream are cut over k when the order is free
# (k of 1,024 and more; the tiny models' sums are never cut).
WIDE_K = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 1024,
          "intermediate_size": 2048, "num_hidden_layers": 2, "num_attention_heads": 16,
          "num_key_value_heads": 4, "head_dim": 64, "vocab_size": 512, "max_position_embeddings": 1024,
          "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "tie_word_embeddings": False}


def _flat(got):
    return np.stack([got[rid][pos] for rid in sorted(got) for pos in sorted(got[rid])])


@pytest.mark.parametrize("graphs", [True, False], ids=["recorded", "plain"])
def test_deterministic_mode_repeats_itself_bit_for_bit(graphs):
    """bfloat16 with every sum in a fixed order: the same trace (portions, mixed batches of 1 to 40
    rows, decode steps) gives the same bits in a second run over another, scrambled pool. The
    default mode cuts sums over k and joins them with atomics: equal within rounding only."""
    from llmengine import Engine
    from llmengine.weights import random_state
    tensors = dict(random_state(WIDE_K, 5, torch.bfloat16, 0.03, 1.0, 0.05))
    reqs = _requests(WIDE_K, 30, 20, 70, seed=3)
    steps = batch_schedule(reqs, 20, portion=40, seed=4)
    pages = replay.trace_peak_tokens(steps, round_to=16) // 16
    runs = []
    for deterministic in (True, True, False):
        engine = Engine(None, "bf16", _config=WIDE_K, _tensors=dict(tensors), deterministic=deterministic,
                        use_graphs=graphs)
        cache = engine.new_cache(pages + 7 * len(runs), 16, max_requests=20)
        if runs:                                        # other physical pages than the first run had
            for i in range(5):
                cache.admit(f"junk{i}")
                engine.step(cache, [replay_entry(f"junk{i}", random_tokens(16 + 3 * i, 512, i))])
            for i in (3, 0, 4, 1, 2):
                cache.release(f"junk{i}")
        runs.append(_flat(replay.run_trace(engine, cache, steps)))
        del engine
    assert np.array_equal(runs[0], runs[1])
    scale = np.abs(runs[0]).max(axis=1, keepdims=True)
    # the free order: the same within bfloat16 rounding (a sum that differs in its last bit moves
    # stored activations across rounding boundaries)
    assert (np.abs(runs[2] - runs[0]) / scale).max() < TOL["bf16"]


def replay_entry(rid, tokens):
    from llmengine import StepEntry
    return StepEntry(rid, tokens, [])


@pytest.mark.parametrize("name", ["A", "B"])
def test_fp32_logits_do_not_depend_on_pages(zoo, name):
    """In 32-bit the logits are the same bits for pages of 4, 16 and 64 tokens and for any
    physical pages: the kernels' sums walk the keys in an order that the paging does not touch."""
    from llmengine import Engine
    cfg, tensors, _ = zoo[name]
    reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 40 + i) for i, n in enumerate([70, 9, 33, 100, 64, 17])}
    steps = replay.mixed(reqs, max_live=4, seed=9)
    engine = Engine(None, "fp32", _config=cfg, _tensors=dict(tensors))
    results = []
    for page, scramble in ((16, False), (16, True), (4, False), (64, True)):
        pages = replay.trace_peak_tokens(steps, round_to=page) // page + 6
        cache = engine.new_cache(pages, page, max_requests=6)
        if scramble:                                    # free pages come back in another order than 0, 1, 2, ..
            for i in range(5):
                cache.admit(f"junk{i}")
                engine.step(cache, [replay_entry(f"junk{i}", random_tokens(page + 1, cfg["vocab_size"], i))])
            for i in (2, 4, 0, 3, 1):
                cache.release(f"junk{i}")
        results.append(_flat(replay.run_trace(engine, cache, steps)))
    for other in results[1:]:
        assert np.array_equal(results[0], other)


# --- recorded decode steps between steps of other kinds ---------------------------------------
# A recorded decode step of 17 to 64 requests cuts its q/k/v product over k and adds the parts into a
# 32-bit buffer. Other kinds of step use the same scratch memory and leave values behind: a prompt
# portion of more than 64 rows where the projection cannot rotate in its epilogue (head sizes that are
# no power of two), a step of up to 16 rows where the fused decode kernel is refused (a width beyond
# what its LDS holds). The replay behind such a step must give what the plain implementation gives.
HEAD_96 = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 192,
           "intermediate_size": 320, "num_hidden_layers": 2, "num_attention_heads": 4,
           "num_key_value_heads": 2, "head_dim": 96, "vocab_size": 300, "max_position_embeddings": 512,
           "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "tie_word_embeddings": True}
WIDTH_5120 = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 5120,
              "intermediate_size": 1024, "num_hidden_layers": 1, "num_attention_heads": 40,
              "num_key_value_heads": 8, "head_dim": 128, "vocab_size": 300, "max_position_embeddings": 512,
              "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "tie_word_embeddings": False}
HEAD_48 = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_size": 144,
           "intermediate_size": 208, "num_hidden_layers": 2, "num_attention_heads": 6,
           "num_key_value_heads": 2, "head_dim": 48, "vocab_size": 331, "max_position_embeddings": 512,
           "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "tie_word_embeddings": False}
DISTURBED = {"head96": (HEAD_96, dict(seed=21, std=0.05, norm_mean=1.0, norm_std=0.1)),
             "width5120": (WIDTH_5120, dict(seed=22, std=0.01, norm_mean=1.0, norm_std=0.05)),
             "head48": (HEAD_48, dict(seed=23, std=0.05, norm_mean=1.0, norm_std=0.1))}


def disturbed_schedule(ids: dict, live: int, late: int, prompt: int = 8, portion: int = 70, dip: int = 10,
                       run: int = 3) -> tuple[list[dict], dict]:
    """`live` requests: their prompts in one step, then `run` decode steps of all of them (the first
    is recorded). Then `late` times: a new request's prompt portion of `portion` tokens beside the
    decoded tokens of all live ones (one of which ends there, so that the number stays), `run`
    decode steps, a decode step of only `dip` of the requests, `run` decode steps. Returns the
    steps and every request cut to the tokens that were fed."""
    names = list(ids)
    main, waiting = names[:live], names[live:live + late]
    pos = {rid: 0 for rid in names}
    steps: list[dict] = []

    def entry(rid, n):
        e = {"id": rid, "tokens": ids[rid][pos[rid]:pos[rid] + n], "want": list(range(n))}
        assert len(e["tokens"]) == n, f"{rid} is too short"
        pos[rid] += n
        return e

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    add([entry(r, prompt) for r in main])
    for _ in range(run):
        add([entry(r, 1) for r in main])
    for new in waiting:
        victim = main.pop(0)
        add([entry(r, 1) for r in [victim] + main] + [entry(new, portion)], end=[victim])
        main.append(new)
        for _ in range(run):
            add([entry(r, 1) for r in main])
        add([entry(r, 1) for r in main[:dip]])
        for _ in range(run):
            add([entry(r, 1) for r in main])
    steps[-1]["end"] = list(main)
    return steps, {rid: ids[rid][:pos[rid]] for rid in names if pos[rid]}


@pytest.mark.parametrize("graphs", [True, False], ids=["recorded", "plain"])
@pytest.mark.parametrize("name", list(DISTURBED))
def test_recorded_decode_steps_between_other_steps(name, graphs):
    from llmengine import Engine
    from llmengine.weights import random_state
    cfg, init = DISTURBED[name]
    tensors = dict(random_state(cfg, init["seed"], torch.bfloat16, init["std"], init["norm_mean"], init["norm_std"]))
    live, late = 24, 3
    ids = {f"r{i}": random_tokens(120, cfg["vocab_size"], 900 + i) for i in range(live + late)}
    steps, reqs = disturbed_schedule(ids, live, late)
    sizes = [(len(st["entries"]), sum(len(e["tokens"]) for e in st["entries"])) for st in steps]
    assert sizes[0][1] > max(t for _, t in sizes[1:]) > 64          # the first step sizes the scratch memory
    assert sum(1 for s, t in sizes if s == t == live) >= 6 * late + 3 and any(s == t <= 16 for s, t in sizes)
    rows = {rid: list(range(len(t))) for rid, t in reqs.items()}
    plain = plain_rows(name, cfg, tensors, reqs, rows, "bf16")
    engine = Engine(None, "bf16", _config=cfg, _tensors=dict(tensors), block_size=16, use_graphs=graphs)
    cache = engine.new_cache(replay.trace_peak_tokens(steps, round_to=16) // 16, 16, max_requests=live + 1)
    got = replay.run_trace(engine, cache, steps)
    if graphs:
        assert engine.runner.graph_replays >= 6 * late + 3
    worst = (0.0, None)
    for rid, t in reqs.items():
        for pos in range(len(t)):
            ref = plain[rid][pos]
            err = np.abs(got[rid][pos].astype(np.float64) - ref).max() / np.abs(ref).max()
            worst = max(worst, (err, (rid, pos)))
    assert worst[0] < TOL["bf16"], f"request and position {worst[1]}: relative error {worst[0]:.3e}"
    assert all(cache.manager.free_pages(g) == cache.manager.num_pages(g) for g in cache.manager.groups)
    del engine
    torch.cuda.empty_cache()


# --- random configurations with many live requests ---------------------------------------------
@pytest.mark.parametrize("case", list(range(14)) + [90])
def test_random_configurations_with_many_live_requests(case):
    """The random configurations of test_engine_gpu (head sizes from 16 to 256, odd numbers of heads
    and groups, widths in and out of the blocked layout, any page size) with 24 live requests and
    recorded decode steps: every route that a step of 17 to 64 rows, or a portion beside two dozen
    decoded tokens, can take at sizes that are not Llama's."""
    from llmengine import Engine
    from llmengine.weights import random_state
    from test_engine_gpu import _random_configuration
    cfg, page, _ = _random_configuration(case)
    tensors = dict(random_state(cfg, case, torch.bfloat16, 0.08, 1.0, 0.1))
    wide = {k: v.double() for k, v in tensors.items()}
    reqs = _requests(cfg, 34, 30, 64, seed=case)
    steps = batch_schedule(reqs, 24, portion=80, seed=case)
    for dtype, rounder in (("fp32", None), ("bf16", bf16_round)):
        plain = {rid: plain_forward(cfg, wide, ids, rounder=rounder).numpy() for rid, ids in reqs.items()}
        engine = Engine(None, dtype, _config=cfg, _tensors=dict(tensors), block_size=page)
        cache = engine.new_cache(replay.trace_peak_tokens(steps, round_to=page) // page, page, max_requests=24)
        got = replay.run_trace(engine, cache, steps)
        assert engine.runner.graph_replays > 10
        worst = max((np.abs(got[rid][pos].astype(np.float64) - plain[rid][pos]).max() / np.abs(plain[rid][pos]).max(),
                     rid, pos) for rid, ids in reqs.items() for pos in range(len(ids)))
        assert worst[0] < TOL[dtype], f"{cfg} page {page} {dtype}: request {worst[1]} position {worst[2]}: {worst[0]:.3e}"
        assert all(cache.manager.free_pages(g) == cache.manager.num_pages(g) for g in cache.manager.groups)
        del engine
    torch.cuda.empty_cache()
