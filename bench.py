#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers L] [--shape 1b|3b|8b]

By default the model has the layer sizes of Llama 3.2 1B (16 layers, width 2048, 32 query / 8 key-value
heads of 64, feed-forward 8192, vocabulary 128256, llama3 rope scaling, tied head) with seeded
random bfloat16 weights; token ids are seeded uniform random numbers. A "step" is one decode
step of the whole batch: the model over one token per request from the paged cache, the choice
of the next token (greedy) and its way back to the host; as in `Engine.generate`, a step is launched
on the tokens the device holds while the host still fetches those of the step before
(`Engine.greedy_chain`). Every request holds `context - steps -
warmup` tokens when decoding starts, put there by real prefill steps, so that the timed steps
run at the configured context length. One JSON line goes to stdout.

`--shape 3b` and `--shape 8b` take the layer sizes of Llama 3.2 3B and Llama 3.1 8B instead (for
measurements at further sizes and context lengths; the default run is the 1B shape).

`--phase mixed` times one step of continuous batching (a prompt portion beside decoded tokens of
other requests), `--phase portion` portions of one long prompt. `--phase serve` is another workload (with `--shape 3b`: 32 requests with prompts of 64 to 3,072
tokens and 128 to 512 new tokens each, 2,048 prompt tokens a step at most) through the
continuous-batching scheduler, prompt portions beside decoded tokens in every step.

Beside the headline value the line holds: `prefill` (one 2,048-token prompt, logits at its last
place), `roofline` (bytes the decode step has to read: every weight once plus the live
requests' cache, over its time, against 8 TB/s), `points` (decode at batch 1 and 64).
"""
from __future__ import annotations

import argparse
import random
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "llm-inference-engine-v6_amd"))

HBM_PEAK = 8.0e12            # bytes/s
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 2048, "intermediate_size": 8192, "num_hidden_layers": 16,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 64,
    "vocab_size": 128256, "max_position_embeddings": 131072, "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
    "tie_word_embeddings": True,
}

# Further shapes of the same architecture (--shape), for measurements beside the default one.
SHAPES = {
    "1b": LLAMA_1B,
    "3b": dict(LLAMA_1B, hidden_size=3072, intermediate_size=8192, num_hidden_layers=28, num_attention_heads=24,
               num_key_value_heads=8, head_dim=128),
    "8b": dict(LLAMA_1B, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32, num_attention_heads=32,
               num_key_value_heads=8, head_dim=128, tie_word_embeddings=False,
               rope_scaling=dict(LLAMA_1B["rope_scaling"], factor=8.0)),
}


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def layer_weight_elements(c: dict) -> int:
    H, FF = c["hidden_size"], c["intermediate_size"]
    q, kv = c["num_attention_heads"] * c["head_dim"], c["num_key_value_heads"] * c["head_dim"]
    return (q + 2 * kv) * H + H * q + 2 * FF * H + H * FF + 2 * H


def decode_bytes(c: dict, batch: int, ctx: float, wbytes: int) -> float:
    """Bytes a decode step has to read: every weight once, and the cache of the live requests."""
    # the output head's matrix once (tied or not, a decode step reads one vocabulary-sized matrix: the
    # embedding is only gathered from)
    weights = (c["num_hidden_layers"] * layer_weight_elements(c) + c["vocab_size"] * c["hidden_size"]
               + c["hidden_size"]) * wbytes
    kv = batch * ctx * 2 * c["num_key_value_heads"] * c["head_dim"] * wbytes * c["num_hidden_layers"]
    return weights + kv


def prefill_flops(c: dict, T: int) -> float:
    """Flops of one T-token prompt from an empty cache, logits at the last place only."""
    L, H = c["num_hidden_layers"], c["hidden_size"]
    q = c["num_attention_heads"] * c["head_dim"]
    gemm = 2.0 * T * L * (layer_weight_elements(c) - 2 * H)
    attn = L * 2.0 * 2.0 * q * (T * (T + 1) / 2)            # QK^T and PV over the causal half
    head = 2.0 * c["vocab_size"] * H
    return gemm + attn + head


def serve(args, engine, cfg: dict, gen, page: int) -> int:
    """Requests of mixed lengths through the continuous-batching scheduler: every step is one
    mixed batch (prompt portions under the token budget beside one token of every decoding
    request). The rate counts generated tokens over the wall time from the first step to the
    last, host work included."""
    import torch
    from llmengine import BlockManager, ContinuousBatchScheduler

    lo, hi = (int(x) for x in args.prompt_range.split(","))
    nlo, nhi = (int(x) for x in args.new_range.split(","))
    V = cfg["vocab_size"]
    prompts = [torch.randint(0, V, (int(torch.randint(lo, hi + 1, (1,), generator=gen)),), generator=gen).tolist()
               for _ in range(args.requests)]
    news = [int(torch.randint(nlo, nhi + 1, (1,), generator=gen)) for _ in range(args.requests)]
    pages = sum((len(p) + n + page - 1) // page for p, n in zip(prompts, news))
    runs = []
    manager = BlockManager(pages, page)                        # one pool for both runs: the second finds the decode
    for rep in range(2):                                       # steps' HIP graphs that the first recorded over it
        sched = ContinuousBatchScheduler(engine, manager, max_concurrent=args.max_concurrent,
                                         max_prefill_tokens_per_step=args.prefill_budget,
                                         temperature=args.temperature, seed=args.seed)
        for p, n in zip(prompts, news):
            sched.enqueue(p, n)
        torch.cuda.synchronize()
        t = time.perf_counter()
        sched.run_until_idle()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        results = sched.results
        generated = sum(len(r.token_ids) - r.prompt_len for r in results)
        reasons = sorted({r.finish_reason for r in results})
        runs.append((dt, generated, sched.steps))
        log(f"serve run {rep}: {len(results)} requests, {sum(map(len, prompts))} prompt tokens, {generated} generated "
            f"in {dt:.2f} s over {sched.steps} steps ({generated / dt:.0f} generated tok/s; finished: {reasons})")
        assert manager.free_blocks == pages, "pages were lost"
        del sched
    dt, generated, steps = runs[-1]
    prompt_tokens = sum(map(len, prompts))
    print(json.dumps({
        "metric": "serve_generated_tokens_per_second", "value": round(generated / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "dtype": args.dtype, "seconds": round(dt, 3), "steps": steps,
        "all_tokens_per_second": round((generated + prompt_tokens) / dt, 1),
        "config": {"model": args.shape, "layers": cfg["num_hidden_layers"], "requests": args.requests,
                   "prompt_range": args.prompt_range, "new_range": args.new_range, "prompt_tokens": prompt_tokens,
                   "generated_tokens": generated, "prefill_budget": args.prefill_budget,
                   "max_concurrent": args.max_concurrent, "page_size": page, "temperature": args.temperature},
    }), flush=True)
    return 0


def portion(args, engine, cfg: dict, gen, page: int) -> int:
    """A long prompt that arrives in portions (a prefill budget per step): the steps of --portion
    tokens once --context tokens are cached. Few rows over many keys."""
    import torch
    from llmengine import StepEntry
    V, n, ctx = cfg["vocab_size"], args.portion, args.context
    steps = max(4, min(args.steps, 16))
    cache = engine.new_cache((ctx + (steps + 2) * n) // page + 2, page, 1)
    cache.admit("p")
    for at in range(0, ctx, 2048):
        engine.step(cache, [StepEntry("p", torch.randint(0, V, (min(2048, ctx - at),), generator=gen).tolist(), [])])
    tokens = torch.randint(0, V, (n,), generator=gen).tolist()
    engine.step(cache, [StepEntry("p", tokens, [n - 1])])
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        engine.step(cache, [StepEntry("p", tokens, [n - 1])])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t) / steps * 1e3
    log(f"portions of {n} tokens behind {ctx}: {ms:.2f} ms a step")
    print(json.dumps({"metric": "portion_tokens_per_second", "value": round(n / (ms / 1e3), 1), "unit": "tokens/s",
                      "n_gpus": 1, "dtype": args.dtype, "ms_per_step": round(ms, 3), "steps": steps,
                      "config": {"model": args.shape, "layers": args.layers, "context": ctx, "portion": n,
                                 "page_size": page}}), flush=True)
    return 0


def mixed(args, engine, cfg: dict, gen, page: int) -> int:
    """The step that continuous batching runs most: a prompt portion of --portion tokens of one
    request (behind --context cached tokens) beside one decoded token of --batch other requests
    (--decode-len tokens and up to 800 more each, 700 to 1,500 by default). Timed as the engine launches it, and once more with the same
    launches recorded as a HIP graph and replayed, which is the GPU's time alone."""
    import torch
    from llmengine import StepEntry
    V, n, nd = cfg["vocab_size"], args.portion, args.batch
    steps = max(4, min(args.steps, 32))
    lens = [args.decode_len + (800 * i) // max(nd, 1) for i in range(nd)]
    cache = engine.new_cache((args.context + n + sum(lens)) // page + nd + 4, page, nd + 1)
    for i, ln in enumerate(lens):
        cache.admit(i)
        engine.step(cache, [StepEntry(i, torch.randint(0, V, (ln,), generator=gen).tolist(), [])])
    cache.admit("p")
    for at in range(0, args.context, 2048):
        engine.step(cache, [StepEntry("p", torch.randint(0, V, (min(2048, args.context - at),), generator=gen).tolist(), [])])
    entries = [StepEntry("p", torch.randint(0, V, (n,), generator=gen).tolist(), [n - 1])] + [
        StepEntry(i, [7], [0]) for i in range(nd)]
    runner, mgr = engine.runner, cache.manager
    # the same tokens at the same places every time: pages are reserved once and never committed
    assert mgr.reserve_batch([(e.request_id, len(e.tokens)) for e in entries])
    ctx, rows = runner._build_context(cache, entries)

    def forward():
        return runner.model.forward(ctx, cache.storage.layers, rows)
    for _ in range(3):
        forward()
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        forward()
    torch.cuda.synchronize()
    launched = (time.perf_counter() - t) / steps * 1e3
    graph = torch.cuda.CUDAGraph()
    import gc
    gc.disable()                            # (a collection must not free device memory while launches are recorded)
    try:
        with torch.cuda.graph(graph):
            forward()
    finally:
        gc.enable()
    graph.replay()
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    gpu = (time.perf_counter() - t) / steps * 1e3
    log(f"mixed step, {n} prompt tokens behind {args.context} beside {nd} decoded tokens: {launched:.3f} ms launched "
        f"by the engine, {gpu:.3f} ms as a recorded graph")
    print(json.dumps({"metric": "mixed_step_tokens_per_second", "value": round((n + nd) / (launched / 1e3), 1),
                      "unit": "tokens/s", "n_gpus": 1, "dtype": args.dtype, "ms_per_step": round(launched, 3),
                      "ms_per_step_gpu_only": round(gpu, 3), "steps": steps,
                      "config": {"model": args.shape, "layers": args.layers, "context": args.context, "portion": n,
                                 "decode_requests": nd, "page_size": page}}), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096, help="context length the decode steps run at")
    ap.add_argument("--context-range", default="", help="decode: contexts drawn uniformly from [a, b] (seeded) instead "
                                                        "of --context for every request")
    ap.add_argument("--decode-order", default="as-drawn", choices=["as-drawn", "longest-first", "rounds"],
                    help="decode with --context-range: the order of the requests in the batch (the scheduler puts "
                         "the longest first)")
    ap.add_argument("--round", type=int, default=32, help="decode order 'rounds': requests per round")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (a multiple of 16 for the bf16 kernels)")
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes: Llama 3.2 1B (the default), 3.2 3B, 3.1 8B")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (named in config)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--phase", default="all", choices=["all", "prefill", "decode", "serve", "portion", "mixed"],
                    help="run only one part (for profiling); the JSON line then lacks the other. 'serve' is another "
                         "workload: requests of mixed lengths through the continuous-batching scheduler; 'portion': "
                         "steps of --portion prompt tokens of one request behind --context tokens; 'mixed': such a "
                         "portion beside one decoded token of --batch other requests")
    ap.add_argument("--portion", type=int, default=256, help="portion: prompt tokens a step")
    ap.add_argument("--decode-len", type=int, default=700, help="mixed: tokens of the shortest decoding request "
                                                                "(the longest has 800 more)")
    ap.add_argument("--requests", type=int, default=32, help="serve: number of requests")
    ap.add_argument("--prompt-range", default="64,3072", help="serve: prompt lengths, uniform in [a, b]")
    ap.add_argument("--new-range", default="128,512", help="serve: new tokens per request, uniform in [a, b]")
    ap.add_argument("--prefill-budget", type=int, default=2048, help="serve: max_prefill_tokens_per_step")
    ap.add_argument("--max-concurrent", type=int, default=32, help="serve: live requests at a time")
    ap.add_argument("--temperature", type=float, default=0.0, help="serve: sampling temperature (0 is greedy)")
    ap.add_argument("--choices", default="", help="fields of llmengine.ops.KernelChoices to set, name=value,... "
                                                  "(for comparisons: which kernels and launch plans the steps may use)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch
    from llmengine import Engine, StepEntry

    full_layers = SHAPES[args.shape]["num_hidden_layers"]
    args.layers = args.layers or full_layers
    cfg = dict(SHAPES[args.shape], num_hidden_layers=args.layers)
    wbytes = 2 if args.dtype == "bf16" else 4
    t0 = time.time()
    log(f"building the model ({args.layers} layers, {args.dtype}) with random weights")
    choices = None
    if args.choices:
        from llmengine.ops import KernelChoices
        choices = KernelChoices()
        for item in args.choices.split(","):
            name, _, value = item.partition("=")
            if not hasattr(choices, name.strip()):
                raise SystemExit(f"--choices: KernelChoices has no field {name.strip()!r}")
            old = getattr(choices, name.strip())
            value = value.strip()
            setattr(choices, name.strip(), None if value == "None" else (value == "True") if isinstance(old, bool)
                    else float(value) if isinstance(old, float) else int(value))
    engine = Engine.from_random(cfg, args.seed, args.dtype, std=0.02, kernel_choices=choices)
    runner = engine.runner
    log(f"model on the device after {time.time() - t0:.1f} s")
    gen = torch.Generator().manual_seed(args.seed + 1)
    V = cfg["vocab_size"]
    page = args.page_size

    def sync():
        torch.cuda.synchronize()

    if args.phase == "serve":
        return serve(args, engine, cfg, gen, page)
    if args.phase == "portion":
        return portion(args, engine, cfg, gen, page)
    if args.phase == "mixed":
        return mixed(args, engine, cfg, gen, page)

    # ---- prefill: one prompt, logits at its last place ----
    T = args.prefill_tokens
    prefill = None
    if args.phase in ("all", "prefill"):
        prompt = torch.randint(0, V, (T,), generator=gen).tolist()
        cache = engine.new_cache((T + page - 1) // page + 1, page, 1)
        pre_ms = []
        for rep in range(8):                                   # the first warms up; the best of the rest counts
            cache.admit("p")
            sync()
            t = time.perf_counter()
            engine.step(cache, [StepEntry("p", prompt, [T - 1])])
            sync()
            pre_ms.append((time.perf_counter() - t) * 1e3)
            cache.release("p")
        prefill_ms = min(pre_ms[1:])
        flops = prefill_flops(cfg, T)
        prefill = {"value": round(T / (prefill_ms / 1e3), 1), "tokens": T, "ms": round(prefill_ms, 3),
                   "frac": round(flops / (prefill_ms / 1e3) / PEAK_FLOPS[args.dtype], 4)}
        log(f"prefill {T} tokens: {prefill_ms:.2f} ms ({prefill['value']:.0f} tok/s, {prefill['frac']:.3f} of peak)")
        del cache
    if args.phase == "prefill":
        print(json.dumps({"metric": "prefill_tokens_per_second", "value": prefill["value"], "unit": "tokens/s",
                          "n_gpus": 1, "dtype": args.dtype, "prefill": prefill}), flush=True)
        return 0

    # ---- decode ----
    def decode_run(batch: int, steps: int, warmup: int):
        if args.context_range:
            lo, hi = (int(x) for x in args.context_range.split(","))
            rnd = random.Random(args.seed * 1000 + batch)
            starts = [rnd.randint(lo, hi) for _ in range(batch)]
        else:
            starts = [args.context - steps - warmup] * batch
        if min(starts) < 1:
            raise SystemExit("--context must exceed --steps + --warmup")
        pages = sum((st + steps + warmup + page - 1) // page + 1 for st in starts)
        cache = engine.new_cache(pages, page, batch)
        ids = [f"r{i}" for i in range(batch)]
        for rid in ids:
            cache.admit(rid)
        chunk = 8192
        sync()
        t_fill = time.perf_counter()
        for rid, start_ctx in zip(ids, starts):                # real prefill fills the pages
            toks = torch.randint(0, V, (start_ctx,), generator=gen).tolist()
            for s in range(0, start_ctx, chunk):
                engine.step(cache, [StepEntry(rid, toks[s:s + chunk], [])])
        sync()
        t_fill = time.perf_counter() - t_fill
        log(f"filled the cache: {batch} requests, {sum(starts)} tokens in portions of {chunk} in {t_fill:.2f} s "
            f"({sum(starts) / t_fill:.0f} tok/s, token generation on the host included)")
        if args.decode_order == "longest-first":
            ids = [rid for _, rid in sorted(zip(starts, ids), key=lambda p: -p[0])]
        elif args.decode_order == "rounds":
            from llmengine.engine.scheduler import rounds_order
            by_length = sorted(range(batch), key=lambda i: -starts[i])
            ids = [ids[by_length[i]] for i in rounds_order(batch, args.round)]
        last = torch.randint(0, V, (batch,), generator=gen).tolist()

        # greedy decoding as `Engine.generate` runs it: every step's tokens feed the next on the device, and
        # the host fetches a step's tokens while the next step runs
        last = engine.greedy_chain(cache, ids, last, warmup)[-1] if warmup > 0 else last
        sync()
        t = time.perf_counter()
        chosen = engine.greedy_chain(cache, ids, last, steps)
        sync()
        dt = time.perf_counter() - t
        assert len(chosen) == steps and all(len(c) == batch for c in chosen)
        for rid in ids:
            cache.release(rid)
        mean_ctx = sum(starts) / batch + warmup + (steps + 1) / 2.0
        return dt / steps, mean_ctx

    log(f"decode: batch {args.batch}, context {args.context}")
    step_s, mean_ctx = decode_run(args.batch, args.steps, args.warmup)
    value = args.batch / step_s
    nbytes = decode_bytes(cfg, args.batch, mean_ctx, wbytes)
    roofline = {"bound": "hbm", "achieved": round(nbytes / step_s / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": round(nbytes / step_s / HBM_PEAK, 4)}
    log(f"decode b{args.batch}: {step_s * 1e3:.3f} ms/step, {value:.0f} tok/s, {roofline['frac']:.3f} of HBM peak")
    points = {}
    for b in [int(x) for x in args.points.split(",") if x.strip()]:
        s, c = decode_run(b, max(16, args.steps // 2), max(4, args.warmup // 2))
        points[f"decode_b{b}"] = round(b / s, 1)
        points[f"decode_b{b}_hbm_frac"] = round(decode_bytes(cfg, b, c, wbytes) / s / HBM_PEAK, 4)
        log(f"decode b{b}: {s * 1e3:.3f} ms/step, {b / s:.0f} tok/s")

    line = {
        "metric": "decode_tokens_per_second", "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic (seeded random weights and token ids)",
        "config": {
            "model": {"1b": "llama-3.2-1b-shape", "3b": "llama-3.2-3b-shape", "8b": "llama-3.1-8b-shape"}[args.shape],
            "global_batch": args.batch, "seq_len": args.context,
            "parallelism": "single-gpu", "layers": args.layers, "layers_full_model": full_layers,
            "hidden_size": cfg["hidden_size"], "intermediate_size": cfg["intermediate_size"],
            "num_attention_heads": cfg["num_attention_heads"], "num_key_value_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "vocab_size": V, "tie_word_embeddings": cfg["tie_word_embeddings"],
            "rope": f"theta 5e5, llama3 scaling {cfg['rope_scaling']['factor']:g}/1/4/8192", "page_size": page,
            "prefill_tokens": T, "decode_context": args.context_range or args.context, "sampling": "greedy",
        },
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
