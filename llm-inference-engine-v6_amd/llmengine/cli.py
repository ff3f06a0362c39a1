"""Command line: generate from token ids with a model folder or a random model.

    llmengine-cli --model DIR --prompt-ids 1,2,3 --max-new-tokens 16
    llmengine-cli --random CONFIG.json --seed 0 --prompt-file prompts.txt --temperature 0.8

The reference has no command line of its own; the options carry the names of its
Python interface (src/bindings.cpp:150-160,312-316): dtype, max_new_tokens,
num_blocks, block_size, max_concurrent, max_prefill_tokens_per_step. One prompt is
run through `Engine.generate`; several (a file with one comma- or space-separated
list of ids per line) go through the continuous-batching scheduler. Output: one
JSON object per request with its ids and finish reason.
"""
from __future__ import annotations

import argparse
import json
import sys


def _ids(text: str) -> list[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="llmengine-cli", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--model", help="folder with config.json and *.safetensors")
    src.add_argument("--random", metavar="CONFIG.json", help="a config.json; weights are random")
    ap.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--dtype", default="bf16", choices=["fp32", "bf16", "float32", "bfloat16"])
    pr = ap.add_mutually_exclusive_group(required=True)
    pr.add_argument("--prompt-ids", help="token ids, comma separated")
    pr.add_argument("--prompt-file", help="one list of token ids per line")
    ap.add_argument("--max-new-tokens", type=int, default=16)
    ap.add_argument("--temperature", type=float, default=0.0, help="0 is greedy")
    ap.add_argument("--sampler-seed", type=int, default=0)
    ap.add_argument("--block-size", type=int, default=16, help="tokens per cache page")
    ap.add_argument("--num-blocks", type=int, default=0, help="pages in the pool (0: enough for all requests)")
    ap.add_argument("--max-concurrent", type=int, default=64)
    ap.add_argument("--prefill-budget", type=int, default=256, help="max_prefill_tokens_per_step")
    ap.add_argument("--max-context", type=int, default=None,
                    help="lower the model's position limit (max_position_embeddings) to this")
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)

    from . import BlockManager, ContinuousBatchScheduler, Engine
    if args.prompt_ids is not None:
        prompts = [_ids(args.prompt_ids)]
    else:
        with open(args.prompt_file) as f:
            prompts = [_ids(line) for line in f if line.strip()]
    if not prompts:
        ap.error("no prompts given")

    kw = dict(device=args.device, temperature=args.temperature, sampler_seed=args.sampler_seed, block_size=args.block_size,
              max_context=args.max_context)
    if args.model:
        engine = Engine(args.model, args.dtype, **kw)
    else:
        with open(args.random) as f:
            engine = Engine.from_random(json.load(f), args.seed, args.dtype, **kw)

    if len(prompts) == 1:
        ids, finish = engine.generate(prompts[0], args.max_new_tokens)
        print(json.dumps({"seq_id": 0, "prompt_len": len(prompts[0]), "token_ids": ids, "finish_reason": finish}))
        return 0
    need = sum((len(p) + args.max_new_tokens + args.block_size - 1) // args.block_size for p in prompts)
    blocks = BlockManager(args.num_blocks or need, args.block_size)
    sched = ContinuousBatchScheduler(engine, blocks, args.max_concurrent, args.prefill_budget,
                                     temperature=args.temperature, seed=args.sampler_seed)
    for p in prompts:
        sched.enqueue(p, args.max_new_tokens)
    sched.run_until_idle()
    for r in sched.results:
        print(json.dumps({"seq_id": r.seq_id, "prompt_len": r.prompt_len, "token_ids": r.token_ids,
                          "finish_reason": r.finish_reason}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
