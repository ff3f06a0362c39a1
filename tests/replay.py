"""Replay schedules for tests: ways of cutting the same requests into steps.

A trace is a list of steps in the format that bin/trace_run reads:
    {"step": i, "entries": [{"id", "tokens", "want"}], "end": [ids]}
Builders below cut given token sequences into steps; `run_trace` drives the engine's
step function with a trace and returns, per request, the logits at every position
that was wanted; `trace_peak_tokens` says how large the page pool must be.
"""
from __future__ import annotations

import numpy as np


def whole(requests: dict) -> list[dict]:
    """Each request alone and whole: one step, logits everywhere."""
    steps = []
    for i, (rid, ids) in enumerate(requests.items()):
        steps.append({"step": i, "entries": [{"id": rid, "tokens": list(ids), "want": list(range(len(ids)))}],
                      "end": [rid]})
    return steps


def tail_one_by_one(requests: dict, tail: int = 32) -> list[dict]:
    """Most of a request in one step, the last `tail` tokens one by one."""
    steps = []
    for rid, ids in requests.items():
        head = max(1, len(ids) - tail) if len(ids) > 1 else 1
        cuts = [head] + [1] * (len(ids) - head)
        pos = 0
        for n in cuts:
            steps.append({"step": len(steps),
                          "entries": [{"id": rid, "tokens": list(ids[pos:pos + n]), "want": list(range(n))}],
                          "end": [rid] if pos + n == len(ids) else []})
            pos += n
    return steps


def portions(requests: dict, sizes=(7, 5, 3, 2, 11, 2, 4)) -> list[dict]:
    """Portions of changing size, down to two tokens (and a last remainder)."""
    steps = []
    for rid, ids in requests.items():
        pos, k = 0, 0
        while pos < len(ids):
            n = min(sizes[k % len(sizes)], len(ids) - pos)
            k += 1
            steps.append({"step": len(steps),
                          "entries": [{"id": rid, "tokens": list(ids[pos:pos + n]), "want": list(range(n))}],
                          "end": [rid] if pos + n == len(ids) else []})
            pos += n
    return steps


def mixed(requests: dict, max_live: int = 4, prompt_frac: float = 0.6, sizes=(5, 2, 9, 3, 2, 6), seed: int = 0
          ) -> list[dict]:
    """Up to `max_live` requests at a time. Each request's first part runs in portions of changing
    size, the rest token by token; portions of some requests share steps with single tokens of
    others; a request sometimes sits out a step. Finished requests make room for waiting ones."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live: list[dict] = []
    steps = []
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, ids = waiting.pop(0)
            live.append({"id": rid, "ids": list(ids), "pos": 0,
                         "prompt": max(1, int(len(ids) * prompt_frac))})
        entries, ended = [], []
        for r in live:
            if len(live) > 1 and rng.random() < 0.2:
                continue                                  # left out of this step
            left = len(r["ids"]) - r["pos"]
            if r["pos"] < r["prompt"]:
                n = min(sizes[k % len(sizes)], r["prompt"] - r["pos"])
                k += 1
            else:
                n = 1
            n = min(n, left)
            entries.append({"id": r["id"], "tokens": r["ids"][r["pos"]:r["pos"] + n], "want": list(range(n))})
            r["pos"] += n
            if r["pos"] == len(r["ids"]):
                ended.append(r["id"])
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        live = [r for r in live if r["id"] not in ended]
    return steps


def trace_peak_tokens(steps: list[dict], round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to a multiple of round_to."""
    held: dict = {}
    peak = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return peak


def want_only(steps: list[dict], places: dict) -> list[dict]:
    """The same steps with logits wanted only at `places[request id]` (positions in the request)."""
    out, done = [], {}
    for st in steps:
        entries = []
        for e in st["entries"]:
            start = done.get(e["id"], 0)
            keep = set(places[e["id"]])
            entries.append({"id": e["id"], "tokens": e["tokens"],
                            "want": [w for w in e["want"] if start + w in keep]})
            done[e["id"]] = start + len(e["tokens"])
        out.append({"step": st["step"], "entries": entries, "end": st["end"]})
    return out


def run_trace(engine, cache, steps: list[dict]) -> dict:
    """Drives engine.step; returns {request id: {position: logits row (numpy)}}."""
    from llmengine import StepEntry
    out: dict = {}
    done: dict = {}
    for st in steps:
        entries = []
        for e in st["entries"]:
            if not cache.manager.is_live(e["id"]):
                cache.admit(e["id"])
                done[e["id"]] = 0
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = engine.step(cache, entries)
        rows = logits.cpu().numpy() if logits is not None else None
        r = 0
        for e in st["entries"]:
            for w in e["want"]:
                out.setdefault(e["id"], {})[done[e["id"]] + w] = rows[r]
                r += 1
            done[e["id"]] += len(e["tokens"])
        for rid in st["end"]:
            cache.release(rid)
        cache.manager.check()
    return out
