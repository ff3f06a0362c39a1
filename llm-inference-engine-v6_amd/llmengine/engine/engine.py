"""The Python entry point: `Engine(model_dir, dtype).generate(ids, max_new_tokens)`.

Names and meanings follow the reference's binding (src/bindings.cpp:150-266,
276-335): `Engine(model_dir, dtype="fp32")`, `.generate(prompt_ids,
max_new_tokens) -> (ids, "stop" | "length")`, `.forward_logits(ids) -> [T, V]`,
properties `dtype`, `cfg`, `max_pos`, `weight_names()`, `has_weight(name)`, and
`BlockManager(num_blocks, block_size, ...)` with `num_blocks`, `block_size`,
`free_blocks`. dtype is "fp32" (everything in true 32-bit) or "bf16" (weights,
activations and cache in bfloat16; accumulation, norms, softmax, rotation and the
residual stream in 32-bit; logits 32-bit). All forward passes of an engine are
serialized by one lock, as the reference's are (include/llmengine/engine.hpp:158).
"""
from __future__ import annotations

import threading
from typing import Sequence

import numpy as np
import torch

from ..config.base import read_model_json
from ..config.registry import architecture_name, parse_config, resolve
from ..parts.base import Placement
from ..sampling import Sampler, uniform_draw
from ..weights import TensorIndex, load_model_weights, load_state_dict, random_state
from .step import CacheContext, CapacityError, ModelRunner, StepCommittedError, StepEntry

_DTYPES = {"fp32": torch.float32, "float32": torch.float32, "bf16": torch.bfloat16,
           "bfloat16": torch.bfloat16}


def parse_dtype(name: str) -> torch.dtype:
    try:
        return _DTYPES[name]
    except KeyError:
        raise ValueError(f"dtype must be 'fp32' | 'bf16', got: {name}") from None


def require_gpu(device: str | torch.device = "cuda:0") -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("this engine runs on an AMD GPU only: no HIP device is visible "
                           f"(asked for {device}); there is no CPU path")
    return device


class BlockManager:
    """The geometry of a page pool (the reference's constructor also takes the
    layer and head sizes, which here come from the model; they are accepted and
    checked when given)."""

    def __init__(self, num_blocks: int, block_size: int, num_layers: int | None = None,
                 num_kv_heads: int | None = None, head_dim: int | None = None):
        for name, v in (("num_blocks", num_blocks), ("block_size", block_size)):
            if v is None or int(v) <= 0:
                raise ValueError("BlockManager: non-positive dim")
        for v in (num_layers, num_kv_heads, head_dim):
            if v is not None and int(v) <= 0:
                raise ValueError("BlockManager: non-positive dim")
        self._num_blocks, self._block_size = int(num_blocks), int(block_size)
        self.dims = (num_layers, num_kv_heads, head_dim)
        self._cache: CacheContext | None = None

    num_blocks = property(lambda self: self._num_blocks)
    block_size = property(lambda self: self._block_size)

    @property
    def free_blocks(self) -> int:
        if self._cache is None:
            return self._num_blocks
        return min(self._cache.manager.free_pages(g) for g in self._cache.manager.groups)


class Engine:
    def __init__(self, model_dir: str | None, dtype: str = "fp32", *, device: str = "cuda:0",
                 max_prefill_tokens_per_step: int = 8192, temperature: float = 0.0, sampler_seed: int = 0,
                 block_size: int = 16, use_graphs: bool = True, max_context: int | None = None,
                 deterministic: bool = False, kernel_choices=None, _config: dict | None = None, _tensors=None):
        self._dtype_name = {"float32": "fp32", "bfloat16": "bf16"}.get(dtype, dtype)
        self._torch_dtype = parse_dtype(dtype)
        if _config is None:
            cfg_dict, gen = read_model_json(model_dir)
        else:
            cfg_dict, gen = _config, None
        if max_context is not None:
            # the position limit may be lowered (never raised): the rotation table is built that far
            if int(max_context) < 1:
                raise ValueError("Engine: max_context must be >= 1")
            have = cfg_dict.get("max_position_embeddings")
            if isinstance(have, int) and have > int(max_context):
                cfg_dict = dict(cfg_dict, max_position_embeddings=int(max_context))
        self.model_dir = model_dir
        self._cfg_dict = cfg_dict
        self._arch = resolve(architecture_name(cfg_dict))
        self.cfg = self._arch.parse_config(cfg_dict, gen, architecture=self._arch.name)
        self._index_names: list[str] | None = None
        self._aliases: dict[str, str] | None = None
        if model_dir is not None and _tensors is None:
            index = TensorIndex(model_dir)          # parse headers now: malformed files fail here
            self._index_names = index.names()
            index.close()
        self._tensors = _tensors
        self._device_name = device
        self._runner: ModelRunner | None = None
        self._lock = threading.RLock()
        self.sampler = Sampler(temperature, sampler_seed)
        self._samplers = {(self.sampler.temperature, self.sampler.seed): self.sampler}   # kept: they hold device rows
        self.block_size = int(block_size)
        self.prefill_chunk = int(max_prefill_tokens_per_step)
        self._own_cache: CacheContext | None = None
        self.use_graphs = bool(use_graphs)
        # deterministic: every sum in one fixed order, so that the same steps give the same bits in
        # every run (bfloat16 products into the residual stream are otherwise cut over k and joined
        # with atomics in the order the workgroups happen to finish).
        self.deterministic = bool(deterministic)
        # which kernels the operations may choose and where launch plans change shape (ops.KernelChoices;
        # None: the defaults): for tests and measurements
        self.kernel_choices = kernel_choices

    # ---- construction from random weights ----
    @classmethod
    def from_random(cls, config: dict, seed: int = 0, dtype: str = "bf16", *, std: float = 0.02,
                    norm_mean: float = 1.0, norm_std: float = 0.0, **kwargs) -> "Engine":
        """An engine over seeded random weights that are never written to disk."""
        store = torch.float32 if parse_dtype(dtype) == torch.float32 else torch.bfloat16
        tensors = dict(random_state(config, seed, store, std, norm_mean, norm_std))
        return cls(None, dtype, _config=config, _tensors=tensors, **kwargs)

    # ---- properties of the reference's binding ----
    @property
    def dtype(self) -> str:
        return self._dtype_name

    @property
    def max_pos(self) -> int:
        return self.cfg.max_pos

    @property
    def vocab_size(self) -> int:
        return self.cfg.vocab_size

    @property
    def eos_token_ids(self):
        return self.cfg.eos_token_ids

    def weight_names(self) -> list[str]:
        """The checkpoint's tensor names, plus the second names under which the model knows some
        of them (a tied head answers to the embedding's name and to its own)."""
        names = set(self._index_names if self._index_names is not None else self._tensors)
        if self._aliases is None:
            self._aliases = self._arch.build_model(self.cfg).named_aliases()     # (the tree alone: no tensors)
        for alias, target in self._aliases.items():
            if target in names:
                names.add(alias)
        return sorted(names)

    def has_weight(self, name: str) -> bool:
        return name in self.weight_names()

    # ---- the model on the device (made at first use, so that bad requests are
    #      refused before a bad checkpoint is: src/engine.cpp:719-742) ----
    @property
    def runner(self) -> ModelRunner:
        with self._lock:
            if self._runner is None:
                device = require_gpu(self._device_name)
                from ..ops import library
                library()                               # fails loudly if the kernels are missing
                model = self._arch.build_model(self.cfg)
                refused = model.tree_refusals()
                if refused:
                    raise ValueError("this engine's kernels do not take this model: " + "; ".join(refused))
                placement = Placement(device, self._torch_dtype)
                with torch.cuda.device(device):
                    if self._tensors is not None:
                        load_state_dict(model, self._tensors, placement)
                        self._tensors = {k: None for k in self._tensors}    # keep the names only
                    else:
                        load_model_weights(model, self.model_dir, placement)
                self._runner = ModelRunner(model, self._torch_dtype, device, use_graphs=self.use_graphs,
                                           deterministic=self.deterministic, choices=self.kernel_choices)
            return self._runner

    @property
    def model(self):
        return self.runner.model

    @property
    def decode_round(self) -> int:
        """What the scheduler orders a step's decoding requests by: the number that the model's first mixer
        with such a number gives (Mixer.decode_round), 0 if none has one."""
        for layer in self.model.layers:
            mixer = getattr(layer, "mixer", None)
            n = int(mixer.decode_round()) if mixer is not None else 0
            if n > 0:
                return n
        return 0

    @property
    def step_rows_round(self) -> tuple[int, int]:
        """(rows, most): steps of up to `most` rows more than a multiple of `rows` run those rows through the
        matrix products in launches of their own (ops.mfma.tail_rows); the scheduler avoids such steps.
        (0, 0) where the products do no such thing."""
        ch = self.runner.choices
        if self._torch_dtype != torch.bfloat16 or not ch.fast_gemm or not ch.tail_rows_apart:
            return (0, 0)
        from ..ops import mfma
        return (mfma.TAIL_ROWS_ROUND, int(ch.tail_rows_most))

    # ---- caches ----
    def new_cache(self, num_blocks: int, block_size: int | None = None, max_requests: int = 64) -> CacheContext:
        with torch.cuda.device(self.runner.device):
            return self.runner.new_cache(int(num_blocks), int(block_size or self.block_size), int(max_requests))

    def open_cache(self, block_manager: BlockManager, max_requests: int) -> CacheContext:
        """The device pool behind a `BlockManager` (made once per manager)."""
        n_layers, n_kv, hd = block_manager.dims
        for given, have, what in ((n_layers, getattr(self.cfg, "num_hidden_layers", None), "num_layers"),
                                  (n_kv, getattr(self.cfg, "num_key_value_heads", None), "num_kv_heads"),
                                  (hd, getattr(self.cfg, "head_dim", None), "head_dim")):
            if given is not None and have is not None and int(given) != int(have):
                raise ValueError(f"BlockManager: {what}={given} does not match the model's {have}")
        if block_manager._cache is None or block_manager._cache.max_requests < max_requests:
            block_manager._cache = self.new_cache(block_manager.num_blocks, block_manager.block_size, max_requests)
        return block_manager._cache

    # ---- the step function ----
    def step(self, cache: CacheContext, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        with self._lock, torch.cuda.device(self.runner.device):
            return self.runner.step(cache, entries, max_position=self.max_pos)

    def run_step(self, cache: CacheContext, entries, draws, temperature: float = 0.0, seed: int = 0) -> list[int]:
        """A step plus the choice of a token for every wanted row (the scheduler's call). A failure
        before the step is committed to the cache raises what it is and has changed nothing; one
        behind that raises StepCommittedError."""
        with self._lock, torch.cuda.device(self.runner.device):
            # a step of single decoded tokens is one recorded launch that ends in the choice of the tokens
            uniforms = None
            if temperature > 0.0 and self.runner.use_graphs and len(draws) == len(entries):
                uniforms = [uniform_draw(seed, r, i) for r, i in draws]
            tokens = self.runner.step_choosing(cache, entries, max_position=self.max_pos, temperature=temperature,
                                             uniforms=uniforms)
            if tokens is not None:
                return tokens
            logits = self.runner.step(cache, entries, max_position=self.max_pos)
            if logits is None:
                return []
            try:
                sampler = self._samplers.get((float(temperature), int(seed)))
                if sampler is None:
                    if len(self._samplers) >= 64:
                        self._samplers = {(self.sampler.temperature, self.sampler.seed): self.sampler}
                    sampler = self._samplers[(float(temperature), int(seed))] = Sampler(temperature, seed)
                return sampler.choose(logits, draws)
            except BaseException as e:                  # (the cache has moved on: the caller must not run the step again)
                raise StepCommittedError(f"the step ran, but no tokens were chosen: {e}") from e

    def greedy_chain(self, cache: CacheContext, request_ids: Sequence, tokens: Sequence[int], steps: int
                     ) -> list[list[int]]:
        """`steps` greedy decode steps of the live requests `request_ids`, the first on `tokens` (one per
        request), every later one on the tokens the step before it chose. Those stay on the device: a
        step is launched before the host has fetched the tokens of the one before, so the host's work
        for a step runs beside the device's. Returns every step's tokens. (Stopping is the caller's
        business: `generate` runs the same loop with its own check.)"""
        ids = list(request_ids)
        first = self._validate_ids(tokens, "greedy_chain")
        if len(first) != len(ids):
            raise ValueError("greedy_chain: one token per request")
        out: list[list[int]] = []
        if steps <= 0:
            return out
        with self._lock, torch.cuda.device(self.runner.device):
            runner = self.runner
            if not runner.use_graphs:
                last = first
                for _ in range(steps):
                    last = self.run_step(cache, [StepEntry(r, [t], [0]) for r, t in zip(ids, last)], None)
                    out.append(last)
                return out
            pending = runner.launch_choosing(cache, ids, first, self.max_pos)
            for i in range(1, steps + 1):
                ahead = runner.launch_choosing(cache, ids, None, self.max_pos) if i < steps else None
                last = runner.chosen_tokens(pending)
                out.append(last)
                if i < steps and ahead is None:          # (the recording changed: the tokens go through the host once)
                    ahead = runner.launch_choosing(cache, ids, last, self.max_pos)
                pending = ahead
        return out

    # ---- whole-sequence logits (src/engine.cpp:694-716) ----
    def _validate_ids(self, ids: Sequence[int], what: str) -> list[int]:
        ids = [int(t) for t in ids]
        V = self.cfg.vocab_size
        for t in ids:
            if t < 0 or t >= V:
                raise ValueError(f"{what}: token id {t} out of range [0, {V})")
        return ids

    def _private_cache(self, tokens: int) -> CacheContext:
        """The engine's own pool for `generate` and `forward_logits`, grown when a
        call needs more pages than it has."""
        pages = max(1, (tokens + self.block_size - 1) // self.block_size)
        c = self._own_cache
        if c is not None:
            for r in c.manager.live_requests():
                c.release(r)
            if min(c.manager.num_pages(g) for g in c.manager.groups) >= pages:
                return c
            self._own_cache = c = None          # drop the small pool before making the larger one
        self._own_cache = self.new_cache(pages, self.block_size, 1)
        return self._own_cache

    def forward_logits(self, ids: Sequence[int]) -> np.ndarray:
        """Logits at every position of a sequence, [T, vocab] float32."""
        ids = self._validate_ids(ids, "forward_logits")
        if not ids:
            raise ValueError("forward_logits: ids is empty")
        if len(ids) > self.max_pos:
            raise RuntimeError("forward_logits: sequence exceeds RoPE max_pos")
        with self._lock:
            cache = self._private_cache(len(ids))
            cache.admit("forward_logits")
            try:
                out = np.empty((len(ids), self.cfg.vocab_size), dtype=np.float32)
                for start in range(0, len(ids), self.prefill_chunk):
                    part = ids[start:start + self.prefill_chunk]
                    logits = self.step(cache, [StepEntry("forward_logits", part, list(range(len(part))))])
                    out[start:start + len(part)] = logits.cpu().numpy()
                return out
            finally:
                cache.release("forward_logits")

    # ---- generation (src/engine.cpp:718-774) ----
    def generate(self, prompt_ids: Sequence[int], max_new_tokens: int) -> tuple[list[int], str]:
        """Decodes up to max_new_tokens after the prompt, greedily unless the engine
        was given a temperature; stops at an EOS id, which is not appended. Returns
        (prompt + generated ids, "stop" | "length")."""
        if len(prompt_ids) == 0:
            raise ValueError("generate: prompt_ids is empty")
        if max_new_tokens < 0:
            raise ValueError("generate: max_new_tokens negative")
        ids = self._validate_ids(prompt_ids, "generate")
        if len(ids) + int(max_new_tokens) > self.max_pos:
            raise RuntimeError("generate: prompt + max_new_tokens exceeds RoPE max_pos")
        out = list(ids)
        if max_new_tokens == 0:
            return out, "length"
        eos = set(self.cfg.eos_token_ids)
        with self._lock:
            cache = self._private_cache(len(ids) + int(max_new_tokens))
            rid = "generate"
            cache.admit(rid)
            try:
                logits = None
                for start in range(0, len(ids), self.prefill_chunk):
                    part = ids[start:start + self.prefill_chunk]
                    last = start + len(part) == len(ids)
                    logits = self.step(cache, [StepEntry(rid, part, [len(part) - 1] if last else [])])
                finish = "length"
                generated = 0
                runner = self.runner
                recorded = runner.use_graphs      # decode steps are recorded launches that end in the choice
                temperature, seed = self.sampler.temperature, self.sampler.seed

                def draw(index: int):
                    return [uniform_draw(seed, 0, index)] if temperature > 0.0 else None
                pending = None
                while generated < max_new_tokens:
                    if pending is None:
                        nxt = self.sampler.choose(logits, [(0, generated)])[0]
                    else:
                        # the step behind this one is launched on the token the device holds before the
                        # host has fetched it (one step more than needed if this one stops)
                        more = generated + 1 < max_new_tokens     # the token being fetched is not the last wanted
                        with torch.cuda.device(runner.device):
                            ahead = runner.launch_choosing(cache, [rid], None, self.max_pos, temperature,
                                                         draw(generated + 1)) if more else None
                            nxt = runner.chosen_tokens(pending)[0]
                    if nxt in eos:
                        finish = "stop"
                        if pending is not None and ahead is not None:
                            runner.chosen_tokens(ahead)
                        break
                    out.append(nxt)
                    generated += 1
                    if generated >= max_new_tokens:
                        break
                    if recorded:
                        with torch.cuda.device(runner.device):
                            if pending is not None and ahead is not None:
                                pending = ahead
                            else:
                                pending = runner.launch_choosing(cache, [rid], [nxt], self.max_pos, temperature,
                                                               draw(generated))
                    else:
                        logits = self.step(cache, [StepEntry(rid, [nxt], [0])])
                return out, finish
            finally:
                cache.release(rid)
