"""Each part of a layer alone on the GPU against its plain formula, and the generality of
the composition: a schedule that names a layer twice and lets a layer read another layer's
cache, a windowed attention with pages given back, and toy parts that are defined here,
registered, built and stepped without a change to the framework: a mixer with state of its own,
a feed-forward with routing, another position encoding and another arrangement of a block."""
import math
from dataclasses import dataclass

import numpy as np
import pytest
import torch

import replay
from plain_llama import (plain_apply_rope, plain_attention, plain_forward, plain_inv_freq, plain_linear,
                         plain_mlp, plain_rmsnorm, plain_rope_tables)
from tiny_models import B_INIT, TINY_B, random_tokens

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _gen(s):
    return torch.Generator().manual_seed(s)


def _rel(a, b):
    a, b = torch.as_tensor(a).double().cpu(), torch.as_tensor(b).double().cpu()
    return float((a - b).abs().max() / b.abs().max())


def _placement(dtype=torch.float32):
    from llmengine.parts import Placement
    return Placement(DEV, dtype)


def _step(new_lens, ctx_lens, page, dtype=torch.float32, tables=None):
    """A StepContext made by hand: requests with ctx tokens cached and n new tokens each."""
    from llmengine.engine.step import StepContext, Workspace
    T, S = sum(new_lens), len(new_lens)
    i32 = dict(dtype=torch.int32, device=DEV)
    positions = torch.cat([torch.arange(c, c + n) for c, n in zip(ctx_lens, new_lens)]).to(**i32)
    seq_idx = torch.cat([torch.full((n,), s) for s, n in enumerate(new_lens)]).to(**i32)
    q_start = torch.tensor([0] + list(np.cumsum(new_lens)), **i32)
    max_blocks = max((c + n + page - 1) // page for c, n in zip(ctx_lens, new_lens))
    if tables is None:
        tables, p = [], 0
        for c, n in zip(ctx_lens, new_lens):
            nb = (c + n + page - 1) // page
            tables.append(list(range(p, p + nb)) + [0] * (max_blocks - nb))
            p += nb
    return StepContext(num_tokens=T, num_seqs=S, tokens=torch.zeros(T, **i32), positions=positions, seq_idx=seq_idx,
                       q_start=q_start, ctx_len=torch.tensor(ctx_lens, **i32), slots=torch.arange(S, **i32),
                       block_tables={"full": torch.tensor(tables, **i32)}, act_dtype=dtype, workspace=Workspace(DEV),
                       new_lens=list(new_lens), ctx_lens=list(ctx_lens), slot_list=list(range(S)),
                       max_position=max(c + n for c, n in zip(ctx_lens, new_lens)) - 1)


def test_rmsnorm_part():
    from llmengine.parts import RMSNorm
    w = 1 + 0.1 * torch.randn(96, generator=_gen(0))
    norm = RMSNorm(96, 1e-6)
    norm.load_tree(lambda n: {"weight": w}[n], _placement())
    x = torch.randn(7, 96, generator=_gen(1))
    out = torch.empty(7, 96, device=DEV)
    norm.forward(x.to(DEV), out)
    assert _rel(out, plain_rmsnorm(x.double(), w.double(), 1e-6)) < 2e-6


@pytest.mark.parametrize("hd,theta,scaling", [
    (32, 500000.0, {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                    "original_max_position_embeddings": 64}),
    (64, 500000.0, {"factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                    "original_max_position_embeddings": 8192}),
    (16, 10000.0, None)])
def test_rotary_tables(hd, theta, scaling):
    from llmengine.parts import RotaryEmbedding
    rope = RotaryEmbedding(hd, theta, 9000, scaling)
    rope.materialize(_placement())
    cos, sin, rot = rope.rotary_tables()
    assert rot == hd and cos.shape == (9000, hd // 2)
    sc = None if scaling is None else (scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"],
                                       scaling["original_max_position_embeddings"])
    inv = plain_inv_freq(hd, theta, sc)
    assert rope.inv_freq.tolist() == inv                                  # the same 32-bit values
    positions = [0, 1, 63, 100, 1000, 8000, 8999]                         # tests/test_real_smoke.py:107-137
    pc, ps = plain_rope_tables(inv, positions, hd)
    for r, p in enumerate(positions):
        tol = max(1e-6, 1e-7 * p)
        assert (cos[p].cpu().double() - pc[r, :hd // 2]).abs().max() <= tol
        assert (sin[p].cpu().double() - ps[r, :hd // 2]).abs().max() <= tol


def test_gated_mlp_part():
    from llmengine.parts import GatedMLP
    H, FF = 96, 176
    w = {"gate_proj.weight": 0.1 * torch.randn(FF, H, generator=_gen(2)),
         "up_proj.weight": 0.1 * torch.randn(FF, H, generator=_gen(3)),
         "down_proj.weight": 0.1 * torch.randn(H, FF, generator=_gen(4))}
    mlp = GatedMLP(H, FF)
    mlp.load_tree(lambda n: w[n], _placement())
    x = torch.randn(5, H, generator=_gen(5))
    base = torch.randn(5, H, generator=_gen(6))
    out = base.clone().to(DEV)
    mlp.forward(x.to(DEV), _step([5], [0], 16), out, accumulate=True)
    ref = base.double() + plain_mlp(x.double(), *(w[k].double() for k in w))
    assert _rel(out, ref) < 3e-6


def test_embedding_and_head_parts():
    from llmengine.parts import Embedding, OutputHead
    E = torch.randn(331, 48, generator=_gen(7))
    emb = Embedding(331, 48)
    emb.load_tree(lambda n: E, _placement())
    out = torch.empty(4, 48, device=DEV)
    toks = torch.tensor([0, 330, 7, 7], dtype=torch.int32, device=DEV)
    emb.forward(toks, out)
    assert torch.equal(out.cpu(), E[[0, 330, 7, 7]])
    head = OutputHead(331, 48, tied_to=emb)
    assert head.param_specs() == {} and head.weight.data_ptr() == emb.weight.data_ptr()
    logits = torch.empty(4, 331, device=DEV)
    head.forward(out, logits)
    assert _rel(logits, plain_linear(out.cpu().double(), E.double())) < 3e-6


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(4, 2, 16, 4), (3, 1, 32, 8), (6, 2, 48, 16)])
def test_attention_part_alone(n_q, n_kv, hd, page):
    """The mixer with its own pages: a first step caches 9 and 4 tokens, a second step brings
    portions of 6 and 1 tokens; the result equals whole-sequence attention at those positions."""
    from llmengine.parts import Attention, RotaryEmbedding
    from llmengine.parts.base import LayerCache
    H = 40
    rope = RotaryEmbedding(hd, 10000.0, 64)
    attn = Attention(H, n_q, n_kv, hd, position=rope)
    w = {f"{p}_proj.weight": 0.2 * torch.randn(o, i, generator=_gen(10 + k)) for k, (p, o, i) in
         enumerate([("q", n_q * hd, H), ("k", n_kv * hd, H), ("v", n_kv * hd, H), ("o", H, n_q * hd)])}
    attn.load_tree(lambda n: w[n], _placement())
    lens = [15, 5]
    xs = [torch.randn(n, H, generator=_gen(20 + i)) for i, n in enumerate(lens)]
    pages = 8
    cache = LayerCache(paged={"k": torch.zeros(pages, n_kv, page, hd, device=DEV),
                              "v": torch.zeros(pages, n_kv, hd, page, device=DEV)}, state={}, page_size=page,
                       group="full")
    nb = [(n + page - 1) // page for n in lens]
    tables = [[5, 2, 7, 0][:nb[0]] + [0] * (4 - nb[0]), [6, 1, 3, 4][:nb[1]] + [0] * (4 - nb[1])]
    tables = [t[:max(nb)] for t in tables]
    outs = []
    for new, ctx in (([9, 4], [0, 0]), ([6, 1], [9, 4])):
        x = torch.cat([xs[s][c:c + n] for s, (c, n) in enumerate(zip(ctx, new))])
        out = torch.zeros(sum(new), H, device=DEV)
        attn.forward(x.to(DEV), _step(new, ctx, page, tables=tables), cache, out, accumulate=False)
        outs.append(out.cpu())
    inv = plain_inv_freq(hd, 10000.0, None)
    for s, n in enumerate(lens):
        x = xs[s].double()
        cos, sin = plain_rope_tables(inv, range(n), hd)
        q = plain_apply_rope(plain_linear(x, w["q_proj.weight"].double()).view(n, n_q, hd), cos, sin)
        k = plain_apply_rope(plain_linear(x, w["k_proj.weight"].double()).view(n, n_kv, hd), cos, sin)
        v = plain_linear(x, w["v_proj.weight"].double()).view(n, n_kv, hd)
        ref = plain_linear(plain_attention(q, k, v).reshape(n, -1), w["o_proj.weight"].double())
        first = outs[0][:9] if s == 0 else outs[0][9:]
        second = outs[1][:6] if s == 0 else outs[1][6:]
        assert _rel(torch.cat([first, second]), ref) < 5e-6


# --- the order of layers is data --------------------------------------------------------
def _engine_with(model_builder, cfg_dict, tensors, dtype="fp32"):
    """An Engine over a model made by `model_builder`, registered under a test-only name."""
    from llmengine import Engine
    from llmengine.config import LlamaConfig, register_architecture
    name = cfg_dict["architectures"][0]
    register_architecture(name, LlamaConfig.from_dict, model_builder, replace=True)
    return Engine(None, dtype, _config=cfg_dict, _tensors=tensors, block_size=8)


def test_schedule_names_a_layer_twice_and_shares_a_cache():
    """Layers run in the order 0, 1, 0 (again, on a cache of its own), 2 reading layer 1's keys
    and values: a schedule, compared with the plain implementation given the same schedule."""
    from llmengine.models.llama import build_llama
    from llmengine.models.model import LayerCall
    from llmengine.weights import random_state
    cfg = dict(TINY_B, architectures=["ScheduledLlama"])
    calls = [LayerCall(0), LayerCall(1), LayerCall(0, cache=7), LayerCall(2, cache=1, write_cache=False)]

    def build(c):
        m = build_llama(c)
        m.schedule = calls
        return m
    tensors = dict(random_state(dict(TINY_B), 5, torch.float32, 0.05, 1.0, 0.1))
    engine = _engine_with(build, cfg, dict(tensors))
    assert sorted(engine.model.cache_specs()) == [0, 1, 7]
    reqs = {"a": random_tokens(37, 384, 1), "b": random_tokens(12, 384, 2)}
    sched = [(0, 0, True), (1, 1, True), (0, 7, True), (2, 1, False)]
    plain = {k: plain_forward(TINY_B, tensors, v, schedule=sched).numpy() for k, v in reqs.items()}
    for steps in (replay.whole(reqs), replay.portions(reqs), replay.mixed(reqs, 2)):
        cache = engine.new_cache(8, 8, 2)
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for p in range(len(ids)):
                assert _rel(got[rid][p], plain[rid][p]) < 1e-5, (rid, p)


def test_windowed_attention_gives_pages_back():
    """The same layers with a window of 11 tokens on every attention: a cache group of kind
    'window', whose pages return to the pool while the request is still running."""
    from llmengine.models.llama import llama_layer_specs
    from llmengine.models.model import DecoderModel
    from llmengine.parts import Embedding, LayerSpec, OutputHead, PartChoice, RMSNorm, build_layer
    from llmengine.weights import random_state
    cfg = dict(TINY_B, architectures=["WindowedLlama"])
    window = 11

    def build(c):
        shared = {}
        layers = []
        for spec in llama_layer_specs(c):
            mixer = PartChoice("attention", dict(spec.mixer.args, window=window))
            layers.append(build_layer(LayerSpec(spec.block, mixer, spec.feed_forward, spec.mixer_norm,
                                                spec.ffn_norm, spec.position), shared))
        emb = Embedding(c.vocab_size, c.hidden_size)
        return DecoderModel(c, emb, layers, RMSNorm(c.hidden_size, c.rms_norm_eps),
                            OutputHead(c.vocab_size, c.hidden_size))
    tensors = dict(random_state(dict(TINY_B), 6, torch.float32, 0.05, 1.0, 0.1))
    engine = _engine_with(build, cfg, dict(tensors))
    ids = random_tokens(90, 384, 9)
    ref = plain_forward(TINY_B, tensors, ids, window=window).numpy()
    assert not np.allclose(ref[-1], plain_forward(TINY_B, tensors, ids).numpy()[-1], atol=1e-4)
    for steps in (replay.whole({"w": ids}), replay.portions({"w": ids}), replay.tail_one_by_one({"w": ids}, 40)):
        cache = engine.new_cache(12, 8, 1)
        assert list(cache.manager.groups) == [f"window{window}"]
        got = replay.run_trace(engine, cache, steps)["w"]
        for p in range(len(ids)):
            assert _rel(got[p], ref[p]) < 1e-5, p
    # decoding 80 tokens one by one needs 3 pages of 8 at most (11 tokens never span more)
    cache = engine.new_cache(3, 8, 1)
    got = replay.run_trace(engine, cache, replay.tail_one_by_one({"w": ids[:80]}, 79))["w"]
    assert _rel(got[79], ref[79]) < 1e-5


# --- a toy mixer with state of its own ---------------------------------------------------
@pytest.mark.parametrize("recordable", [False, True], ids=["launched", "recorded"])
def test_a_toy_mixer_with_state_registers_builds_and_steps(recordable):
    """A mixer that keeps no pages but a running sum and a count per request:
    y_t = W mean(x_0..x_t). Layer 0 uses it, layer 1 is ordinary attention: different mixers in
    different layers of one model. Defined here, registered through the public registries.
    recorded: the mixer says that its steps of single tokens can be recorded as a graph (it then
    reads the slots from the step's device array). Its step advances the state, so it must run
    exactly once for a token: a recording that ran the step to try it would count tokens twice."""
    from llmengine import Engine
    from llmengine.config import register_architecture
    from llmengine.models.model import DecoderModel
    from llmengine.parts import (CacheSpec, Embedding, LayerSpec, Mixer, OutputHead, ParamSpec, PartChoice,
                                 RMSNorm, build_layer, register_part)
    from llmengine.weights import random_state

    class RunningMean(Mixer):
        graph_safe = recordable

        def __init__(self, hidden_size):
            self.hidden_size = hidden_size
            self.w = None

        def param_specs(self):
            return {"proj.weight": ParamSpec((self.hidden_size, self.hidden_size))}

        def load_params(self, get, placement):
            self.w = placement.place(get("proj.weight"), torch.float32)

        def cache_spec(self):
            return CacheSpec(state={"sum": ((self.hidden_size,), torch.float32), "count": ((1,), torch.float32)})

        def forward(self, x, step, cache, out, accumulate, write_cache=True):
            if recordable and step.num_tokens == step.num_seqs:
                # one token of every request: the same launches whatever the requests, nothing from host lists
                slots = step.slots.long()
                cache.state["sum"].index_add_(0, slots, x.float())
                cache.state["count"].index_add_(0, slots, torch.ones_like(x[:, :1], dtype=torch.float32))
                y = (cache.state["sum"][slots] / cache.state["count"][slots]) @ self.w.T
                if accumulate:
                    out.add_(y)
                else:
                    out.copy_(y)
                return
            row = 0
            for n, slot in zip(step.new_lens, step.slot_list):        # tokens of a request in order
                xs = x[row:row + n].float()
                total = cache.state["sum"][slot] + torch.cumsum(xs, dim=0)
                count = cache.state["count"][slot] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                y = (total / count[:, None]) @ self.w.T
                out[row:row + n] = out[row:row + n] + y if accumulate else y
                cache.state["sum"][slot] = total[-1]
                cache.state["count"][slot] = count[-1]
                row += n

    register_part("mixer", "running_mean", RunningMean, replace=True)

    @dataclass(frozen=True)
    class ToyConfig:
        hidden_size: int
        vocab_size: int
        max_pos: int
        eos_token_ids: tuple = ()

    def parse(cfg, gen=None, architecture=""):
        return ToyConfig(cfg["hidden_size"], cfg["vocab_size"], cfg["max_position_embeddings"])

    H, V, FF = 48, 101, 80

    def build(c):
        norm = PartChoice("rmsnorm", {"size": H, "eps": 1e-5})
        ffn = PartChoice("gated_mlp", {"hidden_size": H, "intermediate_size": FF})
        rope = PartChoice("rotary", {"rotary_dim": 16, "theta": 10000.0, "max_position": c.max_pos})
        toy = LayerSpec(PartChoice("prenorm", {"names": {"mixer": "mean_mixer"}}),
                        PartChoice("running_mean", {"hidden_size": H}), ffn, norm, norm)
        att = LayerSpec(PartChoice("prenorm"), PartChoice("attention", {
            "hidden_size": H, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16}), ffn, norm, norm, rope)
        emb = Embedding(V, H)
        return DecoderModel(c, emb, [build_layer(toy), build_layer(att)], RMSNorm(H, 1e-5),
                            OutputHead(V, H, tied_to=emb))

    register_architecture("ToyForCausalLM", parse, build, replace=True)
    cfg = {"architectures": ["ToyForCausalLM"], "hidden_size": H, "vocab_size": V, "max_position_embeddings": 200}
    tensors = dict(random_state(cfg, 11, torch.float32, 0.08, 1.0, 0.1))
    assert "model.layers.0.mean_mixer.proj.weight" in tensors and "model.layers.1.self_attn.q_proj.weight" in tensors
    engine = Engine(None, "fp32", _config=cfg, _tensors=dict(tensors), block_size=8)
    specs = engine.model.cache_specs()
    assert specs[0].state and not specs[0].paged and specs[1].paged
    assert engine.runner.use_graphs == recordable

    def plain_toy(ids):
        w = {k: v.double() for k, v in tensors.items()}
        n = len(ids)
        h = w["model.embed_tokens.weight"][ids]
        x = plain_rmsnorm(h, w["model.layers.0.input_layernorm.weight"], 1e-5)
        mean = torch.cumsum(x, 0) / torch.arange(1, n + 1, dtype=torch.float64)[:, None]
        h = h + mean @ w["model.layers.0.mean_mixer.proj.weight"].T
        p = "model.layers.0."
        h = h + plain_mlp(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], 1e-5),
                          w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        p = "model.layers.1."
        x = plain_rmsnorm(h, w[p + "input_layernorm.weight"], 1e-5)
        cos, sin = plain_rope_tables(plain_inv_freq(16, 10000.0, None), range(n), 16)
        q = plain_apply_rope(plain_linear(x, w[p + "self_attn.q_proj.weight"]).view(n, 3, 16), cos, sin)
        k = plain_apply_rope(plain_linear(x, w[p + "self_attn.k_proj.weight"]).view(n, 1, 16), cos, sin)
        v = plain_linear(x, w[p + "self_attn.v_proj.weight"]).view(n, 1, 16)
        h = h + plain_linear(plain_attention(q, k, v).reshape(n, -1), w[p + "self_attn.o_proj.weight"])
        h = h + plain_mlp(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], 1e-5),
                          w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return plain_linear(plain_rmsnorm(h, w["model.norm.weight"], 1e-5), w["model.embed_tokens.weight"]).numpy()

    reqs = {f"t{i}": random_tokens(n, V, 70 + i) for i, n in enumerate((31, 8, 50, 19, 2))}
    plain = {k: plain_toy(v) for k, v in reqs.items()}
    for steps in (replay.whole(reqs), replay.tail_one_by_one(reqs, 10), replay.portions(reqs),
                  replay.mixed(reqs, max_live=3, seed=4)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 8) // 8, 8, 3)   # slots are reused too
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for pos in range(len(ids)):
                assert _rel(got[rid][pos], plain[rid][pos]) < 1e-5, (rid, pos)
    assert (engine.runner.graph_replays > 40) == recordable
    out, finish = engine.generate(reqs["t1"], 5)
    assert finish == "length" and len(out) == 13


# --- a toy feed-forward with routing, another position encoding, another arrangement -------
def test_toy_routed_feed_forward_position_encoding_and_arrangement():
    """Three more kinds of part, defined here and registered through the public registries: a
    feed-forward that routes each token to one of E small experts, a rotary encoding over a part
    of the head with interpolated positions (p / stretch), and an arrangement in which mixer and
    feed-forward read the same normed input. Layer 0 uses all three, layer 1 is ordinary."""
    from llmengine import Engine
    from llmengine.config import register_architecture
    from llmengine.models.model import DecoderModel
    from llmengine.parts import (Block, Embedding, FeedForward, LayerSpec, OutputHead, ParamSpec, PartChoice,
                                 PositionEncoding, RMSNorm, build_layer, register_part)
    from llmengine.weights import random_state

    class Top1Experts(FeedForward):
        def __init__(self, hidden_size, expert_size, num_experts):
            self.h, self.f, self.e = hidden_size, expert_size, num_experts
            self.p = {}

        def param_specs(self):
            specs = {"router.weight": ParamSpec((self.e, self.h))}
            for e in range(self.e):
                specs[f"experts.{e}.up.weight"] = ParamSpec((self.f, self.h))
                specs[f"experts.{e}.down.weight"] = ParamSpec((self.h, self.f))
            return specs

        def load_params(self, get, placement):
            self.p = {name: placement.place(get(name), torch.float32) for name in self.param_specs()}

        def forward(self, x, step, out, accumulate):
            xs = x.float()
            prob = torch.softmax(xs @ self.p["router.weight"].T, dim=-1)
            weight, choice = prob.max(dim=-1)
            y = torch.zeros_like(xs)
            for e in range(self.e):
                rows = (choice == e).nonzero().flatten()
                if rows.numel():
                    hid = torch.relu(xs[rows] @ self.p[f"experts.{e}.up.weight"].T)
                    y[rows] = weight[rows, None] * (hid @ self.p[f"experts.{e}.down.weight"].T)
            if accumulate:
                out += y
            else:
                out.copy_(y)

    class StretchedRotary(PositionEncoding):
        def __init__(self, rotary_dim, theta, stretch, max_position):
            self.rotary_dim, self.theta, self.stretch, self._max = rotary_dim, theta, stretch, max_position
            self.cos = self.sin = None

        @property
        def max_position(self):
            return self._max

        def materialize(self, placement):
            i = torch.arange(self.rotary_dim // 2, dtype=torch.float64)
            freq = self.theta ** (-2.0 * i / self.rotary_dim)
            angle = (torch.arange(self._max, dtype=torch.float64) / self.stretch)[:, None] * freq[None, :]
            self.cos = torch.cos(angle).float().to(placement.device).contiguous()
            self.sin = torch.sin(angle).float().to(placement.device).contiguous()

        def rotary_tables(self):
            return self.cos, self.sin, self.rotary_dim

    class ParallelBlock(Block):
        """h += mixer(norm(h)) + feed_forward(norm(h)): one norm, both read it."""

        def __init__(self, mixer, feed_forward, mixer_norm, ffn_norm):
            self.mixer, self.feed_forward, self.norm = mixer, feed_forward, mixer_norm

        def children(self):
            return {"norm": self.norm, "attn": self.mixer, "moe": self.feed_forward}

        def forward(self, h, step, cache, write_cache=True):
            x = step.buffer("parallel.normed", tuple(h.shape), step.act_dtype)
            self.norm.forward(h, x)
            self.mixer.forward(x, step, cache, h, True, write_cache)
            self.feed_forward.forward(x, step, h, True)

    register_part("feed_forward", "top1_experts", Top1Experts, replace=True)
    register_part("position", "stretched_rotary", StretchedRotary, replace=True)
    register_part("block", "parallel", ParallelBlock, replace=True)

    @dataclass(frozen=True)
    class ToyConfig:
        max_pos: int
        eos_token_ids: tuple = ()

    H, V, FF, E, EF, HD, ROT, NQ, NKV = 40, 77, 56, 3, 24, 16, 8, 2, 2
    THETA, STRETCH, EPS = 100.0, 2.5, 1e-4

    def build(c):
        norm = PartChoice("rmsnorm", {"size": H, "eps": EPS})
        att = PartChoice("attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV, "head_dim": HD})
        first = LayerSpec(PartChoice("parallel"), att,
                          PartChoice("top1_experts", {"hidden_size": H, "expert_size": EF, "num_experts": E}),
                          norm, norm, PartChoice("stretched_rotary", {"rotary_dim": ROT, "theta": THETA,
                                                                      "stretch": STRETCH, "max_position": c.max_pos}))
        second = LayerSpec(PartChoice("prenorm"), att,
                           PartChoice("gated_mlp", {"hidden_size": H, "intermediate_size": FF}), norm, norm,
                           PartChoice("rotary", {"rotary_dim": HD, "theta": THETA, "max_position": c.max_pos}))
        emb = Embedding(V, H)
        return DecoderModel(c, emb, [build_layer(first), build_layer(second)], RMSNorm(H, EPS),
                            OutputHead(V, H, tied_to=emb))

    register_architecture("ToyRoutedForCausalLM", lambda cfg, gen=None, architecture="":
                          ToyConfig(cfg["max_position_embeddings"]), build, replace=True)
    cfg = {"architectures": ["ToyRoutedForCausalLM"], "max_position_embeddings": 128}
    tensors = dict(random_state(cfg, 23, torch.float32, 0.2, 1.0, 0.1))
    assert "model.layers.0.moe.experts.2.down.weight" in tensors and "model.layers.0.norm.weight" in tensors
    assert "model.layers.0.post_attention_layernorm.weight" not in tensors
    engine = Engine(None, "fp32", _config=cfg, _tensors=dict(tensors), block_size=8)

    def plain_attn(x, w, p, cos, sin, rot):
        n = x.shape[0]
        q = plain_linear(x, w[p + "q_proj.weight"]).view(n, NQ, HD).clone()
        k = plain_linear(x, w[p + "k_proj.weight"]).view(n, NKV, HD).clone()
        v = plain_linear(x, w[p + "v_proj.weight"]).view(n, NKV, HD)
        q[..., :rot] = plain_apply_rope(q[..., :rot], cos, sin)          # the rest of a head is not rotated
        k[..., :rot] = plain_apply_rope(k[..., :rot], cos, sin)
        return plain_linear(plain_attention(q, k, v).reshape(n, -1), w[p + "o_proj.weight"])

    used = set()

    def plain_toy(ids):
        w = {k: v.double() for k, v in tensors.items()}
        n = len(ids)
        h = w["model.embed_tokens.weight"][ids]
        p = "model.layers.0."
        x = plain_rmsnorm(h, w[p + "norm.weight"], EPS)
        freq = [THETA ** (-2.0 * i / ROT) for i in range(ROT // 2)]
        cos, sin = plain_rope_tables(freq, [t / STRETCH for t in range(n)], ROT)
        mixed = plain_attn(x, w, p + "attn.", cos, sin, ROT)
        routed = torch.zeros_like(h)
        for t in range(n):
            logits = plain_linear(x[t:t + 1], w[p + "moe.router.weight"])[0]
            prob = torch.exp(logits - logits.max())
            prob = prob / prob.sum()
            e = int(prob.argmax())
            used.add(e)
            hid = torch.clamp(plain_linear(x[t:t + 1], w[p + f"moe.experts.{e}.up.weight"]), min=0.0)
            routed[t] = prob[e] * plain_linear(hid, w[p + f"moe.experts.{e}.down.weight"])[0]
        h = h + mixed + routed
        p = "model.layers.1."
        cos, sin = plain_rope_tables(plain_inv_freq(HD, THETA, None), range(n), HD)
        h = h + plain_attn(plain_rmsnorm(h, w[p + "input_layernorm.weight"], EPS), w, p + "self_attn.", cos, sin, HD)
        h = h + plain_mlp(plain_rmsnorm(h, w[p + "post_attention_layernorm.weight"], EPS),
                          w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
        return plain_linear(plain_rmsnorm(h, w["model.norm.weight"], EPS), w["model.embed_tokens.weight"]).numpy()

    reqs = {f"m{i}": random_tokens(n, V, 90 + i) for i, n in enumerate((45, 9, 33, 70))}
    plain = {k: plain_toy(v) for k, v in reqs.items()}
    assert used == set(range(E))                                         # every expert took some token
    for steps in (replay.whole(reqs), replay.tail_one_by_one(reqs, 12), replay.portions(reqs),
                  replay.mixed(reqs, max_live=3, seed=9)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 8) // 8, 8, 3)
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for pos in range(len(ids)):
                assert _rel(got[rid][pos], plain[rid][pos]) < 1e-5, (rid, pos)


# --- an encoding that is no table of angles, a norm with another formula, pages of another type ---
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_toy_interleaved_encoding_shifted_norm_and_wide_pages(dtype):
    """Three parts that the Llama kernels' shortcuts must not swallow, defined here and registered:
    a rotation of neighbouring pairs (2i, 2i + 1) that transforms q and k itself (`apply`, no rotary
    tables); a norm y = (1 + w) x / sqrt(mean(x^2) + eps) that subclasses RMSNorm, which the decode
    kernels must not fuse with the Llama formula; an attention that keeps its keys and values in
    32-bit pages inside a bfloat16 model."""
    from llmengine import Engine
    from llmengine.config import register_architecture
    from llmengine.models.model import DecoderModel
    from llmengine.parts import (Attention, CacheSpec, Embedding, LayerSpec, OutputHead, PartChoice, PositionEncoding,
                                 RMSNorm, build_layer, register_part)
    from llmengine.parts.base import PAGE
    from llmengine.weights import random_state

    class InterleavedRotary(PositionEncoding):
        def __init__(self, head_dim, theta, max_position):
            self.hd, self.theta, self._max = head_dim, theta, max_position
            self.freq = None

        @property
        def max_position(self):
            return self._max

        def materialize(self, placement):
            i = torch.arange(self.hd // 2, dtype=torch.float64)
            self.freq = (self.theta ** (-2.0 * i / self.hd)).float().to(placement.device)

        def apply(self, q, k, positions):
            angle = positions.float()[:, None] * self.freq[None, :]                # [T, hd / 2]
            cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
            for x in (q, k):
                if x is None:
                    continue
                a, b = x[..., 0::2].clone(), x[..., 1::2].clone()
                x[..., 0::2] = a * cos - b * sin
                x[..., 1::2] = b * cos + a * sin

    class ShiftedRMSNorm(RMSNorm):
        def forward(self, x, out, rows=None):
            src = x if rows is None else x[rows.long()]
            y = (1.0 + self.weight.float()) * src / torch.sqrt((src * src).mean(-1, keepdim=True) + self.eps)
            out.copy_(y)

    class WidePagesAttention(Attention):
        def cache_spec(self):
            return CacheSpec(paged={"k": ((self.num_kv_heads, PAGE, self.head_dim), torch.float32),
                                    "v": ((self.num_kv_heads, self.head_dim, PAGE), torch.float32)})

    register_part("position", "interleaved_rotary", InterleavedRotary, replace=True)
    register_part("norm", "shifted_rmsnorm", ShiftedRMSNorm, replace=True)
    register_part("mixer", "wide_pages_attention", WidePagesAttention, replace=True)

    @dataclass(frozen=True)
    class ToyConfig:
        max_pos: int
        eos_token_ids: tuple = ()

    H, V, FF, HD, NQ, NKV, THETA, EPS = 64, 90, 96, 16, 4, 2, 50.0, 1e-5

    def build(c):
        norm = PartChoice("shifted_rmsnorm", {"size": H, "eps": EPS})
        layer = LayerSpec(PartChoice("prenorm"),
                          PartChoice("wide_pages_attention", {"hidden_size": H, "num_heads": NQ, "num_kv_heads": NKV,
                                                              "head_dim": HD}),
                          PartChoice("gated_mlp", {"hidden_size": H, "intermediate_size": FF}), norm, norm,
                          PartChoice("interleaved_rotary", {"head_dim": HD, "theta": THETA, "max_position": c.max_pos}))
        emb = Embedding(V, H)
        return DecoderModel(c, emb, [build_layer(layer), build_layer(layer)], ShiftedRMSNorm(H, EPS),
                            OutputHead(V, H, tied_to=emb))

    register_architecture("ToyInterleavedForCausalLM", lambda cfg, gen=None, architecture="":
                          ToyConfig(cfg["max_position_embeddings"]), build, replace=True)
    cfg = {"architectures": ["ToyInterleavedForCausalLM"], "max_position_embeddings": 128}
    store = torch.float32 if dtype == "fp32" else torch.bfloat16
    tensors = dict(random_state(cfg, 31, store, 0.1, 0.0, 0.3))                    # norm weights around 0: 1 + w matters
    engine = Engine(None, dtype, _config=cfg, _tensors=dict(tensors), block_size=16)
    model = engine.model
    assert model.layers[0].mixer_norm.fused_rms() is None and RMSNorm(H, EPS).fused_rms() is not None
    assert not engine.runner.use_graphs                                            # the encoding computes in `apply`

    rnd = (lambda t: t.float().bfloat16().double()) if dtype == "bf16" else (lambda t: t)

    def norm(x, w):
        return rnd((1.0 + w) * x / torch.sqrt((x * x).mean(-1, keepdim=True) + EPS))

    def rotate(x, n):
        angle = torch.arange(n, dtype=torch.float64)[:, None] * (THETA ** (-2.0 * torch.arange(HD // 2, dtype=torch.float64) / HD))
        cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
        out = torch.empty_like(x)
        out[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
        out[..., 1::2] = x[..., 1::2] * cos + x[..., 0::2] * sin
        return out

    def plain_toy(ids):
        w = {k: v.double() for k, v in tensors.items()}
        n = len(ids)
        h = w["model.embed_tokens.weight"][ids]
        for layer in range(2):
            p = f"model.layers.{layer}."
            x = norm(h, w[p + "input_layernorm.weight"])
            q = rnd(rotate(plain_linear(x, w[p + "self_attn.q_proj.weight"]).view(n, NQ, HD), n))
            k = rotate(plain_linear(x, w[p + "self_attn.k_proj.weight"]).view(n, NKV, HD), n)     # 32-bit pages: not rounded
            v = plain_linear(x, w[p + "self_attn.v_proj.weight"]).view(n, NKV, HD)
            h = h + plain_linear(rnd(plain_attention(q, k, v)).reshape(n, -1), w[p + "self_attn.o_proj.weight"])
            h = h + plain_mlp(norm(h, w[p + "post_attention_layernorm.weight"]), w[p + "mlp.gate_proj.weight"],
                              w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"],
                              rnd if dtype == "bf16" else None)
        return plain_linear(norm(h, w["model.norm.weight"]), w["model.embed_tokens.weight"]).numpy()

    reqs = {f"i{i}": random_tokens(n, V, 120 + i) for i, n in enumerate((40, 7, 66, 21))}
    plain = {k: plain_toy(v) for k, v in reqs.items()}
    tol = 1e-5 if dtype == "fp32" else 2e-2
    for steps in (replay.whole(reqs), replay.tail_one_by_one(reqs, 32), replay.portions(reqs),
                  replay.mixed(reqs, max_live=3, seed=2)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 16) // 16, 16, 3)
        assert cache.storage.layers[0].paged["k"].dtype == torch.float32
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for pos in range(len(ids)):
                assert _rel(got[rid][pos], plain[rid][pos]) < tol, (rid, pos)


# --- an embedding with a multiplier and a head with a cap, through the registries' own kinds ---
@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
def test_toy_scaled_embedding_and_capped_head(dtype):
    """The two ends of a model are parts like the others: an embedding that multiplies its rows by
    sqrt(hidden) and a head that caps its logits (cap tanh(z / cap)), defined here against the base
    classes `TokenEmbedding` and `Head`, registered under the kinds "embedding" and "head", built
    into an architecture of their own beside ordinary Llama layers, and stepped under all schedules,
    decode steps recorded. The plain forward gets the multiplier in its table and the cap behind."""
    from llmengine import Engine
    from llmengine.config import register_architecture
    from llmengine.config.llama import LlamaConfig
    from llmengine.models.llama import llama_layer_specs
    from llmengine.models.model import DecoderModel
    from llmengine.parts import ParamSpec, build_layer, make_part, register_part
    from llmengine.parts.base import Head, TokenEmbedding
    from llmengine.weights import random_state
    from plain_llama import bf16_round

    CAP = 3.0

    class ScaledEmbedding(TokenEmbedding):
        graph_safe = True                                   # reads the step's device arrays only

        def __init__(self, vocab_size, hidden_size, multiplier):
            self.vocab_size, self.hidden_size, self.multiplier = vocab_size, hidden_size, multiplier
            self.weight = None

        def param_specs(self):
            return {"weight": ParamSpec((self.vocab_size, self.hidden_size), "linear")}

        def load_params(self, get, placement):
            self.weight = placement.place(get("weight"))

        def forward(self, tokens, out, step=None):
            out.copy_(self.weight[tokens.long()].float() * self.multiplier)

    class CappedHead(Head):
        graph_safe = True

        def __init__(self, vocab_size, hidden_size, cap):
            self.vocab_size, self.hidden_size, self.cap = vocab_size, hidden_size, cap
            self.w = None

        def param_specs(self):
            return {"weight": ParamSpec((self.vocab_size, self.hidden_size), "linear")}

        def load_params(self, get, placement):
            self.w = placement.place(get("weight"), torch.float32)

        def forward(self, x, out, step=None):
            out.copy_(self.cap * torch.tanh((x.float() @ self.w.T) / self.cap))

    register_part("embedding", "toy_scaled", ScaledEmbedding, replace=True)
    register_part("head", "toy_capped", CappedHead, replace=True)

    def build(c):
        shared = {}
        layers = [build_layer(spec, shared) for spec in llama_layer_specs(c)]
        emb = make_part("embedding", "toy_scaled", vocab_size=c.vocab_size, hidden_size=c.hidden_size,
                        multiplier=math.sqrt(c.hidden_size))
        head = make_part("head", "toy_capped", vocab_size=c.vocab_size, hidden_size=c.hidden_size, cap=CAP)
        return DecoderModel(c, emb, layers, make_part("norm", "rmsnorm", size=c.hidden_size, eps=c.rms_norm_eps), head)

    register_architecture("ToyCappedForCausalLM", LlamaConfig.from_dict, build, replace=True)
    cfg = dict(TINY_B, architectures=["ToyCappedForCausalLM"])
    store = torch.float32 if dtype == "fp32" else torch.bfloat16
    tensors = dict(random_state(cfg, 41, store, 0.05, 1.0, 0.1))
    assert "lm_head.weight" in tensors and "model.embed_tokens.weight" in tensors
    engine = Engine(None, dtype, _config=cfg, _tensors=dict(tensors), block_size=8)
    assert engine.runner.use_graphs and not engine.model.head.fuses_norm(None, None, 1, None)

    as_llama = {k: v.double() for k, v in tensors.items()}
    as_llama["model.embed_tokens.weight"] = as_llama["model.embed_tokens.weight"] * math.sqrt(cfg["hidden_size"])
    reqs = {f"c{i}": random_tokens(n, cfg["vocab_size"], 200 + i) for i, n in enumerate((40, 7, 66, 21))}
    plain = {}
    for rid, ids in reqs.items():
        z = plain_forward(TINY_B, as_llama, ids, rounder=bf16_round if dtype == "bf16" else None)
        plain[rid] = (CAP * torch.tanh(z / CAP)).numpy()
    assert max(float(np.abs(v).max()) for v in plain.values()) > 0.5 * CAP          # the cap bends something
    tol = 1e-5 if dtype == "fp32" else 2e-2
    for steps in (replay.whole(reqs), replay.tail_one_by_one(reqs, 32), replay.portions(reqs),
                  replay.mixed(reqs, max_live=3, seed=6)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, 8) // 8, 8, 3)
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for pos in range(len(ids)):
                assert _rel(got[rid][pos], plain[rid][pos]) < tol, (rid, pos)
    assert engine.runner.graph_replays > 0
    # greedy generation through the entry point takes the recorded steps that end in the argmax
    ids, finish = engine.generate(reqs["c1"], 6)
    z = plain_forward(TINY_B, as_llama, ids[:-1], rounder=bf16_round if dtype == "bf16" else None)[-1]
    assert finish == "length" and z[ids[-1]] >= z.max() - (1e-5 if dtype == "fp32" else 2e-2) * z.abs().max()
