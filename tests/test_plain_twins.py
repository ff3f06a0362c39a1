"""The plain C++ twins of the device kernels (csrc/host/plain_kernels.cpp) against the plain
Python implementation of this folder: two independent readings of the reference's formulas,
one serial 32-bit C++ loop nest and one 64-bit tensor expression per operation, have to agree
to 32-bit rounding; so have the whole model put together from each (csrc/host/plain_model.cpp, the
plain backend, against plain_forward). Sizes are the reference's own test sizes and some that are no power of
two. The GPU half holds device kernels against the twins."""
import math

import pytest
import torch

from llmengine.runtime import plain as twin
from plain_llama import (plain_apply_rope, plain_argmax, plain_attention, plain_embed, plain_inv_freq,
                         plain_linear_by_rows, plain_rmsnorm, plain_rope_tables, plain_sample_bounds, plain_silu)

D = torch.float64
DEV = "cuda:0"


def _gen(s):
    return torch.Generator().manual_seed(s)


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


def test_embed_rows_are_copies():
    table = torch.randn(128, 24, generator=_gen(0))
    tokens = [0, 1, 7, 64, 127]                                   # the reference's ids (tests/test_kernels.py:66-71)
    assert torch.equal(twin.embed(table, tokens), plain_embed(table, tokens))
    with pytest.raises(ValueError):
        twin.embed(table, [128])


@pytest.mark.parametrize("dim", [16, 64, 128, 257])               # tests/test_kernels.py:26
def test_rmsnorm(dim):
    x = 3 * torch.randn(4, dim, generator=_gen(1))
    w = 1 + 0.1 * torch.randn(dim, generator=_gen(2))
    assert _rel(twin.rmsnorm(x, w, 1e-6), plain_rmsnorm(x.to(D), w.to(D), 1e-6)) < 2e-6
    assert _rel(twin.rmsnorm(x, 2 * w, 1e-5), 2 * plain_rmsnorm(x.to(D), w.to(D), 1e-5)) < 2e-6   # w, not 1 + w


@pytest.mark.parametrize("M,N,K", [(1, 8, 16), (1, 128, 128), (4, 64, 32), (3, 50, 176)])
def test_linear(M, N, K):
    a, w = torch.randn(M, K, generator=_gen(3)), torch.randn(N, K, generator=_gen(4))
    ref = plain_linear_by_rows(a.to(D), w.to(D))
    assert _rel(twin.linear(a, w), ref) < 2e-6
    base = torch.randn(M, N, generator=_gen(5))
    assert _rel(twin.linear(a, w, into=base), ref + base.to(D)) < 2e-6
    with pytest.raises(ValueError):
        twin.linear(a, torch.randn(N, K + 1))                      # a transposed weight is refused by its shape


@pytest.mark.parametrize("n", [1, 16, 384])                        # tests/test_kernels.py:40-47
def test_swiglu(n):
    g, u = 3 * torch.randn(n, generator=_gen(6)), torch.randn(n, generator=_gen(7))
    assert (twin.swiglu(g, u).to(D) - plain_silu(g.to(D)) * u.to(D)).abs().max() < 1e-6
    assert torch.all(twin.swiglu(torch.zeros(n), u) == 0)


@pytest.mark.parametrize("hd,theta,scaling", [(16, 10000.0, None), (32, 500000.0, (32.0, 1.0, 4.0, 64)),
                                              (64, 500000.0, (32.0, 1.0, 4.0, 8192)), (128, 500000.0, (8.0, 1.0, 4.0, 8192))])
def test_inv_freq_and_tables(hd, theta, scaling):
    inv = twin.inv_freq(hd, theta, scaling)
    ref = plain_inv_freq(hd, theta, scaling)
    for a, b in zip(inv.tolist(), ref):
        assert abs(a - b) <= 1.2e-7 * abs(b)                       # one 32-bit rounding at most
    positions = [0, 1, 5, 15, 100, 1000, 8000]                     # tests/test_kernels.py:131, tests/test_real_smoke.py:107-137
    cos, sin = twin.rope_tables(inv, positions, hd)
    rc, rs = plain_rope_tables(inv.tolist(), positions, hd)
    assert torch.equal(cos, rc.float()) and torch.equal(sin, rs.float())
    assert torch.equal(cos[:, :hd // 2], cos[:, hd // 2:])


def test_rope_apply_pairs_and_sign():
    hd, heads = 32, 3
    inv = twin.inv_freq(hd, 500000.0, (32.0, 1.0, 4.0, 64))
    positions = [0, 1, 5, 70]
    cos, sin = twin.rope_tables(inv, positions, hd)
    x = torch.randn(len(positions), heads, hd, generator=_gen(8))
    got = twin.rope_apply(x, cos, sin)
    assert _rel(got, plain_apply_rope(x.to(D), cos.to(D), sin.to(D))) < 1e-6
    assert torch.equal(got[0], x[0])                               # position 0 is the identity
    assert torch.allclose(got.pow(2).sum(-1), x.pow(2).sum(-1), rtol=1e-5)


@pytest.mark.parametrize("n_q,n_kv,hd,T", [(4, 2, 32, 1), (4, 2, 32, 7), (8, 2, 16, 13), (3, 1, 48, 9)])   # tests/test_kernels.py:194-227
def test_attention(n_q, n_kv, hd, T):
    q = torch.randn(T, n_q, hd, generator=_gen(9))
    k = torch.randn(T, n_kv, hd, generator=_gen(10))
    v = torch.randn(T, n_kv, hd, generator=_gen(11))
    ref = plain_attention(q.to(D), k.to(D), v.to(D))
    assert (twin.attention(q, k, v).to(D) - ref).abs().max() < 1e-5
    # the last rows alone, with the earlier keys as context
    if T > 2:
        assert (twin.attention(q[-2:], k, v).to(D) - ref[-2:]).abs().max() < 1e-5
        w = plain_attention(q.to(D), k.to(D), v.to(D), window=3)
        assert (twin.attention(q, k, v, window=3).to(D) - w).abs().max() < 1e-5


def test_argmax_and_sample():
    row = torch.randn(331, generator=_gen(12))
    row[100] = row[300] = 9.0
    assert twin.argmax(row) == plain_argmax(row) == 100
    cum = plain_sample_bounds(row, 0.8)
    for u in [0.0, 0.1, 0.5, 0.9, 0.999999]:
        tok = twin.sample(row, 0.8, u)
        lo = cum[tok - 1].item() if tok > 0 else 0.0
        assert lo - 1e-9 <= u <= cum[tok].item() + 1e-9


# --- device kernels against the twins --------------------------------------------------------
@pytest.fixture(scope="module")
def ops():
    from llmengine import ops
    ops.library()
    return ops


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_device_norm_linear_swiglu_against_twins(ops, dtype):
    T, H, N = 6, 200, 88
    tol = 2e-6 if dtype == torch.float32 else 8e-3
    x = 2 * torch.randn(T, H, generator=_gen(20))
    w = (1 + 0.1 * torch.randn(H, generator=_gen(21))).to(dtype)
    normed = torch.empty(T, H, dtype=dtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-5, normed)
    assert _rel(normed.cpu().float(), twin.rmsnorm(x, w.float(), 1e-5)) < tol
    a = normed.cpu()
    m = (0.05 * torch.randn(N, H, generator=_gen(22))).to(dtype)
    out = torch.empty(T, N, dtype=torch.float32, device=DEV)
    ops.gemm(a.to(DEV), m.to(DEV), out)
    assert _rel(out.cpu(), twin.linear(a.float(), m.float())) < (2e-6 if dtype == torch.float32 else 1e-5)
    g, u = 3 * torch.randn(T, 48, generator=_gen(23)), torch.randn(T, 48, generator=_gen(24))
    gu = torch.empty(T, 96)
    gu.view(T, 3, 2, 16)[:, :, 0], gu.view(T, 3, 2, 16)[:, :, 1] = g.view(T, 3, 16), u.view(T, 3, 16)
    act = torch.empty(T, 48, dtype=torch.float32, device=DEV)
    ops.swiglu(gu.to(DEV), act, 16)
    assert (act.cpu() - twin.swiglu(g, u)).abs().max() < 1e-5


@pytest.mark.gpu
def test_device_argmax_and_sample_against_twins(ops):
    V, R = 1000, 16
    logits = 2 * torch.randn(R, V, generator=_gen(25))
    logits[3, 10] = logits[3, 900] = 30.0
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert out.tolist() == [twin.argmax(r) for r in logits]
    u = torch.rand(R, generator=_gen(26))
    ops.sample(logits.to(DEV), torch.full((R,), 0.7, device=DEV), u.to(DEV), out)
    for r in range(R):
        # the device sums in 32-bit: its token is the twin's for a draw within rounding of u
        near = {twin.sample(logits[r], 0.7, min(max(u[r].item() + d, 0.0), 0.9999999)) for d in (-2e-5, 0.0, 2e-5)}
        assert out[r].item() in near or min(near) <= out[r].item() <= max(near)


def _tiny(name):
    import tiny_models
    from llmengine.config.registry import parse_config
    from llmengine.weights import random_state
    cfg, init = getattr(tiny_models, f"TINY_{name}"), getattr(tiny_models, f"{name}_INIT")
    tensors = dict(random_state(cfg, init["seed"], torch.float32, init["std"], init["norm_mean"], init["norm_std"]))
    return cfg, parse_config(cfg), tensors


@pytest.mark.parametrize("name,T", [("A", 40), ("B", 70), ("D", 33), ("E", 25), ("F", 30)])
def test_whole_model_backend_against_plain_forward(name, T):
    """The plain C++ backend (all layers, whole sequence, 32-bit) and the plain Python forward in
    64-bit agree to 32-bit rounding at every position; a shift of all positions moves both alike
    (B and F blend rope bands, so a shift is no identity there)."""
    from plain_llama import plain_forward
    from tiny_models import random_tokens
    cfg, typed, tensors = _tiny(name)
    tokens = random_tokens(T, cfg["vocab_size"], 77)
    got = twin.llama_forward(typed, tensors, tokens)
    ref = plain_forward(cfg, tensors, tokens)
    rows = (got.double() - ref).abs().amax(dim=1) / ref.abs().amax(dim=1)
    assert float(rows.max()) < 5e-6, (name, float(rows.max()))
    shifted = list(range(9, 9 + T))
    got_s = twin.llama_forward(typed, tensors, tokens, positions=shifted)
    ref_s = plain_forward(cfg, tensors, tokens, positions=shifted)
    assert float(((got_s.double() - ref_s).abs().amax(dim=1) / ref_s.abs().amax(dim=1)).max()) < 5e-6


def test_whole_model_backend_window_and_refusals():
    from plain_llama import plain_forward
    from tiny_models import random_tokens
    cfg, typed, tensors = _tiny("A")
    tokens = random_tokens(30, 256, 5)
    got = twin.llama_forward(typed, tensors, tokens, window=7)
    ref = plain_forward(cfg, tensors, tokens, window=7)
    assert float(((got.double() - ref).abs().amax(dim=1) / ref.abs().amax(dim=1)).max()) < 5e-6
    assert float((got.double() - plain_forward(cfg, tensors, tokens)).abs().max()) > 1e-4       # the window matters
    with pytest.raises(ValueError):
        twin.llama_forward(typed, tensors, tokens + [256])                                       # an id out of range
    with pytest.raises(ValueError):
        twin.llama_forward(typed, tensors, tokens, positions=[0, 1])
    with pytest.raises(KeyError):
        twin.llama_forward(typed, {k: v for k, v in tensors.items() if "layers.1.mlp.up_proj" not in k}, tokens)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["A", "B", "F"])
def test_device_32_bit_path_against_the_whole_model_backend(name):
    """The engine's 32-bit path (pages, steps of changing size, its own kernels) against the plain
    C++ backend's whole sequences: 1e-5 of a row's largest logit, the same greedy tokens."""
    import replay
    from llmengine import Engine
    from tiny_models import random_tokens
    cfg, typed, tensors = _tiny(name)
    reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 40 + i) for i, n in enumerate((45, 70, 9))}
    ref = {rid: twin.llama_forward(typed, tensors, ids) for rid, ids in reqs.items()}
    engine = Engine(None, "fp32", _config=cfg, _tensors=dict(tensors), block_size=16)
    for steps in (replay.whole(reqs), replay.portions(reqs), replay.mixed(reqs, max_live=2, seed=4)):
        cache = engine.new_cache(replay.trace_peak_tokens(steps, round_to=16) // 16, 16, max_requests=3)
        got = replay.run_trace(engine, cache, steps)
        for rid, ids in reqs.items():
            for p in range(len(ids)):
                row, want = torch.as_tensor(got[rid][p]).double(), ref[rid][p].double()
                assert float((row - want).abs().max() / want.abs().max()) < 1e-5, (name, rid, p)
                assert int(row.argmax()) == int(want.argmax()) or float(want.max() - want[int(row.argmax())]) < 1e-5 * float(want.abs().max())


@pytest.mark.gpu
@pytest.mark.parametrize("n_q,n_kv,hd,page,lens,window", [(4, 2, 32, 4, [7, 1], 0), (3, 1, 48, 16, [33, 17], 0),
                                                          (6, 3, 80, 8, [40], 5)])
def test_device_rotation_cache_write_and_attention_against_twins(ops, n_q, n_kv, hd, page, lens, window):
    """32-bit: rotate and write whole requests into pages (in reversed page order), attend over
    the pages with the plain-precision kernel, and hold both against the twins."""
    T, S = sum(lens), len(lens)
    qkv = torch.randn(T, (n_q + 2 * n_kv) * hd, generator=_gen(30))
    inv = twin.inv_freq(hd, 500000.0, (32.0, 1.0, 4.0, 64))
    cos_all, sin_all = twin.rope_tables(inv, list(range(max(lens))), hd)
    nblk = [(n + page - 1) // page for n in lens]
    pages = list(reversed(range(sum(nblk))))
    table = torch.zeros(S, max(nblk), dtype=torch.int32)
    for s in range(S):
        for b in range(nblk[s]):
            table[s, b] = pages.pop()
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    seq_idx = torch.cat([torch.full((n,), s) for s, n in enumerate(lens)]).to(torch.int32)
    k_cache = torch.zeros(sum(nblk), n_kv, page, hd, device=DEV)
    v_cache = torch.zeros(sum(nblk), n_kv, hd, page, device=DEV)
    q_rot = torch.empty(T, n_q * hd, device=DEV)
    ops.rope_kv_write(qkv.to(DEV), cos_all[:, :hd // 2].contiguous().to(DEV), sin_all[:, :hd // 2].contiguous().to(DEV),
                      positions.to(DEV), seq_idx.to(DEV), table.to(DEV), q_rot, k_cache, v_cache, n_q, n_kv, hd, hd)
    out = torch.empty_like(q_rot)
    ops.attention_generic(q_rot, k_cache, v_cache, out, positions.to(DEV), seq_idx.to(DEV), table.to(DEV),
                          n_q, n_kv, hd, 1.0 / math.sqrt(hd), window)
    row = 0
    for n in lens:
        blk = qkv[row:row + n]
        q = twin.rope_apply(blk[:, :n_q * hd].reshape(n, n_q, hd), cos_all[:n], sin_all[:n])
        k = twin.rope_apply(blk[:, n_q * hd:(n_q + n_kv) * hd].reshape(n, n_kv, hd), cos_all[:n], sin_all[:n])
        v = blk[:, (n_q + n_kv) * hd:].reshape(n, n_kv, hd)
        assert _rel(q_rot[row:row + n].cpu(), q.reshape(n, -1)) < 2e-6
        assert _rel(out[row:row + n].cpu(), twin.attention(q, k, v, window).reshape(n, -1)) < 3e-6
        row += n
