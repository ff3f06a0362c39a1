"""What fixes the plain implementation beside the reference's text: special cases that
reduce to a library routine, invariants, and vectors that the reference's own tests use.
Each case is chosen so that a plausible mistake (a wrong sign or pairing, a norm in the
wrong place, a wrong head mapping) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from plain_llama import (plain_apply_rope, plain_argmax, plain_attention, plain_config, plain_forward,
                         plain_inv_freq, plain_linear, plain_linear_by_rows, plain_mlp, plain_rmsnorm, plain_rope_tables,
                         plain_sample_bounds, plain_silu)
from tiny_models import TINY_A, TINY_B

D = torch.float64


def _gen(s):
    return torch.Generator().manual_seed(s)


# --- RMSNorm -------------------------------------------------------------------------
@pytest.mark.parametrize("dim", [16, 64, 128, 257])        # the reference's sizes (tests/test_kernels.py:26)
def test_rmsnorm_is_the_library_expression(dim):
    x = torch.randn(3, dim, generator=_gen(0), dtype=D)
    w = torch.randn(dim, generator=_gen(1), dtype=D)
    var = x.pow(2).mean(-1, keepdim=True)                   # tests/test_kernels.py:21-23
    assert torch.allclose(plain_rmsnorm(x, w, 1e-5), x * torch.rsqrt(var + 1e-5) * w, atol=1e-12)


def test_rmsnorm_special_cases():
    x = torch.tensor([[3.0, -3.0, 3.0, -3.0]], dtype=D)
    assert torch.allclose(plain_rmsnorm(x, torch.ones(4, dtype=D), 0.0), torch.sign(x))   # |x| const -> sign
    y = torch.randn(2, 32, generator=_gen(2), dtype=D)
    w = 1 + 0.1 * torch.randn(32, generator=_gen(3), dtype=D)
    assert torch.allclose(plain_rmsnorm(7.0 * y, w, 0.0), plain_rmsnorm(y, w, 0.0))        # scale invariance
    assert torch.allclose(plain_rmsnorm(y, 2 * w, 1e-6), 2 * plain_rmsnorm(y, w, 1e-6))    # w multiplies, not 1 + w
    big = plain_rmsnorm(torch.full((1, 8), 1e-4, dtype=D), torch.ones(8, dtype=D), 1.0)
    assert torch.allclose(big, torch.full((1, 8), 1e-4 / math.sqrt(1e-8 + 1.0), dtype=D))  # eps inside the root


# --- linear --------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 8, 16), (1, 128, 128), (4, 64, 32)])     # tests/test_kernels.py:52
def test_linear_is_F_linear(M, N, K):
    a = torch.randn(M, K, generator=_gen(4), dtype=D)
    w = torch.randn(N, K, generator=_gen(5), dtype=D)
    assert torch.allclose(plain_linear_by_rows(a, w), F.linear(a, w), atol=1e-12)
    assert torch.allclose(plain_linear(a, w), plain_linear_by_rows(a, w), atol=1e-12)
    # W is [N, K]: the transposed reading gives another result (and another shape unless N == K)
    if N == K:
        assert not torch.allclose(plain_linear(a, w), a @ w, atol=1e-6)


# --- inverse frequencies -------------------------------------------------------------
def test_inv_freq_without_scaling_is_the_power_law():
    got = plain_inv_freq(64, 10000.0, None)
    for i, v in enumerate(got):
        assert abs(v - 10000.0 ** (-2 * i / 64)) <= 1e-7 * v
    assert got == plain_inv_freq(64, 10000.0, (1.0, 1.0, 4.0, 8192))        # factor 1 changes nothing


def test_inv_freq_bands():
    theta, hd, factor, low, high, orig = 500000.0, 32, 32.0, 1.0, 4.0, 64
    base = plain_inv_freq(hd, theta, None)
    got = plain_inv_freq(hd, theta, (factor, low, high, orig))
    kinds = set()
    for b, g in zip(base, got):
        wavelen = 2 * math.pi / b
        if wavelen < orig / high:
            kinds.add("high")
            assert g == b                                   # short wavelengths untouched
        elif wavelen > orig / low:
            kinds.add("low")
            assert abs(g - b / factor) <= 1e-7 * g          # long wavelengths divided by the factor
        else:
            kinds.add("mid")
            assert b / factor < g < b
    assert kinds == {"high", "low", "mid"}                  # this configuration has all three bands
    assert all(x > y for x, y in zip(got, got[1:]))         # still decreasing


# theta 16 and 32 dims give inverse frequencies 2^(-i/4); with an original length of 16 pi the
# ratio original / wavelength is 8 * 2^(-i/4): 8, 6.7, 5.7, 4.8, 4 (the high edge), 3.4, 2.8, 2.4, 2,
# 1.7, 1.4, 1.2, 1 (the low edge), 0.84, 0.71, 0.59. Entries 5 to 11 lie inside the band, entry 8
# at smooth = (2 - 1) / (4 - 1) = 1/3: 0.25 * (1/3 + (2/3) / 8) = 0.104166..; with high = 5 the
# band starts at entry 3 and entry 8 has smooth 1/4: 0.25 * (1/4 + (3/4) / 8) = 0.0859375.
# Worked by hand from src/kernels.cpp:134-155 (new = (1 - smooth) * f / factor + smooth * f with
# smooth = (original / wavelength - low) / (high - low)). The reference's own tests hold this
# formula against the transformers package (tests/test_kernels.py:88-110); library model code is
# not a source here, so parity with that package is unpinned and these numbers stand in.
_MID_BAND = {
    (1.0, 4.0): [1.0, 0.840896415, 0.707106781, 0.594603558, 0.5, 0.342404254, 0.232741102, 0.156689181,
                 0.104166667, 0.0680823883, 0.0434538841, 0.0267847212, 0.015625, 0.0131390065, 0.0110485435,
                 0.00929068059],
    (1.0, 5.0): [1.0, 0.840896415, 0.707106781, 0.56297435, 0.390625, 0.269942197, 0.18560437, 0.126807567,
                 0.0859375, 0.0576312945, 0.0381146848, 0.0247338812, 0.015625, 0.0131390065, 0.0110485435,
                 0.00929068059],
}


@pytest.mark.parametrize("low,high", list(_MID_BAND))
def test_inv_freq_mid_band_values(low, high):
    """Seven (nine) entries inside the band at known blend weights. A blend with its weights
    swapped, a squared weight, the wavelength in place of its inverse, or a constant weight all
    give other numbers (entry 8 alone: 0.177, 0.0556, 0.0703, 0.141 instead of 0.104)."""
    got = plain_inv_freq(32, 16.0, (8.0, low, high, 16.0 * math.pi))
    want = _MID_BAND[(low, high)]
    for i, (g, w) in enumerate(zip(got, want)):
        assert abs(g - w) <= 2e-7 * w, (i, g, w)
    assert abs(got[8] - (0.25 * (1 / 3 + (2 / 3) / 8) if high == 4.0 else 0.0859375)) < 1e-8


def test_inv_freq_blend_is_affine_in_the_frequency_and_continuous():
    """new / old = 1/factor + smooth (1 - 1/factor) with smooth affine in the frequency itself:
    inside the band the points (old, new / old) lie on one line, which runs from 1/factor at the
    low edge to 1 at the high edge (so the bands meet without a jump)."""
    factor, low, high, orig = 32.0, 1.0, 4.0, 8192
    base = plain_inv_freq(128, 500000.0, None)                       # the sizes of the real models
    got = plain_inv_freq(128, 500000.0, (factor, low, high, orig))
    mid = [(b, g / b) for b, g in zip(base, got) if orig / high <= 2 * math.pi / b <= orig / low]
    assert len(mid) >= 5
    edge_lo, edge_hi = 2 * math.pi * low / orig, 2 * math.pi * high / orig     # the band's frequencies
    for b, ratio in mid:
        smooth = (b - edge_lo) / (edge_hi - edge_lo)
        assert abs(ratio - (1 / factor + smooth * (1 - 1 / factor))) < 1e-6, (b, ratio)
    assert all(r1 > r2 for (_, r1), (_, r2) in zip(mid, mid[1:]))    # higher frequencies keep more


def test_rope_tables_values():
    inv = plain_inv_freq(32, 500000.0, (32.0, 1.0, 4.0, 8192))
    cos, sin = plain_rope_tables(inv, [0, 1, 100, 1000, 8000], 32)      # tests/test_real_smoke.py:107-137
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)
    assert torch.equal(cos[:, :16], cos[:, 16:]) and torch.equal(sin[:, :16], sin[:, 16:])
    for r, p in enumerate([0, 1, 100, 1000, 8000]):
        for i in range(16):
            assert abs(cos[r, i].item() - math.cos(p * inv[i])) < 1e-7
            assert abs(sin[r, i].item() - math.sin(p * inv[i])) < 1e-7
    assert torch.allclose(cos ** 2 + sin ** 2, torch.ones_like(cos), atol=1e-6)


# --- rotation ------------------------------------------------------------------------
def _tables(hd, positions, theta=10000.0, scaling=None):
    return plain_rope_tables(plain_inv_freq(hd, theta, scaling), positions, hd)


def test_rope_is_rotate_half():
    hd = 32
    x = torch.randn(4, 3, hd, generator=_gen(6), dtype=D)
    cos, sin = _tables(hd, [0, 1, 5, 15], 500000.0, (32.0, 1.0, 4.0, 8192))       # tests/test_kernels.py:131
    rot = torch.cat((-x[..., hd // 2:], x[..., :hd // 2]), dim=-1)                 # tests/test_kernels.py:115-121
    want = x * cos[:, None, :] + rot * sin[:, None, :]
    assert torch.allclose(plain_apply_rope(x, cos, sin), want, atol=1e-12)


def test_rope_invariants():
    hd = 16
    q = torch.randn(1, 1, hd, generator=_gen(7), dtype=D)
    k = torch.randn(1, 1, hd, generator=_gen(8), dtype=D)
    cos0, sin0 = _tables(hd, [0])
    assert torch.equal(plain_apply_rope(q, cos0, sin0), q)                          # position 0: identity
    cos, sin = _tables(hd, [37])
    r = plain_apply_rope(q, cos, sin)
    h = hd // 2
    assert torch.allclose(r[..., :h] ** 2 + r[..., h:] ** 2, q[..., :h] ** 2 + q[..., h:] ** 2, atol=1e-6)

    def dot(m, n):
        cm, sm = _tables(hd, [m])
        cn, sn = _tables(hd, [n])
        return float((plain_apply_rope(q, cm, sm) * plain_apply_rope(k, cn, sn)).sum())
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-5              # only the distance counts
    assert abs(dot(9, 4) - dot(4, 9)) > 1e-3                # and its sign does count (a wrong sign fails here)
    # pairing (i, i + h), not (2i, 2i + 1): rotating a vector with one nonzero entry moves
    # weight to the entry h places further on
    e = torch.zeros(1, 1, hd, dtype=D)
    e[0, 0, 1] = 1.0
    c1, s1 = _tables(hd, [3])
    out = plain_apply_rope(e, c1, s1)[0, 0]
    assert out[1 + h].abs() > 1e-3 and out[2].abs() < 1e-12 and out[0].abs() < 1e-12
    assert out[1 + h] > 0                                    # x[i + h] <- b cos + a sin: +sin for a > 0


# --- attention -----------------------------------------------------------------------
@pytest.mark.parametrize("n_q,n_kv,hd,T", [(4, 2, 32, 1), (4, 2, 32, 7), (8, 2, 16, 13)])   # tests/test_kernels.py:194
def test_attention_is_causal_sdpa(n_q, n_kv, hd, T):
    q = torch.randn(T, n_q, hd, generator=_gen(9), dtype=D)
    k = torch.randn(T, n_kv, hd, generator=_gen(10), dtype=D)
    v = torch.randn(T, n_kv, hd, generator=_gen(11), dtype=D)
    g = n_q // n_kv
    kk = k.repeat_interleave(g, dim=1).transpose(0, 1)       # head h reads kv head h // g
    vv = v.repeat_interleave(g, dim=1).transpose(0, 1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, is_causal=True).transpose(0, 1)
    assert torch.allclose(plain_attention(q, k, v), want, atol=1e-10)


def test_attention_special_cases():
    q = torch.randn(5, 4, 8, generator=_gen(12), dtype=D)
    k = torch.randn(5, 2, 8, generator=_gen(13), dtype=D)
    v = torch.randn(5, 2, 8, generator=_gen(14), dtype=D)
    out = plain_attention(q, k, v)
    for h in range(4):
        assert torch.allclose(out[0, h], v[0, h // 2])       # one key: the value row itself
    same = v[:1].expand(5, 2, 8).clone()
    assert torch.allclose(plain_attention(q, k, same), same[:, [0, 0, 1, 1]])      # equal rows: that row
    # head mapping h // group, not h % n_kv: make kv head 1 special
    v2 = torch.zeros(5, 2, 8, dtype=D)
    v2[:, 1] = 1.0
    o2 = plain_attention(q, k, v2)
    assert torch.all(o2[:, :2] == 0) and torch.allclose(o2[:, 2:], torch.ones(5, 2, 8, dtype=D))
    # window 1 sees only the own key; window >= T is no window
    assert torch.allclose(plain_attention(q, k, v, window=1), v[:, [0, 0, 1, 1]])
    assert torch.allclose(plain_attention(q, k, v, window=5), out)
    # scale is 1/sqrt(hd): one query of all ones against keys e_0 * c
    q1 = torch.ones(2, 1, 4, dtype=D)
    k1 = torch.zeros(2, 1, 4, dtype=D)
    k1[1, 0, 0] = 2.0
    v1 = torch.tensor([[[1.0, 0, 0, 0]], [[0, 1.0, 0, 0]]], dtype=D)
    p = math.exp(2.0 / 2.0) / (1 + math.exp(2.0 / 2.0))     # scores 0 and 2 / sqrt(4)
    assert abs(plain_attention(q1, k1, v1)[1, 0, 1].item() - p) < 1e-12


# --- feed-forward --------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 16, 384])                 # tests/test_kernels.py:40-47
def test_silu_is_F_silu(n):
    x = 3 * torch.randn(n, generator=_gen(15), dtype=D)
    assert torch.allclose(plain_silu(x), F.silu(x), atol=1e-12)
    assert plain_silu(torch.zeros(1, dtype=D)).item() == 0.0


def test_mlp_is_gated():
    x = torch.randn(3, 8, generator=_gen(16), dtype=D)
    wg, wu = torch.randn(12, 8, generator=_gen(17), dtype=D), torch.randn(12, 8, generator=_gen(18), dtype=D)
    wd = torch.randn(8, 12, generator=_gen(19), dtype=D)
    want = F.linear(F.silu(F.linear(x, wg)) * F.linear(x, wu), wd)
    assert torch.allclose(plain_mlp(x, wg, wu, wd), want, atol=1e-10)
    assert not torch.allclose(plain_mlp(x, wu, wg, wd), want, atol=1e-3)     # gate and up are not interchangeable


# --- whole model ---------------------------------------------------------------------
def _random_weights(cfg, seed):
    """A checkpoint's tensors by the names and shapes of src/model.cpp:179-287, drawn here (nothing
    of the engine is imported)."""
    c = plain_config(cfg)
    g = _gen(seed)
    H, FF, q_dim, kv_dim = c["H"], c["FF"], c["n_q"] * c["hd"], c["n_kv"] * c["hd"]

    def lin(*shape):
        return 0.05 * torch.randn(*shape, generator=g)

    def norm():
        return 1.0 + 0.1 * torch.randn(H, generator=g)
    w = {"model.embed_tokens.weight": lin(c["V"], H), "model.norm.weight": norm()}
    if not c["tie"]:
        w["lm_head.weight"] = lin(c["V"], H)
    for layer in range(c["L"]):
        p = f"model.layers.{layer}."
        w.update({p + "input_layernorm.weight": norm(), p + "post_attention_layernorm.weight": norm(),
                  p + "self_attn.q_proj.weight": lin(q_dim, H), p + "self_attn.k_proj.weight": lin(kv_dim, H),
                  p + "self_attn.v_proj.weight": lin(kv_dim, H), p + "self_attn.o_proj.weight": lin(H, q_dim),
                  p + "mlp.gate_proj.weight": lin(FF, H), p + "mlp.up_proj.weight": lin(FF, H),
                  p + "mlp.down_proj.weight": lin(H, FF)})
    return w


def test_config_defaults():
    c = plain_config({"hidden_size": 64, "intermediate_size": 8, "num_hidden_layers": 1, "num_attention_heads": 4,
                      "vocab_size": 10, "max_position_embeddings": 16})
    assert (c["n_kv"], c["hd"], c["eps"], c["theta"], c["tie"], c["scaling"]) == (4, 16, 1e-5, 10000.0, False, None)
    assert plain_config(TINY_B)["scaling"] == (32.0, 1.0, 4.0, 64)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_zero_output_projections_leave_the_embedding(cfg):
    w = _random_weights(cfg, 3)
    for k in w:
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            w[k] = torch.zeros_like(w[k])
    ids = [3, 1, 4, 1, 5]
    emb = w["model.embed_tokens.weight"].double()
    head = emb if cfg["tie_word_embeddings"] else w["lm_head.weight"].double()
    x = emb[ids]
    normed = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg["rms_norm_eps"]) * w["model.norm.weight"].double()
    assert torch.allclose(plain_forward(cfg, w, ids), normed @ head.T, atol=1e-10)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B])
def test_a_shift_of_all_positions_changes_nothing(cfg):
    """Only distances between positions count (also under llama3 scaling, which rescales
    frequencies, not positions)."""
    w = _random_weights(cfg, 4)
    ids = [7, 7, 2, 9, 30, 11]
    base = plain_forward(cfg, w, ids)
    shifted = plain_forward(cfg, w, ids, positions=range(40, 46))
    assert torch.allclose(base, shifted, atol=1e-6)
    moved = plain_forward(cfg, w, ids, positions=[0, 1, 2, 3, 4, 9])        # a changed distance does count
    assert not torch.allclose(base[-1], moved[-1], atol=1e-6)


def test_causality_and_layer_composition():
    w = _random_weights(TINY_A, 5)
    ids = [5, 6, 7, 8, 9, 10]
    full = plain_forward(TINY_A, w, ids)
    assert torch.allclose(plain_forward(TINY_A, w, ids[:4]), full[:4], atol=1e-10)    # later tokens are unseen
    one = dict(TINY_A, num_hidden_layers=1)
    assert not torch.allclose(plain_forward(one, w, ids), full, atol=1e-4)            # the second layer acts
    again = plain_forward(TINY_A, w, ids, schedule=[(0, 0, True), (1, 1, True)])
    assert torch.equal(again, full)


def test_argmax_and_sampling_bounds():
    assert plain_argmax(torch.tensor([1.0, 5.0, 5.0, 2.0])) == 1            # first maximum
    cum = plain_sample_bounds(torch.tensor([0.0, math.log(3.0)]), 1.0)
    assert torch.allclose(cum, torch.tensor([0.25, 1.0], dtype=D))
    cold = plain_sample_bounds(torch.tensor([0.0, 1.0]), 1e-3)
    assert cold[0] < 1e-12                                                   # T -> 0 is greedy
