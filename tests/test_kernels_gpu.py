"""Each HIP kernel alone against the plain implementation, at sizes other than the
engine's tiny models: widths and vocabularies that are no power of two, head sizes in
steps of 16, several page sizes, both storage types."""
import math

import pytest
import torch

from plain_llama import (bf16_round, plain_apply_rope, plain_argmax, plain_attention, plain_linear,
                         plain_rmsnorm, plain_sample_bounds, plain_silu)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _rel(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).abs().max() / b.double().abs().max().clamp_min(1e-30))


@pytest.fixture(scope="module")
def ops():
    from llmengine import ops
    ops.library()
    return ops


@pytest.mark.parametrize("V,H,dtype", [(37, 50, torch.float32), (129, 96, torch.bfloat16), (64, 72, torch.float32),
                                       (300, 2048, torch.bfloat16), (41, 100, torch.bfloat16)])
def test_embed_gather(ops, V, H, dtype):
    table = torch.randn(V, H, generator=_gen(0)).to(dtype)
    tokens = torch.tensor([0, 1, 7, V - 1, 3, 3], dtype=torch.int32)
    out = torch.empty(len(tokens), H, dtype=torch.float32, device=DEV)
    ops.embed_gather(table.to(DEV), tokens.to(DEV), out)
    assert torch.equal(out.cpu(), table[tokens.long()].float())       # exact row copies


@pytest.mark.parametrize("H", [16, 64, 257, 2048, 3000])
@pytest.mark.parametrize("wdtype,odtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                           (torch.float32, torch.bfloat16)])
def test_rmsnorm(ops, H, wdtype, odtype):
    x = torch.randn(5, H, generator=_gen(1)) * 3
    w = (1 + 0.1 * torch.randn(H, generator=_gen(2))).to(wdtype)
    out = torch.empty(5, H, dtype=odtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-6, out)
    ref = plain_rmsnorm(x.double(), w.double(), 1e-6)
    if odtype == torch.float32:
        assert _rel(out.cpu(), ref) < 2e-6
    else:
        assert torch.equal(out.cpu().float(), ref.float().to(torch.bfloat16).float()) or \
            _rel(out.cpu().float(), ref) < 8e-3
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=DEV)
    picked = torch.empty(3, H, dtype=odtype, device=DEV)
    ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-6, picked, rows)
    assert torch.equal(picked.cpu(), out.cpu()[[4, 0, 4]])


@pytest.mark.parametrize("M,N,K", [(1, 8, 16), (1, 128, 128), (4, 64, 32), (7, 100, 50), (65, 67, 33),
                                   (130, 331, 144), (3, 96, 176)])
@pytest.mark.parametrize("adt,wdt,odt", [(torch.float32,) * 3, (torch.bfloat16,) * 3,
                                         (torch.bfloat16, torch.bfloat16, torch.float32),
                                         (torch.bfloat16, torch.float32, torch.float32)])
def test_gemm_generic(ops, M, N, K, adt, wdt, odt):
    a = torch.randn(M, K, generator=_gen(3)).to(adt)
    w = torch.randn(N, K, generator=_gen(4)).to(wdt)
    out = torch.full((M, N), 7.0, dtype=odt, device=DEV)
    ops.gemm_generic(a.to(DEV), w.to(DEV), out)
    ref = plain_linear(a.double(), w.double())
    tol = 2e-6 if odt == torch.float32 else 8e-3
    assert _rel(out.cpu().double(), ref) < tol
    # accumulate adds into what is there
    base = torch.randn(M, N, generator=_gen(5)).to(odt)
    out2 = base.clone().to(DEV)
    ops.gemm_generic(a.to(DEV), w.to(DEV), out2, accumulate=True)
    assert _rel(out2.cpu().double(), ref + base.double()) < (4e-6 if odt == torch.float32 else 1.6e-2)


@pytest.mark.parametrize("FF,group", [(176, 16), (50, 50), (384, 16)])
def test_swiglu(ops, FF, group):
    T = 3
    g = 3 * torch.randn(T, FF, generator=_gen(6))
    u = torch.randn(T, FF, generator=_gen(7))
    gu = torch.empty(T, 2 * FF)
    gu.view(T, FF // group, 2, group)[:, :, 0] = g.view(T, FF // group, group)
    gu.view(T, FF // group, 2, group)[:, :, 1] = u.view(T, FF // group, group)
    out = torch.empty(T, FF, dtype=torch.float32, device=DEV)
    ops.swiglu(gu.to(DEV), out, group)
    ref = plain_silu(g.double()) * u.double()
    assert (out.cpu().double() - ref).abs().max() < 1e-5
    z = torch.zeros(1, 2 * FF)
    z.view(1, FF // group, 2, group)[:, :, 1] = 5.0
    outz = torch.empty(1, FF, dtype=torch.float32, device=DEV)
    ops.swiglu(z.to(DEV), outz, group)
    assert torch.all(outz == 0)                      # gate 0 gives 0 whatever up is


def _paged_setup(ops, lens, n_q, n_kv, hd, page, dtype, seed, rotate=True, scramble=True):
    """Random q/k/v for requests of the given lengths, written through rope_kv_write into
    scrambled pages. Returns everything attention needs plus the plain per-request q, k, v."""
    T = sum(lens)
    g = _gen(seed)
    qkv = torch.randn(T, (n_q + 2 * n_kv) * hd, generator=g)
    max_pos = max(lens) + 3
    half = hd // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    nblk = [(n + page - 1) // page for n in lens]
    total_pages = sum(nblk) + 2
    perm = torch.randperm(total_pages, generator=g).tolist() if scramble else list(range(total_pages))
    max_blocks = max(nblk)
    table = torch.zeros(len(lens), max_blocks, dtype=torch.int32)
    p = 0
    for s, nb in enumerate(nblk):
        for b in range(nb):
            table[s, b] = perm[p]
            p += 1
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    seq_idx = torch.cat([torch.full((n,), s) for s, n in enumerate(lens)]).to(torch.int32)
    k_cache = torch.zeros(total_pages, n_kv, page, hd, dtype=dtype, device=DEV)
    v_cache = torch.zeros(total_pages, n_kv, hd, page, dtype=dtype, device=DEV)
    q_out = torch.empty(T, n_q * hd, dtype=dtype, device=DEV)
    ops.rope_kv_write(qkv.to(DEV), cos.to(DEV) if rotate else None, sin.to(DEV) if rotate else None,
                      positions.to(DEV), seq_idx.to(DEV), table.to(DEV), q_out, k_cache, v_cache,
                      n_q, n_kv, hd, hd)
    # plain side
    plain = []
    row = 0
    for n in lens:
        blk = qkv[row:row + n].double()
        q = blk[:, :n_q * hd].reshape(n, n_q, hd)
        k = blk[:, n_q * hd:(n_q + n_kv) * hd].reshape(n, n_kv, hd)
        v = blk[:, (n_q + n_kv) * hd:].reshape(n, n_kv, hd)
        if rotate:
            c = torch.cat([cos[:n], cos[:n]], dim=1).double()
            s_ = torch.cat([sin[:n], sin[:n]], dim=1).double()
            q, k = plain_apply_rope(q, c, s_), plain_apply_rope(k, c, s_)
        if dtype == torch.bfloat16:
            q, k, v = bf16_round(q), bf16_round(k), bf16_round(v)
        plain.append((q, k, v))
        row += n
    return dict(q=q_out, k_cache=k_cache, v_cache=v_cache, positions=positions.to(DEV),
                seq_idx=seq_idx.to(DEV), table=table.to(DEV), plain=plain, T=T, qkv=qkv)


@pytest.mark.parametrize("n_q,n_kv,hd,page,lens", [
    (4, 2, 32, 4, [1]), (4, 2, 32, 4, [7]), (8, 2, 16, 8, [13, 5]), (3, 1, 48, 16, [33, 2, 17]),
    (6, 3, 80, 16, [70]), (4, 4, 128, 32, [65, 40]), (2, 1, 256, 16, [20]),
    (8, 2, 32, 16, [300, 230])])        # (4,096 (token, head) pairs and more: one wavefront each; fewer: 16 that join)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_write_and_attention_generic(ops, n_q, n_kv, hd, page, lens, dtype):
    s = _paged_setup(ops, lens, n_q, n_kv, hd, page, dtype, seed=11)
    # the rotated queries
    q_ref = torch.cat([p[0].reshape(-1, n_q * hd) for p in s["plain"]])
    assert _rel(s["q"].cpu().double(), q_ref) < (2e-6 if dtype == torch.float32 else 1e-9 + 4e-3)
    out = torch.empty_like(s["q"])
    ops.attention_generic(s["q"], s["k_cache"], s["v_cache"], out, s["positions"], s["seq_idx"], s["table"],
                          n_q, n_kv, hd, 1.0 / math.sqrt(hd))
    ref = torch.cat([plain_attention(q, k, v).reshape(-1, n_q * hd) for q, k, v in s["plain"]])
    assert _rel(out.cpu().double(), ref) < (3e-6 if dtype == torch.float32 else 8e-3)


def test_attention_generic_window_and_far_key(ops):
    """A window's edge, and one far key that dominates: the key at position 3 gets a large
    score for the last query; with a window that excludes it the result must change."""
    n_q, n_kv, hd, page = 2, 1, 32, 8
    lens = [300]
    s = _paged_setup(ops, lens, n_q, n_kv, hd, page, torch.float32, seed=5, rotate=False)
    q, k, v = s["plain"][0]
    out = torch.empty_like(s["q"])
    for window in (0, 64, 297, 298):
        ops.attention_generic(s["q"], s["k_cache"], s["v_cache"], out, s["positions"], s["seq_idx"],
                              s["table"], n_q, n_kv, hd, 1.0 / math.sqrt(hd), window)
        ref = plain_attention(q, k, v, window).reshape(-1, n_q * hd)
        assert _rel(out.cpu().double(), ref) < 3e-6, window


def test_attention_single_key_is_value_row(ops):
    s = _paged_setup(ops, [1], 4, 2, 32, 4, torch.float32, seed=3)
    out = torch.empty_like(s["q"])
    ops.attention_generic(s["q"], s["k_cache"], s["v_cache"], out, s["positions"], s["seq_idx"], s["table"],
                          4, 2, 32, 0.5)
    v = s["plain"][0][2]                                     # [1, n_kv, hd]
    want = torch.stack([v[0, h // 2] for h in range(4)]).reshape(1, -1)
    assert torch.allclose(out.cpu().double(), want, atol=1e-6)


@pytest.mark.parametrize("V", [5, 256, 331, 128256])
def test_argmax_first_maximum(ops, V):
    logits = torch.randn(4, V, generator=_gen(9))
    logits[1, V // 2] = logits[1, V - 1] = 50.0          # tie: the lower id wins
    logits[2, 0] = 60.0
    logits[3, V - 1] = 70.0
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops.argmax(logits.to(DEV), out)
    assert out.tolist() == [plain_argmax(r) for r in logits]
    assert out.tolist()[1] == V // 2


@pytest.mark.parametrize("V,R", [(7, 64), (300, 64), (5000, 64), (2049, 3), (128256, 8)])
def test_temperature_sampling_interval(ops, V, R):
    logits = 2 * torch.randn(R, V, generator=_gen(10))
    u = torch.rand(R, generator=_gen(11))
    temp = torch.full((R,), 0.8)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    ops.sample(logits.to(DEV), temp.to(DEV), u.to(DEV), out)
    for r in range(R):
        cum = plain_sample_bounds(logits[r], 0.8)
        tok = out[r].item()
        lo = cum[tok - 1].item() if tok > 0 else 0.0
        assert lo - 1e-5 <= u[r].item() <= cum[tok].item() + 1e-5, (r, tok)
    # temperature 0 is greedy
    zero = torch.zeros(R)
    ops.sample(logits.to(DEV), zero.to(DEV), u.to(DEV), out)
    assert out.tolist() == logits.argmax(dim=1).tolist()


# --- MFMA matrix products ----------------------------------------------------------------
def _bf16_pair(M, N, K, seed):
    a = torch.randn(M, K, generator=_gen(seed)).to(torch.bfloat16)
    w = torch.randn(N, K, generator=_gen(seed + 1)).to(torch.bfloat16)
    return a, w, a.double() @ w.double().T


@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (1, 2048, 2048), (8, 3072, 2048), (3, 100, 176), (16, 331, 144),
                                   (17, 48, 40), (33, 96, 96), (64, 2048, 8192), (50, 129, 1000)])
@pytest.mark.parametrize("waves,ksplit", [(0, 0), (4, 1), (8, 1), (16, 1), (4, 3)])
def test_gemm_skinny(ops, M, N, K, waves, ksplit):
    a, w, ref = _bf16_pair(M, N, K, 20)
    base = torch.randn(M, N, generator=_gen(22))
    if ksplit > 1:
        out = base.clone().to(DEV)
        ops.gemm_bf16(a.to(DEV), w.to(DEV), out, accumulate=True, waves=waves, ksplit=ksplit)
        assert _rel(out.cpu().double(), ref + base.double()) < 2e-5
        return
    out = torch.full((M, N), 3.0, device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), out, waves=waves)
    assert _rel(out.cpu().double(), ref) < 2e-5
    acc = base.clone().to(DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True, waves=waves)
    assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5
    half = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), half, waves=waves)
    assert _rel(half.cpu().double(), ref) < 5e-3


@pytest.mark.parametrize("M,N,K", [(65, 128, 64), (128, 128, 128), (200, 331, 144), (129, 100, 176), (257, 500, 72),
                                   (2048, 3072, 2048), (1000, 2048, 8192), (7, 40, 24)])
@pytest.mark.parametrize("tile", [64, 128, 128096, 128064, 96128, 96064])
def test_gemm_tile(ops, M, N, K, tile):
    a, w, ref = _bf16_pair(M, N, K, 30)
    out = torch.full((M, N), 3.0, device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), out, tile=tile)
    assert _rel(out.cpu().double(), ref) < 2e-5
    base = torch.randn(M, N, generator=_gen(32))
    acc = base.clone().to(DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True, tile=tile)
    assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5
    for ksplit in (2, 5):
        acc = base.clone().to(DEV)
        ops.gemm_bf16(a.to(DEV), w.to(DEV), acc, accumulate=True, tile=tile, ksplit=ksplit)
        assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5, ksplit
    half = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a.to(DEV), w.to(DEV), half, tile=tile)
    assert _rel(half.cpu().double(), ref) < 5e-3


@pytest.mark.parametrize("M,N,K", [(65, 128, 64), (128, 128, 128), (300, 400, 96), (129, 112, 160), (257, 512, 32),
                                   (2048, 3072, 2048), (1000, 2048, 8192), (333, 208, 2080), (513, 528, 192),
                                   (700, 1040, 224), (256, 256, 256), (511, 272, 320)])
def test_gemm_tile_with_slabs_straight_into_lds(ops, M, N, K, tile=256256):
    """The 256 x 256 tile kernel whose slabs go from memory into LDS without passing through
    registers (blocked weights): every epilogue, sums cut over k, tiles that hang over the
    matrix's edges, k of half a slab, of one and of many, ending in half a slab or a whole one;
    against the plain product, and bit for bit against the kernel that stages its slabs through
    registers (both add the same products in the same order)."""
    a, w, ref = _bf16_pair(M, N, K, 35)
    ad, wb = a.to(DEV), ops.block_weight(w.to(DEV))
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 5e-3)):
        direct = torch.full((M, N), 3.0, dtype=dtype, device=DEV)
        staged = torch.full((M, N), 5.0, dtype=dtype, device=DEV)
        ops.gemm_bf16(ad, wb, direct, tile=tile, direct=1)
        ops.gemm_bf16(ad, wb, staged, tile=min(tile, 128), direct=0)
        assert _rel(direct.cpu().double(), ref) < tol
        assert torch.equal(direct, staged)
    base = torch.randn(M, N, generator=_gen(36))
    acc, acc0 = base.clone().to(DEV), base.clone().to(DEV)
    ops.gemm_bf16(ad, wb, acc, accumulate=True, tile=tile, direct=1)
    ops.gemm_bf16(ad, wb, acc0, accumulate=True, tile=min(tile, 128), direct=0)
    assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5 and torch.equal(acc, acc0)
    for ksplit in (2, 5):
        acc = base.clone().to(DEV)
        ops.gemm_bf16(ad, wb, acc, accumulate=True, tile=tile, ksplit=ksplit, direct=1)
        assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5, ksplit
    if N % 32 == 0:                                   # gate and up rows interleaved in groups of 16
        gated = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
        gated0 = torch.empty(M, N // 2, dtype=torch.bfloat16, device=DEV)
        ops.gemm_bf16(ad, wb, gated, gated=True, tile=tile, direct=1)
        ops.gemm_bf16(ad, wb, gated0, gated=True, tile=min(tile, 128), direct=0)
        gu = ref.view(M, N // 32, 2, 16)
        want = (plain_silu(gu[:, :, 0]) * gu[:, :, 1]).reshape(M, N // 2)
        assert _rel(gated.cpu().double(), want) < 8e-3 and torch.equal(gated, gated0)
    from llmengine.ops import KernelError
    with pytest.raises(KernelError):
        ops.gemm_bf16(ad, w.to(DEV), torch.empty(M, N, device=DEV), tile=tile, direct=1)     # row-major weights


@pytest.mark.parametrize("M", [17, 24, 32, 33, 50, 64, 65, 81, 96, 97, 130, 160, 192, 200, 273, 288, 300])
@pytest.mark.parametrize("N,K", [(2048, 8192), (2048, 2048), (3072, 4096)])
def test_gemm_sums_of_a_few_dozen_to_a_few_hundred_rows(ops, M, N, K):
    """Sums into the residual stream at the row counts of decoding at larger batches and of a
    prompt portion beside decoded tokens, whatever tile and cut over k the entry point chooses
    there (tiles of 96 x 64 cut in 2 or 4 for long sums at 129 to 288 rows)."""
    a, w, ref = _bf16_pair(M, N, K, 37)
    base = torch.randn(M, N, generator=_gen(38))
    for weight in (w.to(DEV), ops.block_weight(w.to(DEV))):
        acc = base.clone().to(DEV)
        ops.gemm_bf16(a.to(DEV), weight, acc, accumulate=True)
        assert _rel(acc.cpu().double(), ref + base.double()) < 2e-5


@pytest.mark.parametrize("T,FF,K,tile", [(5, 176, 64, 0), (130, 256, 96, 64), (300, 208, 144, 128), (2048, 8192, 2048, 0),
                                         (257, 320, 128, 128096), (190, 352, 72, 128064), (64, 8192, 2048, 0),
                                         (273, 8192, 2048, 0), (192, 8192, 2048, 0), (190, 352, 72, 96064),
                                         (257, 320, 128, 96128), (33, 8192, 2048, 0), (20, 352, 72, 0)])
def test_gemm_gated(ops, T, FF, K, tile):
    x = torch.randn(T, K, generator=_gen(33)).to(torch.bfloat16)
    wg = (0.1 * torch.randn(FF, K, generator=_gen(34))).to(torch.bfloat16)
    wu = (0.1 * torch.randn(FF, K, generator=_gen(35))).to(torch.bfloat16)
    fused = torch.empty(2 * FF, K, dtype=torch.bfloat16)
    fused.view(FF // 16, 2, 16, K)[:, 0] = wg.view(FF // 16, 16, K)
    fused.view(FF // 16, 2, 16, K)[:, 1] = wu.view(FF // 16, 16, K)
    out = torch.zeros(T, FF, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(x.to(DEV), fused.to(DEV), out, gated=True, tile=tile)
    g, u = x.double() @ wg.double().T, x.double() @ wu.double().T
    ref = plain_silu(g) * u
    assert _rel(out.cpu().double(), ref) < 5e-3
    # the dispatcher's other way: 32-bit product, then the activation kernel
    ops.policy.fast_gemm = False
    try:
        out2 = torch.zeros(T, FF, dtype=torch.bfloat16, device=DEV)
        ops.gemm_gated(x.to(DEV), fused.to(DEV), out2, 16, lambda shape, dtype: torch.empty(shape, dtype=dtype, device=DEV))
    finally:
        ops.policy.fast_gemm = True
    assert _rel(out2.cpu().double(), ref) < 5e-3


def test_gemm_dispatch_and_refusals(ops):
    from llmengine.ops import KernelError
    a, w, ref = _bf16_pair(5, 30, 36, 40)               # K = 36 is no multiple of 8: the plain kernel takes it
    out = torch.empty(5, 30, device=DEV)
    ops.gemm(a.to(DEV), w.to(DEV), out)
    assert _rel(out.cpu().double(), ref) < 2e-5
    with pytest.raises(KernelError):
        ops.gemm_bf16(a.to(DEV), w.to(DEV), out)
    with pytest.raises(KernelError):
        ops.gemm(a.to(DEV), w.to(DEV)[:, :30].contiguous(), out)      # inner sizes differ
    with pytest.raises(KernelError):
        ops.gemm(a, w, out.cpu())                                      # not on the GPU


# --- MFMA attention ----------------------------------------------------------------------
def _attn_case(ops, lens, news, n_q, n_kv, hd, page, window=0, seed=50, prefill_splits=None, prefill_run=1, tuning=0):
    """Requests with lens[i] tokens in the cache, of which the last news[i] are this step's.
    prefill_splits, prefill_run: cut the keys of the prompt portions into at most that many runs of that
    many 64-key stretches, whatever the plan says."""
    s = _paged_setup(ops, lens, n_q, n_kv, hd, page, torch.bfloat16, seed=seed)
    rows, q_start, ctx = [], [0], []
    base = 0
    for n, new in zip(lens, news):
        rows += list(range(base + n - new, base + n))
        q_start.append(q_start[-1] + new)
        ctx.append(n - new)
        base += n
    q = s["q"][torch.tensor(rows, device=DEV)].contiguous()
    out = torch.zeros_like(q)
    i32 = dict(dtype=torch.int32, device=DEV)
    plan = ops.mfma.plan_attention(news, ctx, n_q, n_kv, hd, tuning=tuning)
    S = len(lens)
    part_o = torch.empty(S * n_q * plan["nsplit"] * hd, device=DEV)
    part_ml = torch.empty(S * n_q * plan["nsplit"] * 2, device=DEV)
    if prefill_splits is not None:
        plan["prefill_splits"], plan["prefill_run"] = prefill_splits, prefill_run
    # (the scratch starts as NaN: a part that is joined without having been written shows)
    pre_o = torch.full((len(rows) * n_q * plan["prefill_splits"] * hd,), float("nan"), device=DEV)
    pre_ml = torch.full((len(rows) * n_q * plan["prefill_splits"] * 2,), float("nan"), device=DEV)
    ops.mfma.attention_bf16(q, s["k_cache"], s["v_cache"], out, torch.tensor(q_start, **i32), torch.tensor(ctx, **i32),
                            s["table"], n_q, n_kv, hd, 1.0 / math.sqrt(hd), window, plan, part_o, part_ml, pre_o, pre_ml)
    ref = torch.cat([plain_attention(qq, kk, vv, window)[n - new:].reshape(new, n_q * hd)
                     for (qq, kk, vv), n, new in zip(s["plain"], lens, news)])
    return out.cpu().double(), ref, plan


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(4, 2, 16, 16), (3, 1, 32, 16), (6, 2, 48, 32), (32, 8, 64, 16),
                                              (5, 5, 80, 16), (8, 2, 96, 64), (4, 1, 112, 16), (8, 2, 128, 16),
                                              (34, 2, 64, 16)])
def test_attention_mfma_decode(ops, n_q, n_kv, hd, page):
    lens = [1, 2, 31, 32, 33, 300, 77]
    out, ref, plan = _attn_case(ops, lens, [1] * len(lens), n_q, n_kv, hd, page)
    assert plan["n_decode"] == len(lens) and plan["groups"] == 0
    assert _rel(out, ref) < 8e-3


def test_attention_mfma_decode_splits(ops, monkeypatch):
    """Few requests with a long context: the keys are cut into many splits and joined."""
    out, ref, plan = _attn_case(ops, [1500, 40], [1, 1], 8, 2, 64, 16)
    assert plan["nsplit"] > 4
    assert _rel(out, ref) < 8e-3
    monkeypatch.setattr(ops.policy, "decode_blocks_wanted", 1)     # (the choices of calls without a step)
    out1, ref1, plan1 = _attn_case(ops, [1500, 40], [1, 1], 8, 2, 64, 16)
    assert plan1["nsplit"] == 1 and _rel(out1, ref1) < 8e-3


def _plain_attention_last_row(q, k, v):
    """plain_attention's formula for the last position alone (which sees every key): [n_q, hd]."""
    n_q, hd = q.shape[1], q.shape[2]
    group = n_q // k.shape[1]
    out = torch.zeros(n_q, hd, dtype=torch.float64)
    for h in range(n_q):
        scores = (k[:, h // group] * q[-1, h]).sum(dim=-1) / math.sqrt(float(hd))
        e = torch.exp(scores - scores.max())
        out[h] = ((e / e.sum())[:, None] * v[:, h // group]).sum(dim=0)
    return out


@pytest.mark.parametrize("lens,n_q,n_kv,hd,N", [
    ([4000], 32, 8, 64, 2048),                          # one row, 32 splits dealt out over four threads each
    ([1500, 40], 8, 2, 64, 96),                         # two rows, one of them with a single split's worth of keys
    ([600, 650, 700, 512, 513, 1, 300, 640], 32, 8, 64, 2064),   # the columns end inside a block of tiles
    ([150 + 40 * i for i in range(16)], 6, 2, 48, 160),  # 16 rows; the last stretch of k has fewer heads
    ([900, 100, 1000], 8, 2, 128, 528),
    ([700, 701], 4, 2, 80, 64),
    ([300, 301, 302], 4, 2, 112, 96),
    ([700], 3, 1, 32, 48),                              # one stretch of k with fewer heads than it could hold
    ([260, 500], 8, 4, 96, 112),
    ([520, 300, 900, 50], 34, 2, 16, 48),               # 16 heads of 16 to a stretch of k, the last stretch one block
    ([2000, 1800, 1900, 100, 2100], 24, 8, 128, 3072),  # three tiles per wavefront
    ([800, 900, 1000, 1100, 1200], 32, 8, 64, 6160)])   # four, and the last block of tiles not whole
def test_attention_join_project(ops, lens, n_q, n_kv, hd, N):
    """The join of the decode kernel's splits and the output projection as one kernel, against the
    join kernel followed by a 32-bit product of the joined rows, and against plain attention."""
    page, S, K = 16, len(lens), n_q * hd
    s = _paged_setup(ops, lens, n_q, n_kv, hd, page, torch.bfloat16, seed=61)
    last = torch.tensor([sum(lens[:i + 1]) - 1 for i in range(S)], device=DEV)
    q = s["q"][last].contiguous()
    i32 = dict(dtype=torch.int32, device=DEV)
    q_start, ctx = torch.arange(S + 1, **i32), torch.tensor([n - 1 for n in lens], **i32)
    plan = ops.mfma.plan_attention([1] * S, [n - 1 for n in lens], n_q, n_kv, hd)
    assert plan["nsplit"] > 1
    g = torch.Generator().manual_seed(62)
    w = (torch.randn(N, K, generator=g) / math.sqrt(K)).bfloat16()
    base = torch.randn(S, N, generator=g)
    wd = ops.block_weight(w.to(DEV))
    scale = 1.0 / math.sqrt(hd)

    def parts():
        return (torch.full((S * n_q * plan["nsplit"] * hd,), float("nan"), device=DEV),
                torch.full((S * n_q * plan["nsplit"] * 2,), float("nan"), device=DEV))
    part_o, part_ml = parts()
    o = torch.zeros_like(q)
    ops.mfma.attention_bf16(q, s["k_cache"], s["v_cache"], o, q_start, ctx, s["table"], n_q, n_kv, hd, scale, 0, plan,
                            part_o, part_ml)
    apart = base.double() + o.cpu().double() @ w.double().T
    part_o2, part_ml2 = parts()
    o2 = torch.zeros_like(q)
    ops.mfma.attention_bf16(q, s["k_cache"], s["v_cache"], o2, q_start, ctx, s["table"], n_q, n_kv, hd, scale, 0,
                            dict(plan, tuning=ops.mfma.TUNING_NO_JOIN), part_o2, part_ml2)
    assert not o2.any()                                  # left unjoined: nothing wrote the rows
    out = base.to(DEV)
    ops.mfma.attention_join_project(part_o2, part_ml2, wd, out, S, n_q, hd, plan["nsplit"])
    assert _rel(out.cpu().double(), apart) < 1e-4
    ref = torch.cat([_plain_attention_last_row(qq, kk, vv).reshape(1, K) for (qq, kk, vv) in s["plain"]])
    assert _rel(out.cpu().double(), base.double() + ref @ w.double().T) < 8e-3


@pytest.mark.parametrize("lens,n_q,n_kv,hd,page,window", [
    ([1, 2, 17, 33, 64, 65, 300, 77, 129] * 2, 32, 8, 64, 16, 0),
    ([40 + 7 * i for i in range(24)], 24, 8, 128, 16, 0),
    ([5, 90, 200, 31, 32, 33] * 3, 8, 8, 64, 32, 0),          # one query head per kv head, pages of 32
    ([20 + 5 * i for i in range(20)], 16, 1, 128, 64, 0),      # 16 query heads on one kv head
    ([30, 100, 120, 61] * 5, 8, 2, 64, 16, 48)])               # a window
def test_attention_decode_with_rotation_inside(ops, lens, n_q, n_kv, hd, page, window):
    """Decoded tokens whose q/k/v rows are still 32-bit and unrotated: the attention kernel rotates, writes
    key and value into the pages, attends and clears the rows. Against the rotation kernel followed by
    the decode kernel (same pages afterwards, same output) and against plain attention."""
    import types
    S, T = len(lens), sum(lens)
    g = _gen(71)
    width = (n_q + 2 * n_kv) * hd
    qkv = torch.randn(T, width, generator=g)
    half = hd // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(max(lens) + 3, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    nblk = [(n + page - 1) // page for n in lens]
    total_pages = sum(nblk) + 2
    perm = torch.randperm(total_pages, generator=g).tolist()
    table = torch.zeros(S, max(nblk), dtype=torch.int32)
    p = 0
    for s_, nb in enumerate(nblk):
        for b in range(nb):
            table[s_, b] = perm[p]
            p += 1
    table = table.to(DEV)
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32)
    seq_idx = torch.cat([torch.full((n,), s_) for s_, n in enumerate(lens)]).to(torch.int32)
    last = torch.tensor([sum(lens[:i + 1]) - 1 for i in range(S)])
    is_last = torch.zeros(T, dtype=torch.bool)
    is_last[last] = True

    def caches():
        return (torch.zeros(total_pages, n_kv, page, hd, dtype=torch.bfloat16, device=DEV),
                torch.zeros(total_pages, n_kv, hd, page, dtype=torch.bfloat16, device=DEV))
    i32 = dict(dtype=torch.int32, device=DEV)
    q_start, ctx = torch.arange(S + 1, **i32), torch.tensor([n - 1 for n in lens], **i32)
    scale = 1.0 / math.sqrt(hd)
    # apart: every token through the rotation kernel, then the decode kernel over the last ones
    k1, v1 = caches()
    q_all = torch.empty(T, n_q * hd, dtype=torch.bfloat16, device=DEV)
    ops.rope_kv_write(qkv.to(DEV), cos, sin, positions.to(DEV), seq_idx.to(DEV), table, q_all, k1, v1, n_q, n_kv, hd, hd)
    plan = ops.mfma.plan_attention([1] * S, [n - 1 for n in lens], n_q, n_kv, hd)
    assert plan["nsplit"] == 1
    apart = torch.zeros(S, n_q * hd, dtype=torch.bfloat16, device=DEV)
    ops.mfma.attention_bf16(q_all[last.to(DEV)].contiguous(), k1, v1, apart, q_start, ctx, table, n_q, n_kv, hd, scale,
                            window, plan)
    # together: the earlier tokens through the rotation kernel, the last ones raw
    k2, v2 = caches()
    before = ~is_last
    if before.any():
        ops.rope_kv_write(qkv[before].contiguous().to(DEV), cos, sin, positions[before].contiguous().to(DEV),
                          seq_idx[before].contiguous().to(DEV), table, torch.empty(int(before.sum()), n_q * hd,
                          dtype=torch.bfloat16, device=DEV), k2, v2, n_q, n_kv, hd, hd)
    raw = qkv[last].contiguous().to(DEV)
    step = types.SimpleNamespace(num_seqs=S, new_lens=[1] * S, ctx_lens=[n - 1 for n in lens], plan_len=None, extra={},
                                 q_start=q_start, ctx_len=ctx)
    out = torch.zeros(S, n_q * hd, dtype=torch.bfloat16, device=DEV)
    assert ops.mfma.attention_decode_rope(raw, cos, sin, k2, v2, out, step, table, n_q, n_kv, hd, scale, window)
    assert not raw.any(), "the rows are left zero"
    assert torch.equal(k1, k2) and torch.equal(v1, v2), "the pages hold what the rotation kernel writes"
    assert torch.equal(out, apart)
    # plain attention of the last rows
    rows = []
    for s_, n in enumerate(lens):
        blk = qkv[last[s_] - n + 1:last[s_] + 1].double()
        q = blk[:, :n_q * hd].reshape(n, n_q, hd)
        k = blk[:, n_q * hd:(n_q + n_kv) * hd].reshape(n, n_kv, hd)
        v = blk[:, (n_q + n_kv) * hd:].reshape(n, n_kv, hd)
        c = torch.cat([cos[:n].cpu(), cos[:n].cpu()], dim=1).double()
        sn = torch.cat([sin[:n].cpu(), sin[:n].cpu()], dim=1).double()
        q, k = plain_apply_rope(q, c, sn), plain_apply_rope(k, c, sn)
        lo = max(0, n - window) if window > 0 else 0
        rows.append(_plain_attention_last_row(q[lo:], k[lo:], v[lo:]).reshape(1, n_q * hd))
    assert _rel(out.cpu().double(), torch.cat(rows)) < 8e-3


def test_attention_join_project_refuses(ops):
    from llmengine.ops import KernelError
    w = ops.block_weight(torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(KernelError):                     # 17 rows
        ops.mfma.attention_join_project(torch.zeros(17 * 2 * 2 * 64, device=DEV), torch.zeros(17 * 2 * 2 * 2, device=DEV), w,
                                        torch.zeros(17, 64, device=DEV), 17, 2, 64, 2)
    with pytest.raises(KernelError):                     # scratch too small for the splits
        ops.mfma.attention_join_project(torch.zeros(2 * 2 * 64, device=DEV), torch.zeros(2 * 2 * 2, device=DEV), w,
                                        torch.zeros(1, 64, device=DEV), 1, 2, 64, 4)
    with pytest.raises(KernelError):                     # a projection that is not blocked
        ops.mfma.attention_join_project(torch.zeros(2 * 2 * 64, device=DEV), torch.zeros(2 * 2 * 2, device=DEV),
                                        torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV),
                                        torch.zeros(1, 64, device=DEV), 1, 2, 64, 2)


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(4, 2, 16, 16), (3, 1, 32, 16), (6, 2, 48, 32), (32, 8, 64, 16),
                                              (5, 5, 80, 16), (8, 2, 128, 16)])
def test_attention_mfma_prefill_and_mixed(ops, n_q, n_kv, hd, page):
    lens = [70, 2, 130, 17, 64, 200, 9]
    news = [70, 2, 35, 1, 64, 3, 1]                      # whole prompts, portions with context, decoded tokens
    out, ref, plan = _attn_case(ops, lens, news, n_q, n_kv, hd, page)
    assert plan["n_decode"] == 2 and plan["groups"] >= 5
    assert _rel(out, ref) < 8e-3


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(8, 2, 64, 16), (4, 2, 64, 48), (6, 2, 64, 32), (3, 3, 64, 16),
                                              (8, 2, 128, 16), (2, 1, 128, 32), (5, 5, 128, 16)])
@pytest.mark.parametrize("rows,shared", [(0, -1), (0, 2), (0, 3), (32, 0), (0, 0)])
def test_attention_prefill_shared_and_direct(ops, n_q, n_kv, hd, page, rows, shared):
    """The prefill kernel that shares K and V through LDS, for 4, 2 and 1 heads of a kv head per
    workgroup, spans that end inside a 64-key stretch, portions that start deep in a context,
    and the kernel without LDS at the same sizes."""
    lens = [330, 2, 131, 64, 517, 65, 9]
    news = [330, 2, 67, 64, 130, 3, 1]
    out, ref, plan = _attn_case(ops, lens, news, n_q, n_kv, hd, page, seed=61,
                                tuning=ops.mfma.attention_tuning(rows=rows, shared=shared))
    assert plan["n_decode"] == 1 and plan["groups"] >= 6
    assert _rel(out, ref) < 8e-3


@pytest.mark.parametrize("window", [1, 7, 64, 65, 200])
@pytest.mark.parametrize("n_q,n_kv", [(8, 2), (3, 3)])
def test_attention_prefill_shared_window(ops, window, n_q, n_kv):
    lens = [300, 70, 190]
    news = [140, 70, 2]
    out, ref, _ = _attn_case(ops, lens, news, n_q, n_kv, 64, 16, window=window, seed=62)
    assert _rel(out, ref) < 8e-3


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(8, 2, 64, 16), (6, 2, 64, 32), (3, 3, 64, 16), (8, 2, 128, 16),
                                              (5, 5, 128, 48)])
@pytest.mark.parametrize("splits,key_waves,run", [(2, -1, 1), (3, 2, 2), (7, 3, 1), (16, -1, 3), (4, -1, 5), (4, 3, 100)])
def test_attention_prefill_cut_keys(ops, n_q, n_kv, hd, page, splits, key_waves, run):
    """Prompt portions whose keys are cut into runs that a second kernel joins: runs that end
    inside a span's own rows, a last run that takes the rest, items with a single run beside items
    with several (and all of them single), whole prompts and decoded tokens beside them, with one
    and two wavefronts per tile."""
    lens = [700, 2, 131, 64, 517, 65, 9]
    news = [40, 2, 67, 64, 130, 3, 1]
    out, ref, plan = _attn_case(ops, lens, news, n_q, n_kv, hd, page, seed=63, prefill_splits=splits, prefill_run=run,
                                tuning=ops.mfma.attention_tuning(shared=key_waves))
    assert plan["n_decode"] == 1 and plan["prefill_splits"] == splits
    assert not out.isnan().any()
    assert _rel(out, ref) < 8e-3


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(8, 2, 64, 16), (12, 4, 64, 16), (6, 2, 128, 32), (6, 2, 48, 16)])
@pytest.mark.parametrize("splits,key_waves", [(1, -1), (3, -1), (4, 3), (2, 2)])
def test_attention_decoded_tokens_beside_prompt_portions(ops, n_q, n_kv, hd, page, splits, key_waves):
    """A step with decoded tokens far into their requests (their keys cut into several splits) and
    prompt portions (their keys whole or cut into runs): where the prompt kernel shares K and V
    through LDS, one launch holds both kinds of work and one launch both joins; head size 48 takes
    the separate kernels."""
    lens = [900, 700, 1300, 2, 640, 33, 257]
    news = [1, 40, 1, 2, 1, 1, 130]
    out, ref, plan = _attn_case(ops, lens, news, n_q, n_kv, hd, page, seed=66, prefill_splits=splits if hd != 48 else None,
                                prefill_run=3, tuning=ops.mfma.attention_tuning(shared=key_waves))
    assert plan["n_decode"] == 4 and plan["nsplit"] > 1
    assert not out.isnan().any()
    assert _rel(out, ref) < 8e-3


@pytest.mark.parametrize("window", [1, 64, 65, 200])
def test_attention_prefill_cut_keys_window(ops, window):
    out, ref, _ = _attn_case(ops, [600, 70, 190], [140, 70, 2], 8, 2, 64, 16, window=window, seed=64, prefill_splits=4,
                             prefill_run=2)
    assert not out.isnan().any()
    assert _rel(out, ref) < 8e-3


def test_attention_prefill_cut_keys_by_plan(ops):
    """A short portion far into a prompt: the plan cuts its keys by itself."""
    n_q, n_kv, hd, page = 8, 2, 64, 16
    lens, news = [2100], [48]
    out, ref, plan = _attn_case(ops, lens, news, n_q, n_kv, hd, page, seed=65)
    assert plan["prefill_splits"] > 1                    # the plan cuts this one by itself
    assert _rel(out, ref) < 8e-3


def test_attention_plan_cuts_only_few_rows_over_many_keys(ops):
    plan = ops.mfma.plan_attention([256], [16128], 32, 8, 64)
    assert plan["prefill_splits"] == 8
    assert ops.mfma.plan_attention([1024], [15360], 32, 8, 128)["prefill_splits"] == 1  # one item per compute unit
    plan = ops.mfma.plan_attention([512], [15872], 32, 8, 128)
    assert (plan["prefill_splits"], plan["prefill_run"]) == (4, 64)
    assert ops.mfma.plan_attention([2048], [0], 32, 8, 64)["prefill_splits"] == 1       # many items
    assert ops.mfma.plan_attention([64], [300], 32, 8, 64)["prefill_splits"] == 1       # few keys
    assert ops.mfma.plan_attention([64], [3000], 6, 2, 48)["prefill_splits"] == 1       # a head size without the kernel
    assert ops.mfma.plan_attention([1, 1], [5000, 9000], 32, 8, 64)["prefill_splits"] == 1
    # more than a quarter of an item per compute unit: whole keys (in items of half the rows) until the keys are long
    for rows, behind, cut in ((512, 1024, False), (512, 4096, False), (512, 8192, True), (320, 2048, False),
                              (320, 8192, True), (256, 4096, True), (256, 8192, True), (768, 8192, False),
                              (768, 16384, True), (896, 32768, False)):
        plan = ops.mfma.plan_attention([rows, 1, 1], [behind, 700, 900], 32, 8, 64)
        assert (plan["prefill_splits"] > 1) == cut, (rows, behind, plan)
        assert cut or plan["tuning"] & ops.mfma.TUNING_HALF_ROWS


@pytest.mark.parametrize("window", [1, 5, 16, 33, 100])
def test_attention_mfma_window(ops, window):
    lens = [150, 40, 90]
    news = [1, 40, 30]
    out, ref, _ = _attn_case(ops, lens, news, 4, 2, 32, 16, window=window)
    assert _rel(out, ref) < 8e-3


def test_attention_mfma_finds_one_far_key(ops):
    """One early key is made to dominate (its query-key score is far above the rest): the output
    must be that key's value row, for a decoded token and for a row of a prompt portion."""
    n_q, n_kv, hd, page = 4, 2, 64, 16
    lens, far = [400, 400], 37
    T = sum(lens)
    g = _gen(77)
    qkv = 0.1 * torch.randn(T, (n_q + 2 * n_kv) * hd, generator=g)
    for base in (0, 400):
        qkv[base + 399, :n_q * hd] = 0.0
        qkv[base + 399, :n_q * hd:hd] = 8.0                          # every head of the last query: e_0 * 8
        qkv[base + far, n_q * hd:(n_q + n_kv) * hd:hd] = 8.0         # key `far`: e_0 * 8 -> score 64 / 8
    i32 = dict(dtype=torch.int32, device=DEV)
    nblk = 400 // page
    table = torch.arange(2 * nblk, dtype=torch.int32).view(2, nblk)
    positions = torch.cat([torch.arange(400), torch.arange(400)]).to(torch.int32)
    seq_idx = torch.cat([torch.zeros(400), torch.ones(400)]).to(torch.int32)
    k_cache = torch.zeros(2 * nblk, n_kv, page, hd, dtype=torch.bfloat16, device=DEV)
    v_cache = torch.zeros(2 * nblk, n_kv, hd, page, dtype=torch.bfloat16, device=DEV)
    q_all = torch.empty(T, n_q * hd, dtype=torch.bfloat16, device=DEV)
    ops.rope_kv_write(qkv.to(DEV), None, None, positions.to(DEV), seq_idx.to(DEV), table.to(DEV), q_all, k_cache,
                      v_cache, n_q, n_kv, hd, hd)
    rows = [399] + list(range(400 + 390, 800))                       # request 0 decodes, request 1 brings 10 rows
    q = q_all[torch.tensor(rows, device=DEV)].contiguous()
    out = torch.zeros_like(q)
    plan = ops.mfma.plan_attention([1, 10], [399, 390], n_q, n_kv, hd)
    part_o = torch.empty(2 * n_q * plan["nsplit"] * hd, device=DEV)
    part_ml = torch.empty(2 * n_q * plan["nsplit"] * 2, device=DEV)
    v = qkv[:, (n_q + n_kv) * hd:].to(torch.bfloat16).double().view(T, n_kv, hd)
    # whole, and with the portion's keys cut into runs of 128: the far key lies in the first run,
    # the rows' own keys in the last
    for splits, run in ((1, 1), (4, 2)):
        plan["prefill_splits"], plan["prefill_run"] = splits, run
        pre_o = torch.full((len(rows) * n_q * splits * hd,), float("nan"), device=DEV)
        pre_ml = torch.full((len(rows) * n_q * splits * 2,), float("nan"), device=DEV)
        out.zero_()
        ops.mfma.attention_bf16(q, k_cache, v_cache, out, torch.tensor([0, 1, 11], **i32),
                                torch.tensor([399, 390], **i32), table.to(DEV), n_q, n_kv, hd, 1.0, 0, plan, part_o,
                                part_ml, pre_o, pre_ml)
        for row, base in ((0, 0), (10, 400)):
            for h in range(n_q):
                got = out[row].cpu().double().view(n_q, hd)[h]
                assert (got - v[base + far, h // 2]).abs().max() < 2e-2, (splits, row, h)
    # cut keys need their scratch, and a head size that the kernel with LDS takes
    from llmengine.ops import KernelError
    with pytest.raises(KernelError):
        ops.mfma.attention_bf16(q, k_cache, v_cache, out, torch.tensor([0, 1, 11], **i32),
                                torch.tensor([399, 390], **i32), table.to(DEV), n_q, n_kv, hd, 1.0, 0, plan, part_o,
                                part_ml, pre_o[:100], pre_ml)
    with pytest.raises(KernelError):
        ops.mfma.attention_bf16(q, k_cache, v_cache, out, torch.tensor([0, 1, 11], **i32),
                                torch.tensor([399, 390], **i32), table.to(DEV), n_q, n_kv, hd, 1.0, 0, plan, part_o,
                                part_ml)
    q32 = q.view(len(rows), 2 * n_q, 32).contiguous().view(len(rows), -1)      # the same bytes as heads of 32
    k32, v32 = k_cache.view(2 * nblk, 2 * n_kv, page, 32), v_cache.view(2 * nblk, 2 * n_kv, 32, page)
    with pytest.raises(KernelError):
        ops.mfma.attention_bf16(q32, k32, v32, out, torch.tensor([0, 1, 11], **i32), torch.tensor([399, 390], **i32),
                                table.to(DEV), 2 * n_q, 2 * n_kv, 32, 1.0, 0, plan, part_o, part_ml,
                                torch.empty(len(rows) * 2 * n_q * 4 * 32, device=DEV), pre_ml.repeat(2))


# --- projections fused with the norm in front of them -----------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (8, 3072, 2048), (16, 100, 96), (5, 331, 144), (3, 128256, 2048),
                                   (7, 64, 4096), (8, 5120, 3072), (9, 5120, 3072), (6, 6144, 4096)])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tpr,grid", [(0, 0), (1, 0), (2, 3), (4, 0), (4, 5)])
def test_gemv_norm(ops, M, N, K, wdtype, tpr, grid):
    if N > 10000 and (tpr, grid) not in ((0, 0), (4, 0)):
        pytest.skip("large case twice")
    if N > 4000 and K > 2048 and (tpr, grid) not in ((0, 0), (2, 3)):
        pytest.skip("large case twice")
    h = 2 * torch.randn(M + 3, K, generator=_gen(60))
    nw = (1 + 0.1 * torch.randn(K, generator=_gen(61))).to(wdtype)
    w = (0.05 * torch.randn(N, K, generator=_gen(62))).to(torch.bfloat16)
    rows = torch.tensor([(3 * i + 1) % (M + 3) for i in range(M)], dtype=torch.int32)
    out = torch.empty(M, N, device=DEV)
    ops.gemv_norm(h.to(DEV), nw.to(DEV), 1e-5, w.to(DEV), out, rows=rows.to(DEV), tiles_per_round=tpr, grid=grid)
    x = plain_rmsnorm(h[rows.long()].double(), nw.double(), 1e-5)
    ref = plain_linear(x, w.double())
    assert _rel(out.cpu().double(), ref) < 4e-3          # activations enter the product in bfloat16
    direct = torch.empty(M, N, device=DEV)
    ops.gemv_norm(h[:M].contiguous().to(DEV), nw.to(DEV), 1e-5, w.to(DEV), direct, tiles_per_round=tpr, grid=grid)
    ref2 = plain_linear(plain_rmsnorm(h[:M].double(), nw.double(), 1e-5), w.double())
    assert _rel(direct.cpu().double(), ref2) < 4e-3


@pytest.mark.parametrize("M,FF,K", [(1, 176, 64), (8, 8192, 2048), (16, 256, 96), (4, 208, 144)])
def test_gemv_norm_gated(ops, M, FF, K):
    h = 2 * torch.randn(M, K, generator=_gen(63))
    nw = (1 + 0.1 * torch.randn(K, generator=_gen(64))).to(torch.bfloat16)
    wg = (0.1 * torch.randn(FF, K, generator=_gen(65))).to(torch.bfloat16)
    wu = (0.1 * torch.randn(FF, K, generator=_gen(66))).to(torch.bfloat16)
    fused = torch.empty(2 * FF, K, dtype=torch.bfloat16)
    fused.view(FF // 16, 2, 16, K)[:, 0] = wg.view(FF // 16, 16, K)
    fused.view(FF // 16, 2, 16, K)[:, 1] = wu.view(FF // 16, 16, K)
    out = torch.empty(M, FF, dtype=torch.bfloat16, device=DEV)
    x = plain_rmsnorm(h.double(), nw.double(), 1e-6)
    ref = plain_silu(plain_linear(x, wg.double())) * plain_linear(x, wu.double())
    for tpr, grid in ((0, 0), (1, 0), (2, 2), (4, 0)):
        out.zero_()
        ops.gemv_norm(h.to(DEV), nw.to(DEV), 1e-6, fused.to(DEV), out, gated=True, tiles_per_round=tpr, grid=grid)
        assert _rel(out.cpu().double(), ref) < 1e-2, (tpr, grid)


@pytest.mark.parametrize("M,K", [(1, 64), (3, 2048), (8, 2048), (16, 2048), (1, 3072), (8, 3072), (8, 4096), (16, 4096),
                                 (2, 4104), (13, 1000)])
@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
def test_gemv_norm_rounds_what_the_norm_kernel_rounds(ops, M, K, wdtype):
    """A token's normed activations are rounded to the same bfloat16 values whether the norm is
    its own kernel (prompts) or part of the projection (decoding): the two ways then differ by the
    order of 32-bit sums only. (Scaling after the product instead of before the rounding is as
    accurate but differs from the norm kernel's result by a bfloat16 rounding, a thousand times more.)
    Rows are shared by several wavefronts, held in registers or read twice, depending on M and K."""
    h = 3 * torch.randn(M, K, generator=_gen(80))
    nw = (1 + 0.2 * torch.randn(K, generator=_gen(81))).to(wdtype)
    hd, nwd = h.to(DEV), nw.to(DEV)
    x = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    ops.rmsnorm(hd, nwd, 1e-5, x)
    # plain epilogue: few tiles (a workgroup of 8 wavefronts each)
    w = (0.05 * torch.randn(272, K, generator=_gen(82))).to(torch.bfloat16).to(DEV)
    fused, apart = torch.empty(M, 272, device=DEV), torch.empty(M, 272, device=DEV)
    ops.gemv_norm(hd, nwd, 1e-5, w, fused)
    ops.gemm(x, w, apart)
    # (the two kernels add the squares in another order: a scale that differs in its last bit moves
    # one value in some ten thousand across a rounding boundary, which is 1e-5 of a sum; rounding
    # before the scale would be 4e-3)
    assert _rel(fused.cpu().double(), apart.cpu().double()) < 1e-4
    # gated epilogue with more than 256 tiles: workgroups of 16 wavefronts
    FF = 4352
    wgu = (0.05 * torch.randn(2 * FF, K, generator=_gen(83))).to(torch.bfloat16).to(DEV)
    fused_g = torch.empty(M, FF, dtype=torch.bfloat16, device=DEV)
    apart_g = torch.empty(M, FF, dtype=torch.bfloat16, device=DEV)
    ops.gemv_norm(hd, nwd, 1e-5, wgu, fused_g, gated=True)
    ops.gemm_gated(x, wgu, apart_g, 16, lambda shape, dtype: torch.empty(shape, dtype=dtype, device=DEV))
    differ = (fused_g != apart_g).float().mean().item()
    # (sums that differ by 1e-5 put up to one output in a hundred on the other side of a rounding
    # boundary; with the activations rounded before the scale, every second output differs)
    assert differ < 0.05, differ
    assert _rel(fused_g.cpu().double(), apart_g.cpu().double()) < 8e-3


def test_gemv_norm_refusals(ops):
    from llmengine.ops import KernelError
    h = torch.randn(17, 64, device=DEV)
    nw = torch.ones(64, device=DEV)
    w = torch.randn(32, 64, device=DEV).bfloat16()
    with pytest.raises(KernelError):
        ops.gemv_norm(h, nw, 1e-5, w, torch.empty(17, 32, device=DEV))          # more than 16 rows
    with pytest.raises(KernelError):
        ops.gemv_norm(h[:4, :60].contiguous(), nw[:60].contiguous(), 1e-5, w[:, :60].contiguous(),
                      torch.empty(4, 32, device=DEV))                              # K no multiple of 8


@pytest.mark.parametrize("M,n_q,n_kv,hd,K,page", [(1, 4, 2, 32, 64, 16), (8, 32, 8, 64, 2048, 16), (16, 3, 1, 96, 96, 32),
                                                  (5, 6, 2, 128, 144, 16), (3, 40, 8, 64, 256, 64), (4, 5, 1, 48, 72, 16),
                                                  (2, 2, 2, 16, 40, 16), (7, 24, 8, 128, 512, 16),
                                                  (8, 24, 8, 128, 3072, 16), (11, 24, 8, 128, 3072, 16),
                                                  (5, 32, 8, 128, 4096, 16)])
@pytest.mark.parametrize("grid", [0, 3])
def test_gemv_norm_rope(ops, M, n_q, n_kv, hd, K, page, grid):
    """The fused kernel against its parts: norm, projection, rotation, cache write."""
    g = _gen(70)
    h = 2 * torch.randn(M, K, generator=g)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16)
    N = (n_q + 2 * n_kv) * hd
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    positions = torch.randint(0, 5 * page, (M,), generator=g).to(torch.int32)
    seq_idx = torch.arange(M, dtype=torch.int32)                  # one request per row
    table = torch.randperm(M * 5, generator=g).to(torch.int32).view(M, 5)
    half = hd // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(5 * page, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    k_cache = torch.zeros(M * 5, n_kv, page, hd, dtype=torch.bfloat16, device=DEV)
    v_cache = torch.zeros(M * 5, n_kv, hd, page, dtype=torch.bfloat16, device=DEV)
    q_out = torch.zeros(M, n_q * hd, dtype=torch.bfloat16, device=DEV)
    paired = ops.pair_rows_for_rotation(w, n_q + n_kv, hd)          # the kernel's own order of the q and k rows
    ops.gemv_norm_rope(h.to(DEV), nw.to(DEV), 1e-5, paired.to(DEV), positions.to(DEV), seq_idx.to(DEV), table.to(DEV),
                       cos.to(DEV), sin.to(DEV), q_out, k_cache, v_cache, n_q, n_kv, hd, grid=grid)
    x = plain_rmsnorm(h.double(), nw.double(), 1e-5)
    qkv = plain_linear(x, w.double())
    c = torch.cat([cos, cos], dim=1)[positions.long()].double()
    s_ = torch.cat([sin, sin], dim=1)[positions.long()].double()
    q_ref = plain_apply_rope(qkv[:, :n_q * hd].reshape(M, n_q, hd), c, s_).reshape(M, -1)
    k_ref = plain_apply_rope(qkv[:, n_q * hd:(n_q + n_kv) * hd].reshape(M, n_kv, hd), c, s_)
    v_ref = qkv[:, (n_q + n_kv) * hd:].reshape(M, n_kv, hd)
    assert _rel(q_out.cpu().double(), q_ref) < 8e-3
    kc, vc = k_cache.cpu().double(), v_cache.cpu().double()
    scale = qkv.abs().max()
    for m in range(M):
        pos = int(positions[m])
        pg, off = int(table[m, pos // page]), pos % page
        assert (kc[pg, :, off, :] - k_ref[m]).abs().max() < 8e-3 * scale
        assert (vc[pg, :, :, off] - v_ref[m]).abs().max() < 8e-3 * scale
    assert int((kc != 0).sum()) <= M * n_kv * hd and int((vc != 0).sum()) <= M * n_kv * hd   # nothing else written


@pytest.mark.parametrize("n_q,n_kv,hd,page", [(4, 2, 64, 16), (3, 1, 128, 48), (6, 3, 80, 32), (2, 2, 16, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("new", [[40, 50, 3, 16, 33], [104, 114, 3, 48, 65]])     # a workgroup per token; 16 tokens per workgroup
def test_rope_write_of_many_tokens(ops, n_q, n_kv, hd, page, dtype, new):
    """Rotation and cache write for a step of many tokens (16 tokens per workgroup, v written in
    pieces of 16 positions where they lie together in a page): portions that start at multiples
    of 16, portions that do not, a request shorter than a group, and groups that span two
    requests. Every written place of both caches is compared, and no other place is touched."""
    ctx = [32, 5, 0, 48, 16]                      # tokens already cached
    T, S = sum(new), len(new)
    g = _gen(71)
    qkv = torch.randn(T, (n_q + 2 * n_kv) * hd, generator=g)
    half = hd // 2
    max_pos = max(c + n for c, n in zip(ctx, new))
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float(), torch.sin(ang).float()
    nblk = [(c + n + page - 1) // page for c, n in zip(ctx, new)]
    total_pages = sum(nblk) + 3
    perm = torch.randperm(total_pages, generator=g).tolist()
    table = torch.zeros(S, max(nblk), dtype=torch.int32)
    p = 0
    for s, nb in enumerate(nblk):
        for b in range(nb):
            table[s, b] = perm[p]
            p += 1
    positions = torch.cat([torch.arange(c, c + n) for c, n in zip(ctx, new)]).to(torch.int32)
    seq_idx = torch.cat([torch.full((n,), s) for s, n in enumerate(new)]).to(torch.int32)
    mark = 7.0                                    # what the caches hold before
    k_cache = torch.full((total_pages, n_kv, page, hd), mark, dtype=dtype, device=DEV)
    v_cache = torch.full((total_pages, n_kv, hd, page), mark, dtype=dtype, device=DEV)
    q_out = torch.empty(T, n_q * hd, dtype=dtype, device=DEV)
    ops.rope_kv_write(qkv.to(DEV), cos.to(DEV), sin.to(DEV), positions.to(DEV), seq_idx.to(DEV), table.to(DEV),
                      q_out, k_cache, v_cache, n_q, n_kv, hd, hd)
    blk = qkv.double()
    c2 = torch.cat([cos[positions.long()], cos[positions.long()]], dim=1).double()
    s2 = torch.cat([sin[positions.long()], sin[positions.long()]], dim=1).double()
    q = plain_apply_rope(blk[:, :n_q * hd].reshape(T, n_q, hd), c2, s2)
    k = plain_apply_rope(blk[:, n_q * hd:(n_q + n_kv) * hd].reshape(T, n_kv, hd), c2, s2)
    v = blk[:, (n_q + n_kv) * hd:].reshape(T, n_kv, hd)
    tol = 2e-6 if dtype == torch.float32 else 4e-3
    assert _rel(q_out.cpu().double(), q.reshape(T, -1)) < tol
    k_ref = torch.full(k_cache.shape, mark, dtype=torch.float64)
    v_ref = torch.full(v_cache.shape, mark, dtype=torch.float64)
    for t in range(T):
        pos, s = int(positions[t]), int(seq_idx[t])
        pg, off = int(table[s, pos // page]), pos % page
        k_ref[pg, :, off, :] = k[t]
        v_ref[pg, :, :, off] = v[t]
    assert float((k_cache.cpu().double() - k_ref).abs().max()) < tol * 8
    assert float((v_cache.cpu().double() - v_ref).abs().max()) < tol * 8


@pytest.mark.parametrize("n_q,n_kv,hd,K,page", [(4, 2, 64, 128, 16), (32, 8, 64, 2048, 16), (3, 1, 128, 96, 32), (5, 3, 32, 72, 16),
                                                 (6, 2, 16, 64, 48), (24, 8, 128, 512, 16)])
@pytest.mark.parametrize("new", [[70, 130, 3, 16, 33], [300], [1, 90, 17]])
@pytest.mark.parametrize("tile", [0, 64, 128, 128064, 96064, 96128])
def test_gemm_qkv_rope(ops, n_q, n_kv, hd, K, page, new, tile):
    """The q/k/v projection with rotation and cache write in its epilogue against the three kernels
    it replaces (product into 32-bit rows, rotation + cache write): portions that start anywhere in
    their requests, groups of 16 rows that span two requests or two pages, tiles that hang over the
    rows and over the heads, row-major and blocked weights."""
    if tile in (64, 128064, 96064) and hd > 64:
        pytest.skip("a 64-column tile does not hold a head of 128")
    g = _gen(90)
    T = sum(new)
    N = (n_q + 2 * n_kv) * hd
    x = torch.randn(T, K, generator=g).to(torch.bfloat16)
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16)
    ctx = [int(c) for c in torch.randint(0, 3 * page, (len(new),), generator=g)]       # tokens cached before
    ctx[0] = 16                                                                          # one portion starts at a multiple of 16
    positions = torch.cat([torch.arange(c, c + n) for c, n in zip(ctx, new)]).to(torch.int32)
    seq_idx = torch.cat([torch.full((n,), s) for s, n in enumerate(new)]).to(torch.int32)
    blocks = [(c + n + page - 1) // page for c, n in zip(ctx, new)]
    perm = torch.randperm(sum(blocks) + 2, generator=g).tolist()
    table = torch.zeros(len(new), max(blocks), dtype=torch.int32)
    p = 0
    for s, nb in enumerate(blocks):
        for b in range(nb):
            table[s, b] = perm[p]
            p += 1
    max_pos = max(c + n for c, n in zip(ctx, new))
    inv = 1.0 / (10000.0 ** (torch.arange(hd // 2, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    pages = sum(blocks) + 2

    def fresh():
        return (torch.zeros(T, n_q * hd, dtype=torch.bfloat16, device=DEV),
                torch.zeros(pages, n_kv, page, hd, dtype=torch.bfloat16, device=DEV),
                torch.zeros(pages, n_kv, hd, page, dtype=torch.bfloat16, device=DEV))
    xd, pd, sd, td = x.to(DEV), positions.to(DEV), seq_idx.to(DEV), table.to(DEV)
    q0, k0, v0 = fresh()
    qkv = torch.empty(T, N, device=DEV)
    ops.gemm(xd, w.to(DEV), qkv)
    ops.rope_kv_write(qkv, cos, sin, pd, sd, td, q0, k0, v0, n_q, n_kv, hd, hd)
    for wd in ([w.to(DEV)] + ([ops.block_weight(w.to(DEV))] if K % 32 == 0 else [])):
        q1, k1, v1 = fresh()
        ops.gemm_qkv_rope(xd, wd, cos, sin, pd, sd, td, q1, k1, v1, n_q, n_kv, hd, tile=tile)
        for got, want in ((q1, q0), (k1, k0), (v1, v0)):
            # (the same sums; the rotation may contract a product and a difference into one rounding)
            assert (got.float() - want.float()).abs().max() <= 1.6e-2 * want.float().abs().max()
            assert ((got != want).float().mean()) < 2e-3
            assert torch.equal(got == 0, want == 0)            # nothing else was written
