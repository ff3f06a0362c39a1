"""The blocked weight layout of the matrix kernels: where an element lies, and every kernel
that reads weights with the blocked copy against the same kernel with the row-major matrix
(the same sums in the same order, so equal bit for bit unless parts are joined by atomic
additions) and against the plain product."""
import math

import pytest
import torch

from plain_llama import plain_apply_rope, plain_linear, plain_rmsnorm, plain_silu

DEV = "cuda:0"


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


@pytest.fixture(scope="module")
def ops():
    from llmengine import ops
    return ops


def test_where_an_element_lies(ops):
    N, K = 48, 96
    w = torch.arange(N * K, dtype=torch.float32).view(N, K).to(torch.bfloat16)
    b = ops.block_weight(w)
    assert tuple(b.shape) == (3, 3, 4, 16, 8) and b.is_contiguous() and ops.is_blocked(b)
    assert ops.weight_shape(b) == (N, K) and ops.weight_shape(w) == (N, K)
    for n, k in [(0, 0), (1, 0), (0, 8), (17, 40), (47, 95), (16, 31), (15, 32)]:
        assert b[n // 16, k // 32, (k % 32) // 8, n % 16, k % 8] == w[n, k]
    # a wavefront's lane l = 16 q + r reads bytes 16 l .. 16 l + 15 of a block: row r, k = 8 q .. 8 q + 7
    flat = b[1, 2].reshape(64, 8)
    for lane in (0, 5, 16, 63):
        r, q = lane % 16, lane // 16
        assert torch.equal(flat[lane], w[16 + r, 64 + 8 * q:64 + 8 * q + 8])
    assert torch.equal(ops.unblock_weight(b), w)
    assert torch.equal(ops.unblock_weight(b[:2]), w[:32])            # row groups are slices
    from llmengine.ops import KernelError
    for bad in (w[:40], w[:, :72].contiguous(), w.float()):
        assert not ops.can_block(bad)
        with pytest.raises(KernelError):
            ops.block_weight(bad)


def test_rows_paired_for_rotation(ops):
    """Within a rotated head: dims 0 .. 7, their partners hd/2 .. hd/2 + 7, then 8 .. 15 and so on."""
    n_q, n_kv, hd, K = 2, 1, 32, 8
    w = torch.arange((n_q + 2 * n_kv) * hd, dtype=torch.float32)[:, None].repeat(1, K)     # row n holds n
    got = ops.pair_rows_for_rotation(w, n_q + n_kv, hd)[:, 0].tolist()
    head = list(range(0, 8)) + list(range(16, 24)) + list(range(8, 16)) + list(range(24, 32))
    want = [h * hd + d for h in range(n_q + n_kv) for d in head] + list(range((n_q + n_kv) * hd, (n_q + 2 * n_kv) * hd))
    assert got == want
    same = ops.pair_rows_for_rotation(w[:, :8].contiguous(), 0, hd)
    assert torch.equal(same, w[:, :8])
    assert torch.equal(ops.pair_rows_for_rotation(torch.arange(64.)[:, None].repeat(1, 8), 4, 16)[:, 0], torch.arange(64.))
    from llmengine.ops import KernelError
    with pytest.raises(KernelError):
        ops.pair_rows_for_rotation(w, 3, 24)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 2048, 2048), (8, 3072, 2048), (16, 48, 96), (33, 96, 96), (64, 2048, 8192),
                                   (50, 128, 992), (3, 16, 32)])
def test_skinny_product(ops, M, N, K):
    ops.library()
    a = torch.randn(M, K, generator=_gen(1)).to(torch.bfloat16).to(DEV)
    w = torch.randn(N, K, generator=_gen(2)).to(torch.bfloat16).to(DEV)
    wb = ops.block_weight(w)
    ref = a.double() @ w.double().T
    for waves in (0, 4, 8, 16):
        out, outb = torch.empty(M, N, device=DEV), torch.empty(M, N, device=DEV)
        ops.gemm_bf16(a, w, out, waves=waves)
        ops.gemm_bf16(a, wb, outb, waves=waves)
        assert torch.equal(out, outb), waves
        assert _rel(outb, ref) < 2e-5
    base = torch.randn(M, N, generator=_gen(3)).to(DEV)
    for ksplit in (0, 3):
        acc = base.clone()
        ops.gemm_bf16(a, wb, acc, accumulate=True, ksplit=ksplit)
        assert _rel(acc, ref + base.double()) < 2e-5, ksplit
    half = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a, wb, half)
    assert _rel(half, ref) < 5e-3
    plain = torch.empty(M, N, device=DEV)
    ops.gemm_generic(a, wb, plain)                                    # the plain-precision kernel reads it too
    assert _rel(plain, ref) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(65, 128, 64), (128, 128, 128), (200, 336, 160), (129, 112, 96), (257, 496, 32),
                                   (2048, 3072, 2048), (1000, 2048, 8192), (7, 48, 224)])
@pytest.mark.parametrize("tile", [64, 128, 128096, 128064])
def test_tile_product(ops, M, N, K, tile):
    ops.library()
    a = torch.randn(M, K, generator=_gen(4)).to(torch.bfloat16).to(DEV)
    w = torch.randn(N, K, generator=_gen(5)).to(torch.bfloat16).to(DEV)
    wb = ops.block_weight(w)
    ref = a.double() @ w.double().T
    out, outb = torch.empty(M, N, device=DEV), torch.full((M, N), 3.0, device=DEV)
    ops.gemm_bf16(a, w, out, tile=tile)
    ops.gemm_bf16(a, wb, outb, tile=tile)
    assert torch.equal(out, outb)
    assert _rel(outb, ref) < 2e-5
    base = torch.randn(M, N, generator=_gen(6)).to(DEV)
    for ksplit in (0, 2, 5):
        acc = base.clone()
        ops.gemm_bf16(a, wb, acc, accumulate=True, tile=tile, ksplit=ksplit)
        assert _rel(acc, ref + base.double()) < 2e-5, ksplit
    half = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(a, wb, half, tile=tile)
    assert _rel(half, ref) < 5e-3


def _interleaved(wg, wu):
    FF, K = wg.shape
    fused = torch.empty(2 * FF, K, dtype=wg.dtype)
    fused.view(FF // 16, 2, 16, K)[:, 0] = wg.view(FF // 16, 16, K)
    fused.view(FF // 16, 2, 16, K)[:, 1] = wu.view(FF // 16, 16, K)
    return fused


@pytest.mark.gpu
@pytest.mark.parametrize("T,FF,K,tile", [(5, 176, 64, 0), (130, 256, 96, 64), (300, 208, 160, 128),
                                         (2048, 8192, 2048, 0), (257, 320, 128, 128096), (190, 352, 96, 128064),
                                         (64, 8192, 2048, 0)])
def test_gated_product(ops, T, FF, K, tile):
    ops.library()
    x = torch.randn(T, K, generator=_gen(7)).to(torch.bfloat16)
    wg = (0.1 * torch.randn(FF, K, generator=_gen(8))).to(torch.bfloat16)
    wu = (0.1 * torch.randn(FF, K, generator=_gen(9))).to(torch.bfloat16)
    fused = _interleaved(wg, wu).to(DEV)
    out = torch.zeros(T, FF, dtype=torch.bfloat16, device=DEV)
    outb = torch.zeros(T, FF, dtype=torch.bfloat16, device=DEV)
    ops.gemm_bf16(x.to(DEV), fused, out, gated=True, tile=tile)
    ops.gemm_bf16(x.to(DEV), ops.block_weight(fused), outb, gated=True, tile=tile)
    assert torch.equal(out, outb)
    ref = plain_silu(x.double() @ wg.double().T) * (x.double() @ wu.double().T)
    assert _rel(outb, ref) < 5e-3


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 48, 64), (8, 3072, 2048), (16, 96, 96), (5, 336, 160), (3, 128256, 2048),
                                   (7, 64, 4096)])
@pytest.mark.parametrize("tpr,grid", [(0, 0), (1, 0), (2, 3), (4, 0), (4, 5), (12, 0)])
def test_norm_and_product(ops, M, N, K, tpr, grid):
    if N > 10000 and (tpr, grid) not in ((0, 0), (4, 0)):
        pytest.skip("large case twice")
    ops.library()
    h = (2 * torch.randn(M + 3, K, generator=_gen(10))).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=_gen(11))).to(torch.bfloat16).to(DEV)
    w = (0.05 * torch.randn(N, K, generator=_gen(12))).to(torch.bfloat16).to(DEV)
    rows = torch.tensor([(3 * i + 1) % (M + 3) for i in range(M)], dtype=torch.int32, device=DEV)
    out, outb = torch.empty(M, N, device=DEV), torch.empty(M, N, device=DEV)
    ops.gemv_norm(h, nw, 1e-5, w, out, rows=rows, tiles_per_round=tpr, grid=grid)
    ops.gemv_norm(h, nw, 1e-5, ops.block_weight(w), outb, rows=rows, tiles_per_round=tpr, grid=grid)
    assert torch.equal(out, outb)
    x = plain_rmsnorm(h[rows.long()].double().cpu(), nw.double().cpu(), 1e-5)
    assert _rel(outb.cpu(), plain_linear(x, w.double().cpu())) < 4e-3


@pytest.mark.gpu
@pytest.mark.parametrize("M,FF,K", [(1, 176, 64), (8, 8192, 2048), (16, 256, 96), (4, 208, 160)])
def test_norm_and_gated_product(ops, M, FF, K):
    ops.library()
    h = (2 * torch.randn(M, K, generator=_gen(13))).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=_gen(14))).to(torch.bfloat16).to(DEV)
    wg = (0.1 * torch.randn(FF, K, generator=_gen(15))).to(torch.bfloat16)
    wu = (0.1 * torch.randn(FF, K, generator=_gen(16))).to(torch.bfloat16)
    fused = _interleaved(wg, wu).to(DEV)
    x = plain_rmsnorm(h.double().cpu(), nw.double().cpu(), 1e-6)
    ref = plain_silu(plain_linear(x, wg.double())) * plain_linear(x, wu.double())
    for tpr, grid in ((0, 0), (1, 0), (2, 2), (4, 0)):
        out = torch.zeros(M, FF, dtype=torch.bfloat16, device=DEV)
        outb = torch.zeros(M, FF, dtype=torch.bfloat16, device=DEV)
        ops.gemv_norm(h, nw, 1e-6, fused, out, gated=True, tiles_per_round=tpr, grid=grid)
        ops.gemv_norm(h, nw, 1e-6, ops.block_weight(fused), outb, gated=True, tiles_per_round=tpr, grid=grid)
        assert torch.equal(out, outb), (tpr, grid)
        assert _rel(outb.cpu(), ref) < 1e-2, (tpr, grid)


@pytest.mark.gpu
@pytest.mark.parametrize("M,n_q,n_kv,hd,K,page", [(1, 4, 2, 32, 64, 16), (8, 32, 8, 64, 2048, 16), (16, 3, 1, 96, 96, 32),
                                                  (5, 6, 2, 128, 160, 16), (3, 40, 8, 64, 256, 64)])
@pytest.mark.parametrize("grid", [0, 3])
def test_norm_product_rotation_and_cache_write(ops, M, n_q, n_kv, hd, K, page, grid):
    ops.library()
    g = _gen(17)
    h = (2 * torch.randn(M, K, generator=g)).to(DEV)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16).to(DEV)
    N = (n_q + 2 * n_kv) * hd
    w = (0.05 * torch.randn(N, K, generator=g)).to(torch.bfloat16).to(DEV)
    positions = torch.randint(0, 5 * page, (M,), generator=g).to(torch.int32).to(DEV)
    seq_idx = torch.arange(M, dtype=torch.int32, device=DEV)
    table = torch.randperm(M * 5, generator=g).to(torch.int32).view(M, 5).to(DEV)
    half = hd // 2
    inv = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) * 2 / hd))
    ang = torch.arange(5 * page, dtype=torch.float64)[:, None] * inv[None, :]
    cos, sin = torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)
    got = []
    paired = ops.pair_rows_for_rotation(w, n_q + n_kv, hd)
    for weight in (paired, ops.block_weight(paired)):
        k_cache = torch.zeros(M * 5, n_kv, page, hd, dtype=torch.bfloat16, device=DEV)
        v_cache = torch.zeros(M * 5, n_kv, hd, page, dtype=torch.bfloat16, device=DEV)
        q_out = torch.zeros(M, n_q * hd, dtype=torch.bfloat16, device=DEV)
        ops.gemv_norm_rope(h, nw, 1e-5, weight, positions, seq_idx, table, cos, sin, q_out, k_cache, v_cache,
                           n_q, n_kv, hd, grid=grid)
        got.append((q_out, k_cache, v_cache))
    for plain_t, blocked_t in zip(*got):
        assert torch.equal(plain_t, blocked_t)
    x = plain_rmsnorm(h.double().cpu(), nw.double().cpu(), 1e-5)
    qkv = plain_linear(x, w.double().cpu())
    c = torch.cat([cos, cos], dim=1)[positions.long()].double().cpu()
    s_ = torch.cat([sin, sin], dim=1)[positions.long()].double().cpu()
    q_ref = plain_apply_rope(qkv[:, :n_q * hd].reshape(M, n_q, hd), c, s_).reshape(M, -1)
    assert _rel(got[1][0].cpu(), q_ref) < 8e-3


@pytest.mark.gpu
@pytest.mark.parametrize("V,H", [(48, 96), (128256, 2048), (64, 32)])
def test_rows_of_a_blocked_table(ops, V, H):
    ops.library()
    table = torch.randn(V, H, generator=_gen(18)).to(torch.bfloat16)
    tokens = torch.tensor([0, 1, 7, V - 1, 17, 17, V // 2], dtype=torch.int32)
    out = torch.empty(len(tokens), H, dtype=torch.float32, device=DEV)
    ops.embed_gather(ops.block_weight(table.to(DEV)), tokens.to(DEV), out)
    assert torch.equal(out.cpu(), table[tokens.long()].float())
