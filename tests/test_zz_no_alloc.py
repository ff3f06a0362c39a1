"""The decode attention entry point that allocates nothing, called through ctypes as a caller
without torch would: its output against the existing entry point's (same kernels, the splits'
partial results in a workspace that the caller brings) and against the plain attention, on two
calls in a row, the second with a smaller input that finds the first call's leftovers in the
library's fixed array."""
import ctypes
import math

import pytest
import torch

from plain_llama import plain_attention

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

_vp, _i, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


@pytest.fixture(scope="module")
def lib():
    from llmengine.ops import build
    path = build.ensure_built()
    lib = ctypes.CDLL(path)
    lib.llme_noalloc_init.argtypes = []
    lib.llme_noalloc_init.restype = _i
    lib.llme_attention_decode_noalloc_scratch_floats.argtypes = [_i, _i, _i, _i]
    lib.llme_attention_decode_noalloc_scratch_floats.restype = ctypes.c_long
    lib.llme_attention_decode_noalloc.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i,
                                                  _i, _i, _vp]
    lib.llme_attention_decode_noalloc.restype = _i
    lib.llme_attention_bf16.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i,
                                        _i, _i, _i, _i, _vp, _i, _i, _i, _vp, _vp, _i, _vp]
    lib.llme_attention_bf16.restype = _i
    return lib


def _case(lens, n_q, n_kv, hd, page, seed):
    """Requests of the given lengths in scrambled pages; the step's token is each request's last."""
    import llmengine.ops as ops
    from test_kernels_gpu import _paged_setup
    s = _paged_setup(ops, lens, n_q, n_kv, hd, page, torch.bfloat16, seed=seed)
    last_rows, base = [], 0
    for n in lens:
        last_rows.append(base + n - 1)
        base += n
    q = s["q"][torch.tensor(last_rows, device=DEV)].contiguous()
    i32 = dict(dtype=torch.int32, device=DEV)
    q_start = torch.arange(len(lens) + 1, **i32)
    ctx_len = torch.tensor([n - 1 for n in lens], **i32)
    ref = torch.cat([plain_attention(qq, kk, vv)[n - 1:].reshape(1, n_q * hd) for (qq, kk, vv), n in zip(s["plain"], lens)])
    return s, q, q_start, ctx_len, ref


def _run_both(lib, lens, n_q, n_kv, hd, page, split_len, nsplit, seed):
    s, q, q_start, ctx_len, ref = _case(lens, n_q, n_kv, hd, page, seed)
    S = len(lens)
    scale = 1.0 / math.sqrt(hd)
    stream = torch.cuda.current_stream().cuda_stream
    table = s["table"]
    # the existing entry point, its workspace brought by the caller (NaN: an unwritten part would show)
    part_o = torch.full((S * n_q * nsplit * hd,), float("nan"), device=DEV)
    part_ml = torch.full((S * n_q * nsplit * 2,), float("nan"), device=DEV)
    out_ws = torch.zeros_like(q)
    rc = lib.llme_attention_bf16(q.data_ptr(), s["k_cache"].data_ptr(), s["v_cache"].data_ptr(), out_ws.data_ptr(),
                                 part_o.data_ptr(), part_ml.data_ptr(), q_start.data_ptr(), ctx_len.data_ptr(),
                                 table.data_ptr(), table.shape[1], S, n_q, n_kv, hd, page, scale, 0, S, split_len,
                                 nsplit, 0, None, S, 1, 1, None, None, 0, stream)
    assert rc == 0
    out_na = torch.zeros_like(q)

    def call():
        return lib.llme_attention_decode_noalloc(q.data_ptr(), s["k_cache"].data_ptr(), s["v_cache"].data_ptr(),
                                                 out_na.data_ptr(), q_start.data_ptr(), ctx_len.data_ptr(),
                                                 table.data_ptr(), table.shape[1], S, n_q, n_kv, hd, page, scale, 0,
                                                 split_len, nsplit, stream)
    # Free device memory as the driver counts it (torch's own counters would not see a hipMalloc inside
    # the library), around a second call of the same sizes: what the runtime sets up for a kernel's
    # first launch is done by then.
    assert call() == 0
    torch.cuda.synchronize()
    free_before, allocated_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    out_na.zero_()
    assert call() == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == allocated_before
    return out_na, out_ws, ref


def test_no_alloc_decode_attention_twice(lib):
    assert lib.llme_noalloc_init() == 0
    assert lib.llme_noalloc_init() == 0                     # asking again is harmless
    # first call: three requests, 16 splits of 96 keys
    n_q, n_kv, hd, page = 8, 2, 64, 16
    assert lib.llme_attention_decode_noalloc_scratch_floats(3, n_q, hd, 16) == 3 * n_q * 16 * (hd + 2)
    out_na, out_ws, ref = _run_both(lib, [1500, 40, 700], n_q, n_kv, hd, page, split_len=96, nsplit=16, seed=71)
    assert torch.equal(out_na, out_ws)
    assert (out_na.cpu().double() - ref).abs().max() / ref.abs().max() < 8e-3
    # second call, smaller in every size: one request, other heads, 3 splits
    out_na2, out_ws2, ref2 = _run_both(lib, [300], 6, 3, 32, 16, split_len=128, nsplit=3, seed=72)
    assert torch.equal(out_na2, out_ws2)
    assert (out_na2.cpu().double() - ref2).abs().max() / ref2.abs().max() < 8e-3
    # and a third without splits (the array is not used at all)
    out_na3, out_ws3, ref3 = _run_both(lib, [45, 17], 4, 4, 128, 32, split_len=64, nsplit=1, seed=73)
    assert torch.equal(out_na3, out_ws3)
    assert (out_na3.cpu().double() - ref3).abs().max() / ref3.abs().max() < 8e-3


def test_no_alloc_decode_attention_recorded_into_a_graph(lib):
    """After llme_noalloc_init the entry point may be called while a HIP graph is being recorded.
    The graph is replayed several times over changing queries, with eager calls (which use the same
    fixed array) and synchronizations between the replays; every replay must give what the eager
    call gives for the same query."""
    assert lib.llme_noalloc_init() == 0
    lens, n_q, n_kv, hd, page, split_len, nsplit = [900, 130, 520, 64], 8, 2, 64, 16, 128, 8
    s, q, q_start, ctx_len, _ = _case(lens, n_q, n_kv, hd, page, seed=74)
    S, scale, table = len(lens), 1.0 / math.sqrt(hd), None
    table = s["table"]
    out_graph, out_eager = torch.zeros_like(q), torch.zeros_like(q)

    def call(out, stream):
        return lib.llme_attention_decode_noalloc(q.data_ptr(), s["k_cache"].data_ptr(), s["v_cache"].data_ptr(),
                                                 out.data_ptr(), q_start.data_ptr(), ctx_len.data_ptr(),
                                                 table.data_ptr(), table.shape[1], S, n_q, n_kv, hd, page, scale, 0,
                                                 split_len, nsplit, stream)
    assert call(out_eager, torch.cuda.current_stream().cuda_stream) == 0      # (every kernel has been launched once)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert call(out_graph, torch.cuda.current_stream().cuda_stream) == 0
    g = torch.Generator(device="cpu").manual_seed(5)
    for replay_no in range(4):
        q.copy_((torch.randn(q.shape, generator=g) * 0.7).to(torch.bfloat16))
        out_graph.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert call(out_eager, torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(out_graph, out_eager) and out_graph.abs().max() > 0, replay_no


def test_no_alloc_refuses_what_does_not_fit(lib):
    q = torch.zeros(1, 64, dtype=torch.bfloat16, device=DEV)
    kc = torch.zeros(1, 1, 16, 64, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(1, 1, 64, 16, dtype=torch.bfloat16, device=DEV)
    i32 = dict(dtype=torch.int32, device=DEV)
    qs, cl, tb = torch.tensor([0, 1], **i32), torch.tensor([0], **i32), torch.zeros(1, 1, **i32)
    stream = torch.cuda.current_stream().cuda_stream

    def call(n_seq, n_q, n_kv, hd, split_len, nsplit):
        return lib.llme_attention_decode_noalloc(q.data_ptr(), kc.data_ptr(), vc.data_ptr(), q.data_ptr(), qs.data_ptr(),
                                                 cl.data_ptr(), tb.data_ptr(), 1, n_seq, n_q, n_kv, hd, 16, 0.125, 0,
                                                 split_len, nsplit, stream)
    # 4,096 requests x 64 heads x 64 splits x 130 floats are beyond the fixed array: refused, nothing launched
    assert call(4096, 64, 8, 128, 32, 64) == 10002
    assert call(1, 1, 1, 64, 33, 2) == 10001                # a split length that is no multiple of 32
    assert call(1, 1, 1, 64, 32, 65) == 10001               # more splits than the join takes
    assert call(1, 1, 1, 72, 32, 2) == 10002                # a head size the kernels do not have
    torch.cuda.synchronize()
