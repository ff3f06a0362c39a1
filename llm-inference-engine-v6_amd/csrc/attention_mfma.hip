// Attention over bfloat16 cache pages on the matrix cores (v_mfma_f32_16x16x32_bf16).
// Formula as in the plain-precision kernel (src/kernels.cpp:413-474): kv head = q head /
// (n_q / n_kv), scores scaled by `scale`, softmax over the keys a token may see, weighted
// sum of values. Softmax statistics and accumulation are 32-bit; probabilities enter the
// second product rounded to bfloat16.
//
// Layouts: k_cache [pages, n_kv, page, hd]; v_cache [pages, n_kv, hd, page] (keys contiguous
// for a fixed dimension, which is what the second product's operand wants); q, out
// [T, n_q * hd]; block_table [n_seq, max_blocks].
//
// One wavefront handles a tile of 16 query rows against 32 keys at a time:
//   S^T[key, row] = sum_d K[key, d] Q[row, d]      first operand K (16 keys x 32 d, one
//                                                   16-byte load per lane), second Q^T
//   lane l then holds, for row l % 16, the keys 4 (l / 16) + e of both 16-key halves:
//   exactly the 8 keys this lane must supply as first operand of
//   O[row, d] += sum_key P[row, key] V[key, d]      second operand V^T read 4 keys (8 bytes)
//                                                   at a time from the transposed pages
// so probabilities never pass through LDS. The running maximum m and sum l are kept per
// lane for row l % 16; O's rows are 4 (l / 16) + e, so rescaling fetches factors by shuffle.
//
// Two kernels share this tile code:
//  * decode: requests that bring one token. The 16 rows are the query heads of one kv
//    head; grid (kv head x head tile, request, split of the keys); partial results of the
//    splits are joined by a small second kernel. The kv head runs fastest because workgroups
//    go to the chip's 8 dies in turn: with the request fastest and a number of requests that
//    is a multiple of 8, a die got all heads of every eighth request, and the dies' loads
//    differed as the requests' lengths do (44 requests of 256 to 6,144 tokens at the 1B
//    sizes: 2.45 -> 2.18 ms a step; requests of one length: no difference).
//  * prefill: requests that bring several tokens. The rows are 16 consecutive tokens of one
//    query head; a wavefront takes QT such tiles so that every K and V load is used QT
//    times; a workgroup's four wavefronts take four neighbouring heads of the same tokens,
//    so their K and V loads hit the same cache lines. Causal by position: row at position
//    p sees keys max(0, p - window + 1) .. p; key blocks past the last row are not visited.
// Requests are told apart on the device from q_start (first batch row of each request).
//
// Limits (the caller checks them and otherwise uses the plain-precision kernel): head size a
// multiple of 16 up to 128; page size a multiple of 16.
#include <mutex>

#include "attention_tiles.h"
#include "llmengine_noalloc.h"

namespace llme {

// ------------------------------------------------------------------------------------------
// decode: one token per request; the work of a workgroup is decode_item (attention_tiles.h).
template <int HD, bool STREAM>
__global__ __launch_bounds__(DEC_WAVES * 64) void attention_decode_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int max_blocks, int n_q, int n_kv, int page, float scale, int window, int split_len, int nsplit) {
    __shared__ float sh[decode_lds_floats(HD)];
    decode_item<HD, STREAM>(q, k_cache, v_cache, out, part_o, part_ml, q_start, ctx_len, block_table, max_blocks, n_q,
                            n_kv, page, scale, window, split_len, nsplit, blockIdx.y, blockIdx.x, blockIdx.z, sh);
}

// The same for a step whose q/k/v rows are still as the projection left them (RAW in attention_tiles.h):
// grid (request, kv head); a single split, so the output rows are written at once.
template <int HD>
__global__ __launch_bounds__(DEC_WAVES * 64) void attention_decode_raw_kernel(
    float* qkv, const float* __restrict__ cos_t, const float* __restrict__ sin_t, bf16* k_cache, bf16* v_cache,
    bf16* __restrict__ out, const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale, int window,
    int split_len) {
    __shared__ float sh[decode_lds_floats(HD)];
    const RawQkv raw{qkv, cos_t, sin_t, k_cache, v_cache};
    decode_item<HD, true, true>(nullptr, k_cache, v_cache, out, nullptr, nullptr, q_start, ctx_len, block_table,
                                max_blocks, n_q, n_kv, page, scale, window, split_len, 1, blockIdx.y, blockIdx.x, 0, sh,
                                raw);
}

// Joins the splits of one (row, head): one wavefront, lanes over the splits for the statistics,
// then over the head's dimensions for the weighted sum. nsplit <= 64. `base` is the first of the
// nsplit parts. The partial outputs are asked for 16 splits at a time, the first 16 together with
// the statistics: asked for one after the other, the trips to memory were most of the time.
constexpr int JOIN_AT_A_TIME = 16;
__device__ __forceinline__ void join_splits(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                            bf16* __restrict__ out_row, size_t base, int hd, int nsplit,
                                            float* weight) {
    const int lane = threadIdx.x;
    float part[JOIN_AT_A_TIME];
    auto ask = [&](int first, int d) {                 // (splits past the last: the last again, with weight 0)
#pragma unroll
        for (int u = 0; u < JOIN_AT_A_TIME; ++u) {
            const int i = first + u < nsplit ? first + u : nsplit - 1;
            part[u] = part_o[(base + i) * hd + (d < hd ? d : 0)];
        }
    };
    ask(0, lane);
    float mi = -INFINITY, li = 0.f;
    if (lane < nsplit) {
        mi = part_ml[(base + lane) * 2];
        li = part_ml[(base + lane) * 2 + 1];
    }
    const float mx = wave_max(mi);
    const float f = (mi <= kNoMax) ? 0.f : exp2f(mi - mx);
    const float total = wave_sum(f * li);
    weight[lane] = f / total;                          // 0 for lanes past the last split
    __syncthreads();
    for (int d = lane; d < hd; d += 64) {
        float acc = 0.f;
        for (int first = 0; first < nsplit; first += JOIN_AT_A_TIME) {
            if (d != lane || first != 0) ask(first, d);            // (the first are on their way)
#pragma unroll
            for (int u = 0; u < JOIN_AT_A_TIME; ++u)
                acc += (first + u < nsplit ? weight[first + u] : 0.f) * part[u];
        }
        out_row[d] = static_cast<bf16>(acc);
    }
}

// The decode kernel's splits of (request s, head h); parts indexed by request.
__device__ __forceinline__ void join_decode_splits(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                   bf16* __restrict__ out, const int* __restrict__ q_start, int n_q,
                                                   int hd, int nsplit, int s, int h, float* weight) {
    const int row0 = q_start[s];
    if (q_start[s + 1] - row0 != 1) return;
    join_splits(part_o, part_ml, out + (static_cast<size_t>(row0) * n_q + h) * hd,
                (static_cast<size_t>(s) * n_q + h) * nsplit, hd, nsplit, weight);
}

// The prefill kernel's key runs of (batch row, head h); parts indexed by batch row. Rows of
// requests that bring one token belong to the decode kernel and are left alone, and so are rows
// of work items with a single run, which wrote their output themselves. span_rows: rows of one
// work item; the row's item and its number of runs are found as the prefill kernel finds them.
__device__ __forceinline__ void join_row_runs(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              bf16* __restrict__ out, const int* __restrict__ q_start,
                                              const int* __restrict__ ctx_len, int n_seq, int n_q, int hd, int nsplit,
                                              int run, int span_rows, int window, int row, int h, float* weight) {
    const int lane = threadIdx.x;
    int first_row = -1, n_new = 0, ctx = 0;             // the row's request (the same in every lane)
    for (int first = 0; first < n_seq; first += 64) {
        const int i = first + lane;
        int a = 0, b = 0, c = 0;
        bool hit = false;
        if (i < n_seq) {
            a = q_start[i];
            b = q_start[i + 1];
            hit = a <= row && row < b && b - a >= 2;
            if (hit) c = ctx_len[i];
        }
        const unsigned long long votes = __ballot(hit);
        if (votes != 0) {
            const int src = __ffsll(static_cast<long long>(votes)) - 1;
            first_row = __shfl(a, src, 64);
            n_new = __shfl(b, src, 64) - first_row;
            ctx = __shfl(c, src, 64);
        }
    }
    if (first_row < 0) return;
    const int span = (row - first_row) / span_rows;
    const int pos_span = ctx + span * span_rows;
    const int n_span = n_new - span * span_rows < span_rows ? n_new - span * span_rows : span_rows;
    const int key_lo = (window > 0 && pos_span - window + 1 > 0) ? pos_span - window + 1 : 0;
    const int runs = key_runs(key_lo & ~63, pos_span + n_span, run, nsplit);
    if (runs == 1) return;
    join_splits(part_o, part_ml, out + (static_cast<size_t>(row) * n_q + h) * hd,
                (static_cast<size_t>(row) * n_q + h) * nsplit, hd, runs, weight);
}

// grid (request, head)
__global__ __launch_bounds__(64) void attention_join_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml, bf16* __restrict__ out,
                                                            const int* __restrict__ q_start, int n_q, int hd, int nsplit) {
    __shared__ float weight[64];
    join_decode_splits(part_o, part_ml, out, q_start, n_q, hd, nsplit, blockIdx.x, blockIdx.y, weight);
}

// grid (batch row, head)
__global__ __launch_bounds__(64) void attention_join_rows_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 bf16* __restrict__ out, const int* __restrict__ q_start,
                                                                 const int* __restrict__ ctx_len, int n_seq, int n_q,
                                                                 int hd, int nsplit, int run, int span_rows, int window) {
    __shared__ float weight[64];
    join_row_runs(part_o, part_ml, out, q_start, ctx_len, n_seq, n_q, hd, nsplit, run, span_rows, window, blockIdx.x,
                  blockIdx.y, weight);
}

// Both joins of a step that holds decoded tokens and prompt portions, in one launch: grid
// (requests + batch rows, head); the first n_seq workgroups of a head join the decode splits.
__global__ __launch_bounds__(64) void attention_join_both_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, int nsplit,
    const float* __restrict__ pre_part_o, const float* __restrict__ pre_part_ml, int pre_nsplit, int run, int span_rows,
    bf16* __restrict__ out, const int* __restrict__ q_start, const int* __restrict__ ctx_len, int n_seq, int n_q, int hd,
    int window) {
    __shared__ float weight[64];
    const int x = blockIdx.x;
    if (x < n_seq) join_decode_splits(part_o, part_ml, out, q_start, n_q, hd, nsplit, x, blockIdx.y, weight);
    else join_row_runs(pre_part_o, pre_part_ml, out, q_start, ctx_len, n_seq, n_q, hd, pre_nsplit, run, span_rows, window,
                       x - n_seq, blockIdx.y, weight);
}

// ------------------------------------------------------------------------------------------
// prefill: several tokens per request; a wavefront takes QT tiles of 16 tokens of one head
template <int HD, int QT>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int max_blocks, int n_seq, int n_q, int n_kv, int page, float scale,
    int window) {
    constexpr int DC = (HD + 31) / 32, DT = HD / 16, ROWS = 16 * QT;
    // which request and which of its row groups this workgroup has
    int s = 0, first = 0, n_rows = 0, acc = 0;
    bool found = false;
    for (int i = 0; i < n_seq; ++i) {
        const int a = q_start[i], n = q_start[i + 1] - a;
        const int nt = (n >= 2) ? (n + ROWS - 1) / ROWS : 0;
        if (!found && static_cast<int>(blockIdx.x) < acc + nt) {
            s = i;
            first = (nt - 1 - (blockIdx.x - acc)) * ROWS; // first row of the group within the request; the
                                                          // last groups see the most keys and start first
            n_rows = n - first < ROWS ? n - first : ROWS;
            first += a;                                   // as a batch row
            found = true;
        }
        acc += nt;
    }
    if (!found) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // scalar: so are the head's addresses
    const int lane = threadIdx.x & 63, r = lane & 15, g4 = lane >> 4;
    const int head = blockIdx.y * 4 + wave;
    if (head >= n_q) return;
    const int kvh = head / (n_q / n_kv);
    const int pos0 = ctx_len[s] + (first - q_start[s]);  // position of the group's first row

    bf16x8 qf[QT][DC];
    int row_pos[QT], row_lo[QT], tile_free[QT];
    float m[QT], l[QT];
    f32x4 o[QT][DT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int rr = qt * 16 + r;
        const bool ok = rr < n_rows;
        load_q<HD>(q + (static_cast<size_t>(first + (ok ? rr : 0)) * n_q + head) * HD, ok, qf[qt]);
        row_pos[qt] = ok ? pos0 + rr : -1;
        row_lo[qt] = (window > 0 && pos0 + rr - window + 1 > 0) ? pos0 + rr - window + 1 : 0;
        tile_free[qt] = (window == 0 && qt * 16 + 16 <= n_rows) ? pos0 + qt * 16 : -1;
        m[qt] = kNoMax;
        l[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int key_end = pos0 + n_rows;                    // the last row sees keys < key_end
    const int key_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;   // the first row's first key
    const int k_begin = key_lo & ~31;
    PagedKV kv{k_cache, v_cache, block_table + static_cast<size_t>(s) * max_blocks, page, n_kv, kvh, HD,
               page_magic_of(page), static_cast<unsigned>(n_kv) * page * HD, static_cast<unsigned>(kvh) * page * HD};
    const float scale_log2 = scale * kLog2e;
    attend_range<HD, QT>(kv, k_begin, 32, key_lo, key_end, qf, row_pos, row_lo, tile_free, scale_log2, m, l, o);

#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float lt = l[qt];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int rr = g4 * 4 + e;
            const float l_row = __shfl(lt, rr, 64);
            const int row = qt * 16 + rr;
            if (row >= n_rows) continue;
            const float inv = 1.0f / l_row;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                out[(static_cast<size_t>(first + row) * n_q + head) * HD + dt * 16 + r] =
                    static_cast<bf16>(o[qt][dt][e] * inv);
        }
    }
}

// What a caller may override of the launch choices, for tests and measurements, packed into
// the entry points' `tuning` argument (0: every choice is the entry point's):
//   bits 0-7   rows per work item of the prefill kernel without LDS: 16, 32 or 64 (0: by head size)
//   bits 8-11  1 + shared: -1 the kernel that shares K and V through LDS where it takes the sizes
//              (the default), 0 never, 1 wherever it can, 2 / 3 the same with one / two wavefronts
//              per tile whatever the number of work items
//   bits 12-13 1 + read_once: whether the decode kernel loads keys and values with the read-once
//              hint: -1 the entry point chooses, 0 never, 1 always
//   bit 14     the decode kernel's splits are left unjoined in part_o / part_ml: the caller joins them
//              (llme_attention_join_project); only for steps without prompt portions
//   bit 15     the prefill kernel that shares K and V through LDS takes work items of half the rows (16
//              per row group instead of 32): for steps with few items (see attention_prefill.hip)
struct Tuning {
    int rows, shared, key_waves, read_once, no_join, half_rows;
};
static bool parse_tuning(int packed, Tuning* t) {
    if (packed < 0 || packed >= (1 << 16)) return false;
    const int rows = packed & 0xFF, shared = ((packed >> 8) & 0xF) - 1, read_once = ((packed >> 12) & 0x3) - 1;
    if (rows % 16 != 0 || rows > 64 || shared > 3 || read_once > 1) return false;
    *t = Tuning{rows, shared > 1 ? 1 : shared, shared > 1 ? shared - 1 : 0, read_once, (packed >> 14) & 1,
                (packed >> 15) & 1};
    return true;
}
static bool decode_reads_once(const Tuning& t) { return t.read_once != 0; }

template <int HD>
static int launch_for_head(const bf16* q, const bf16* kc, const bf16* vc, bf16* out, float* part_o, float* part_ml,
                           const int* q_start, const int* ctx_len, const int* table, int max_blocks, int n_seq,
                           int n_q, int n_kv, int page, float scale, int window, int n_decode, int split_len,
                           int nsplit, int prefill_groups, int qt, int shared_rows, int* queue, int n_rows,
                           int prefill_splits, int prefill_run, float* pre_part_o, float* pre_part_ml,
                           const Tuning& tuning, hipStream_t stream) {
    const int head_tiles = n_kv * ((n_q / n_kv + 15) / 16);
    // A step with decoded tokens and prompt portions: where the prompt kernel that shares K and V
    // through LDS runs, it takes the decode work items into its launch (the two kinds of work do
    // not depend on each other; measured at the 1B sizes, a 256-token portion beside 17 decoded
    // tokens, one after the other they took 17.8 + 21.4 us a layer).
    const bool together = n_decode > 0 && prefill_groups > 0 && shared_rows > 0 && decode_reads_once(tuning);
    if (n_decode > 0 && !together) {
        const dim3 grid(head_tiles, n_seq, nsplit);
        if (decode_reads_once(tuning))
            hipLaunchKernelGGL((attention_decode_kernel<HD, true>), grid, dim3(DEC_WAVES * 64), 0, stream, q, kc, vc, out,
                               part_o, part_ml, q_start, ctx_len, table, max_blocks, n_q, n_kv, page, scale, window,
                               split_len, nsplit);
        else
            hipLaunchKernelGGL((attention_decode_kernel<HD, false>), grid, dim3(DEC_WAVES * 64), 0, stream, q, kc, vc, out,
                               part_o, part_ml, q_start, ctx_len, table, max_blocks, n_q, n_kv, page, scale, window,
                               split_len, nsplit);
        if (nsplit > 1 && !tuning.no_join)
            hipLaunchKernelGGL(attention_join_kernel, dim3(n_seq, n_q), dim3(64), 0, stream, part_o, part_ml, out,
                               q_start, n_q, HD, nsplit);
    }
    if (prefill_groups > 0) {
        if (shared_rows > 0) {
            DecodeBeside beside;
            if (together) {
                beside.part_o = part_o;
                beside.part_ml = part_ml;
                beside.head_tiles = head_tiles;
                beside.split_len = split_len;
                beside.nsplit = nsplit;
                beside.blocks = n_seq * head_tiles * nsplit;
            }
            const int status = launch_prefill_shared(q, kc, vc, out, q_start, ctx_len, table, max_blocks, n_seq, n_q,
                                                     n_kv, HD, page, scale, window, prefill_groups, shared_rows, queue,
                                                     prefill_splits, prefill_run, pre_part_o, pre_part_ml,
                                                     tuning.key_waves, beside, stream);
            if (status != 0) return status;
            if (together && nsplit > 1 && prefill_splits > 1) {
                hipLaunchKernelGGL(attention_join_both_kernel, dim3(n_seq + n_rows, n_q), dim3(64), 0, stream, part_o,
                                   part_ml, nsplit, pre_part_o, pre_part_ml, prefill_splits, prefill_run, shared_rows, out,
                                   q_start, ctx_len, n_seq, n_q, HD, window);
                return launch_status();
            }
            if (together && nsplit > 1)
                hipLaunchKernelGGL(attention_join_kernel, dim3(n_seq, n_q), dim3(64), 0, stream, part_o, part_ml, out,
                                   q_start, n_q, HD, nsplit);
            if (prefill_splits <= 1) return launch_status();
            hipLaunchKernelGGL(attention_join_rows_kernel, dim3(n_rows, n_q), dim3(64), 0, stream, pre_part_o,
                               pre_part_ml, out, q_start, ctx_len, n_seq, n_q, HD, prefill_splits, prefill_run,
                               shared_rows, window);
            return launch_status();
        }
        const dim3 grid(prefill_groups, (n_q + 3) / 4);
#define LLME_PREFILL(QT)                                                                                       \
    hipLaunchKernelGGL((attention_prefill_kernel<HD, QT>), grid, dim3(256), 0, stream, q, kc, vc, out, q_start, \
                       ctx_len, table, max_blocks, n_seq, n_q, n_kv, page, scale, window)
        if (qt == 4 && HD <= 64) LLME_PREFILL(4);
        else if (qt == 2) LLME_PREFILL(2);
        else LLME_PREFILL(1);
#undef LLME_PREFILL
    }
    return launch_status();
}

}  // namespace llme

using namespace llme;

// Rows per prefill work item for a model's head sizes: the caller sizes the grid with it. More
// rows reuse every K and V load more often; fewer rows give more wavefronts to hide latencies
// and to even out the causal triangle. The kernel that shares K and V through LDS is used
// where it takes the sizes.
static int direct_rows(int hd, const Tuning& t) {
    int rows = hd <= 64 ? 64 : 32;
    if (t.rows == 16 || t.rows == 32 || t.rows == 64) rows = t.rows;
    if (hd > 64 && rows > 32) rows = 32;
    return rows;
}
static int shared_rows_for(int hd, int n_q, int n_kv, const Tuning& t) {
    const int rows = t.shared == 0 ? 0 : prefill_shared_rows(hd, n_q, n_kv);
    return t.half_rows ? rows / 2 : rows;
}
extern "C" int llme_attention_bf16_rows(int hd, int n_q, int n_kv, int tuning) {
    Tuning t;
    if (!parse_tuning(tuning, &t)) return -1;
    const int shared = shared_rows_for(hd, n_q, n_kv, t);
    return shared > 0 ? shared : direct_rows(hd, t);
}

// n_decode: requests with one token (0: none, skip the decode kernels); split_len (multiple of
// 32) and nsplit: how the decode kernel cuts the keys; part_o [n_seq, n_q, nsplit, hd] and
// part_ml [n_seq, n_q, nsplit, 2] floats (needed when nsplit > 1). prefill_groups: number of
// row groups of llme_attention_bf16_rows(hd, n_q, n_kv, tuning) rows over the requests with two or more tokens.
// queue: two integers, zero, for the prefill kernel's work counter (needed when prefill_groups > 0;
// the kernel leaves them zero; launches that may overlap need separate ones).
// prefill_splits > 1 (only where llme_attention_bf16_splits_prefill says so): the keys of a prefill
// work item are cut into runs of prefill_run stretches of 64 keys, at most prefill_splits (the
// last run takes the rest), joined by a second kernel over the batch's n_rows rows; pre_part_o
// [n_rows, n_q, prefill_splits, hd] and pre_part_ml [n_rows, n_q, prefill_splits, 2] floats are
// their scratch.
extern "C" int llme_attention_bf16_splits_prefill(int hd, int n_q, int n_kv, int tuning) {
    Tuning t;
    if (!parse_tuning(tuning, &t)) return 0;
    return shared_rows_for(hd, n_q, n_kv, t) > 0 ? 1 : 0;
}

extern "C" int llme_attention_bf16(const void* q, const void* k_cache, const void* v_cache, void* out, float* part_o,
                                   float* part_ml, const int* q_start, const int* ctx_len, const int* block_table,
                                   int max_blocks, int n_seq, int n_q, int n_kv, int hd, int page, float scale,
                                   int window, int n_decode, int split_len, int nsplit, int prefill_groups,
                                   int* queue, int n_rows, int prefill_splits, int prefill_run, float* pre_part_o,
                                   float* pre_part_ml, int tuning, hipStream_t stream) {
    if (n_seq <= 0) return 0;
    Tuning tune;
    if (!parse_tuning(tuning, &tune)) return kErrBadArgument;
    if (prefill_splits < 1 || prefill_splits > 64 || n_rows < 0) return kErrBadArgument;
    if (prefill_splits > 1 && (shared_rows_for(hd, n_q, n_kv, tune) <= 0 || prefill_run < 1 || pre_part_o == nullptr ||
                               pre_part_ml == nullptr))
        return kErrBadArgument;
    if (hd % 16 != 0 || hd > 128 || hd <= 0 || page % 16 != 0 || n_kv <= 0 || n_q % n_kv != 0) return kErrUnsupported;
    if (!(scale > 0.f)) return kErrBadArgument;      // the lazy maximum compares scaled scores
    // page lookups divide by multiplication, exact while (keys / 16) * (page / 16) < 2^32
    if (static_cast<double>(max_blocks) * (page / 16) * (page / 16) >= 4294967296.0) return kErrUnsupported;
    if (static_cast<double>(n_kv) * page * hd >= 4294967296.0) return kErrUnsupported;   // a page's elements: 32 bits
    if (n_decode > 0 && (split_len <= 0 || split_len % 32 != 0 || nsplit <= 0 || nsplit > 64)) return kErrBadArgument;
    if (n_decode > 0 && n_seq > 65535) return kErrUnsupported;      // (the decode grid counts requests in y)
    if (tune.no_join && prefill_groups > 0) return kErrBadArgument;
    const int qt = direct_rows(hd, tune) / 16;
    const int shared_rows = shared_rows_for(hd, n_q, n_kv, tune);
#define LLME_HEAD(HD)                                                                                           \
    case HD:                                                                                                    \
        return launch_for_head<HD>(static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache),              \
                                   static_cast<const bf16*>(v_cache), static_cast<bf16*>(out), part_o, part_ml, \
                                   q_start, ctx_len, block_table, max_blocks, n_seq, n_q, n_kv, page, scale,    \
                                   window, n_decode, split_len, nsplit, prefill_groups, qt, shared_rows, queue, n_rows, \
                                   prefill_splits, prefill_run, pre_part_o, pre_part_ml, tune, stream)
    switch (hd) {
        LLME_HEAD(16); LLME_HEAD(32); LLME_HEAD(48); LLME_HEAD(64);
        LLME_HEAD(80); LLME_HEAD(96); LLME_HEAD(112); LLME_HEAD(128);
        default: return kErrUnsupported;
    }
#undef LLME_HEAD
}

// Decode attention over a step of single tokens whose q/k/v rows are still 32-bit and unrotated (what a
// projection cut over k has added up): rotation, cache write and the clearing of the rows happen inside
// the attention kernel, one workgroup per (request, kv head) and a single split of the keys. qkv
// [n_seq, (n_q + 2 n_kv) hd] float32 (row s is request s; left zero), cos/sin [max_pos, hd / 2]; the caches
// as in llme_attention_bf16, written at each request's position ctx_len[s]; out [n_seq, n_q hd] bfloat16.
// Head size 64 or 128, up to 16 query heads per kv head; split_len a multiple of 32 that covers the longest
// request.
extern "C" int llme_attention_decode_rope_bf16(float* qkv, const float* cos_t, const float* sin_t, void* k_cache,
                                               void* v_cache, void* out, const int* q_start, const int* ctx_len,
                                               const int* block_table, int max_blocks, int n_seq, int n_q, int n_kv,
                                               int hd, int page, float scale, int window, int split_len,
                                               hipStream_t stream) {
    if (n_seq <= 0) return 0;
    if (!qkv || !cos_t || !sin_t || !k_cache || !v_cache || !out || !q_start || !ctx_len || !block_table) return kErrBadArgument;
    if ((hd != 64 && hd != 128) || page % 16 != 0 || n_kv <= 0 || n_q % n_kv != 0 || n_q / n_kv > 16) return kErrUnsupported;
    if (!(scale > 0.f) || split_len <= 0 || split_len % 32 != 0) return kErrBadArgument;
    if (n_seq > 65535) return kErrUnsupported;                      // (the grid counts requests in y)
    if (static_cast<double>(max_blocks) * (page / 16) * (page / 16) >= 4294967296.0) return kErrUnsupported;
    if (static_cast<double>(n_kv) * page * hd >= 4294967296.0) return kErrUnsupported;
    if (reinterpret_cast<uintptr_t>(qkv) % 16 != 0 || reinterpret_cast<uintptr_t>(cos_t) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(sin_t) % 16 != 0 || reinterpret_cast<uintptr_t>(k_cache) % 16 != 0)
        return kErrUnsupported;
    const dim3 grid(n_kv, n_seq);
    if (hd == 64)
        hipLaunchKernelGGL(attention_decode_raw_kernel<64>, grid, dim3(DEC_WAVES * 64), 0, stream, qkv, cos_t, sin_t,
                           static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache), static_cast<bf16*>(out), q_start,
                           ctx_len, block_table, max_blocks, n_q, n_kv, page, scale, window, split_len);
    else
        hipLaunchKernelGGL(attention_decode_raw_kernel<128>, grid, dim3(DEC_WAVES * 64), 0, stream, qkv, cos_t, sin_t,
                           static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache), static_cast<bf16*>(out), q_start,
                           ctx_len, block_table, max_blocks, n_q, n_kv, page, scale, window, split_len);
    return launch_status();
}

// ------------------------------------------------------------------------------------------
// Decode attention for callers that cannot allocate (declared in llmengine_noalloc.h). The split
// decode kernel and its join are the ones above; the splits' partial results go into a fixed
// array in device memory instead of a workspace that the caller brings. Every device the library
// runs on holds its own copy of the array, at its own address, until the process ends; the address
// is asked for once per device, with that device current, and kept.
static __device__ __align__(256) float scratch[LLME_NOALLOC_SCRATCH_FLOATS];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices] = {};

// The array's address on the current device (host code must never use the array's name as one).
int scratch_of_current_device(float** ptr) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return static_cast<int>(err);
    if (device < 0 || device >= kMaxDevices) return kErrUnsupported;
    std::lock_guard<std::mutex> guard(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        void* address = nullptr;
        err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return static_cast<int>(err);
        if (address == nullptr) return kErrUnsupported;
        g_scratch_ptr[device] = static_cast<float*>(address);
    }
    *ptr = g_scratch_ptr[device];
    return 0;
}
}  // namespace

extern "C" int llme_noalloc_init(void) {
    float* ptr = nullptr;
    return scratch_of_current_device(&ptr);
}

extern "C" long llme_attention_decode_noalloc_scratch_floats(int n_seq, int n_q, int hd, int nsplit) {
    return static_cast<long>(n_seq) * n_q * nsplit * (hd + 2);
}

extern "C" int llme_attention_decode_noalloc(const void* q, const void* k_cache, const void* v_cache, void* out,
                                             const int* q_start, const int* ctx_len, const int* block_table,
                                             int max_blocks, int n_seq, int n_q, int n_kv, int hd, int page,
                                             float scale, int window, int split_len, int nsplit,
                                             hipStream_t stream) {
    if (n_seq <= 0) return 0;
    if (q == nullptr || k_cache == nullptr || v_cache == nullptr || out == nullptr || q_start == nullptr ||
        ctx_len == nullptr || block_table == nullptr || max_blocks <= 0)
        return kErrBadArgument;
    if (n_q <= 0 || n_kv <= 0 || hd <= 0 || split_len <= 0 || split_len % 32 != 0 || nsplit <= 0 || nsplit > 64)
        return kErrBadArgument;
    // the partial results of all splits must fit into the fixed array
    const double need = static_cast<double>(n_seq) * n_q * nsplit * (hd + 2);
    if (nsplit > 1 && need > static_cast<double>(LLME_NOALLOC_SCRATCH_FLOATS)) return kErrUnsupported;
    float* base = nullptr;
    const int status = scratch_of_current_device(&base);
    if (status != 0) return status;
    // Layout: part_o [n_seq, n_q, nsplit, hd], then part_ml [n_seq, n_q, nsplit, 2] (hd is a multiple
    // of 16, so part_ml starts on a 64-byte boundary). Every part the join reads has been written by
    // the decode kernel of the same call (a split past a request's last key writes an empty part),
    // so nothing has to be cleared between calls.
    float* part_o = base;
    float* part_ml = base + static_cast<size_t>(n_seq) * n_q * nsplit * hd;
    return llme_attention_bf16(q, k_cache, v_cache, out, part_o, part_ml, q_start, ctx_len, block_table, max_blocks,
                               n_seq, n_q, n_kv, hd, page, scale, window, /*n_decode=*/n_seq, split_len, nsplit,
                               /*prefill_groups=*/0, /*queue=*/nullptr, /*n_rows=*/n_seq, /*prefill_splits=*/1,
                               /*prefill_run=*/1, nullptr, nullptr, /*tuning=*/0, stream);
}

LLME_LOAD_ENTRY(attention_mfma)
