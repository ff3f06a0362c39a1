// Attention over cache pages, plain-precision kernel: one wavefront per (token, query
// head), or, when a step has few tokens (decoding), several that take every NW-th chunk of the
// keys and join their results through LDS; scores, softmax statistics and the weighted sum all
// in 32-bit. It serves the
// 32-bit model, and the bfloat16 model for head sizes or page sizes that the MFMA
// kernels refuse. Any head size up to 256, any page size, any head counts.
//
// Formula (src/kernels.cpp:413-474): kv head = q head / (n_q / n_kv);
// s_t = (q . K[t]) * scale for the keys t the token may see; p = softmax(s);
// out = sum_t p_t V[t]. The softmax is evaluated online over chunks of 64 keys
// (running maximum m, running sum l), which equals the reference's two-pass form
// up to rounding. A token at position p sees keys [lo, p] of its own request, with
// lo = 0, or p - window + 1 when a window is given; the step's own keys are in the
// pages already, so prompts, portions and decoded tokens are the same case.
//
//   q, out     [T, n_q * hd]
//   k_cache    [pages, n_kv, page, hd]      v_cache [pages, n_kv, hd, page]
//   block_table[n_seq, max_blocks]; key t of request s lies in page
//              block_table[s][t / page] at offset t % page
#include "common.h"
#include <math.h>

namespace llme {

constexpr int kMaxHead = 256;

template <typename TQ, typename TC, int NW>
__global__ __launch_bounds__(NW * 64) void attention_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    TQ* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ seq_idx,
    const int* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int hd, int page, float scale,
    int window) {
    constexpr int PER_LANE = kMaxHead / kWave;
    __shared__ float qs[kMaxHead];
    __shared__ float join_m[NW], join_l[NW];
    __shared__ float join_acc[NW > 1 ? NW : 1][NW > 1 ? kMaxHead : 1];
    const int t = blockIdx.x;
    const int h = blockIdx.y;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int kvh = h / (n_q / n_kv);
    const int pos = positions[t];
    const int* table = block_table + static_cast<size_t>(seq_idx[t]) * max_blocks;
    const int hi = pos + 1;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

    const TQ* qrow = q + (static_cast<size_t>(t) * n_q + h) * hd;
    for (int d = threadIdx.x; d < hd; d += NW * kWave) qs[d] = to_float(qrow[d]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[PER_LANE] = {0.f, 0.f, 0.f, 0.f};

    // this wavefront's chunks of 64 keys (no barrier inside: the wavefronts take different numbers of turns)
    for (int t0 = lo + wave * kWave; t0 < hi; t0 += NW * kWave) {
        const int key = t0 + lane;
        float sc = -INFINITY;
        if (key < hi) {
            const int pg = table[key / page];
            const TC* kr = k_cache + ((static_cast<size_t>(pg) * n_kv + kvh) * page + key % page) * hd;
            float dot = 0.f;
            for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
            sc = dot * scale;
        }
        const float m_new = fmaxf(m, wave_max(sc));       // finite: the chunk holds at least key t0
        const float alpha = expf(m - m_new);              // 0 on the first chunk (m = -inf)
        const float p = (key < hi) ? expf(sc - m_new) : 0.f;
        l = l * alpha + wave_sum(p);
        m = m_new;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) acc[i] *= alpha;
        const int n = (hi - t0 < kWave) ? hi - t0 : kWave;
        for (int j = 0; j < n; ++j) {
            const int kj = t0 + j;
            const int pg = table[kj / page];
            const TC* vb = v_cache + (static_cast<size_t>(pg) * n_kv + kvh) * hd * page + kj % page;
            const float pj = __shfl(p, j, kWave);
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) {
                const int d = lane + i * kWave;
                if (d < hd) acc[i] = fmaf(pj, to_float(vb[static_cast<size_t>(d) * page]), acc[i]);
            }
        }
    }
    if (NW > 1) {
        // join the wavefronts' parts: each is scaled to the common maximum (a wavefront that saw no
        // key has m = -inf and l = 0: its weight is 0; the first wavefront always saw key lo)
        if (lane == 0) {
            join_m[wave] = m;
            join_l[wave] = l;
        }
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) join_acc[wave][lane + i * kWave] = acc[i];
        __syncthreads();
        if (wave != 0) return;
        float mx = -INFINITY;
        for (int w = 0; w < NW; ++w) mx = fmaxf(mx, join_m[w]);
        l = 0.f;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) acc[i] = 0.f;
        for (int w = 0; w < NW; ++w) {
            const float f = expf(join_m[w] - mx);
            l += f * join_l[w];
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) acc[i] += f * join_acc[w][lane + i * kWave];
        }
    }
    const float inv = 1.0f / l;
    TQ* orow = out + (static_cast<size_t>(t) * n_q + h) * hd;
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const int d = lane + i * kWave;
        if (d < hd) orow[d] = from_float<TQ>(acc[i] * inv);
    }
}

}  // namespace llme

using namespace llme;

extern "C" int llme_attention_generic(const void* q, int q_dtype, const void* k_cache, const void* v_cache,
                                      int cache_dtype, void* out, const int* positions, const int* seq_idx,
                                      const int* block_table, int max_blocks, int T, int n_q, int n_kv,
                                      int hd, int page, float scale, int window, hipStream_t stream) {
    if (T <= 0) return 0;
    if (hd <= 0 || hd > kMaxHead || n_kv <= 0 || n_q % n_kv != 0 || page <= 0) return kErrBadArgument;
    const dim3 grid(T, n_q);
    // few (token, head) pairs, as in decoding: 16 wavefronts each, so that the chip has work
    const bool few = static_cast<long>(T) * n_q < 4096;
#define LLME_ATTN(TQ, TC)                                                                              \
    do {                                                                                               \
        if (few)                                                                                       \
            hipLaunchKernelGGL((attention_generic_kernel<TQ, TC, 16>), grid, dim3(16 * 64), 0, stream, \
                               static_cast<const TQ*>(q), static_cast<const TC*>(k_cache),             \
                               static_cast<const TC*>(v_cache), static_cast<TQ*>(out), positions,      \
                               seq_idx, block_table, max_blocks, n_q, n_kv, hd, page, scale, window);  \
        else                                                                                           \
            hipLaunchKernelGGL((attention_generic_kernel<TQ, TC, 1>), grid, dim3(64), 0, stream,       \
                               static_cast<const TQ*>(q), static_cast<const TC*>(k_cache),             \
                               static_cast<const TC*>(v_cache), static_cast<TQ*>(out), positions,      \
                               seq_idx, block_table, max_blocks, n_q, n_kv, hd, page, scale, window);  \
    } while (0)
    if (q_dtype == kF32 && cache_dtype == kF32) LLME_ATTN(float, float);
    else if (q_dtype == kBF16 && cache_dtype == kBF16) LLME_ATTN(bf16, bf16);
    else if (q_dtype == kF32 && cache_dtype == kBF16) LLME_ATTN(float, bf16);
    else if (q_dtype == kBF16 && cache_dtype == kF32) LLME_ATTN(bf16, float);
    else return kErrBadArgument;
#undef LLME_ATTN
    return launch_status();
}

LLME_LOAD_ENTRY(attention_generic)
