// Tile code shared by the attention kernels on the matrix cores (v_mfma_f32_16x16x32_bf16):
// the paged K and V operands of a 32-key block, its scores, its softmax weights with a lazily
// moved reference maximum, and the walk over a range of blocks with loads straight from the
// cache pages into registers.
//
// One wavefront handles a tile of 16 query rows against 32 keys at a time:
//   S^T[key, row] = sum_d K[key, d] Q[row, d]      first operand K (16 keys x 32 d, 16 bytes
//                                                   per lane), second Q^T
//   lane l then holds, for row l % 16, the keys 4 (l / 16) + e of both 16-key halves:
//   exactly the 8 keys this lane must supply as first operand of
//   O[row, d] += sum_key P[row, key] V[key, d]      second operand V^T, 4 keys (8 bytes) of
//                                                   each half from the transposed pages
// so probabilities never pass through LDS. The running maximum m and sum l are kept per
// lane for row l % 16; O's rows are 4 (l / 16) + e, so rescaling fetches factors by shuffle.
//
// Cache pages hold finite numbers everywhere (the pool starts zeroed and only kernels write
// it), so a key that a row must not see may be loaded: its weight is exactly zero.
#pragma once

#include "common.h"
#include <math.h>

namespace llme {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLazy = 8.0f;

// 2^x by the hardware instruction alone: arguments here are <= 0, results below the normal
// range may flush to zero, which is what a softmax weight that small amounts to.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct PagedKV {
    const bf16* k;
    const bf16* v;
    const int* table;       // this request's row of the block table
    int page, n_kv, kvh, hd;
    unsigned page_magic;    // ceil(2^32 / (page / 16)): key / page without a division, see page_of
    unsigned page_stride;   // elements from one page to the next: n_kv * page * hd
    unsigned head_off;      // elements from a page's start to this kv head's part: kvh * page * hd
};

// Keys come in halves of 16 and the page size is a multiple of 16, so a half's page is
// (t / 16) / (page / 16). With M = ceil(2^32 / d) the quotient u / d equals the high word of
// u * M as long as u * d < 2^32, which the entry point checks for the longest block table.
__device__ __forceinline__ unsigned page_magic_of(int page) {
    const unsigned d = static_cast<unsigned>(page) / 16;
    return d == 1 ? 0u : static_cast<unsigned>((0x100000000ull + d - 1) / d);
}
struct PagePlace {
    int block;      // index into the block table
    int offset;     // first key of the half within its page
};
__device__ __forceinline__ PagePlace page_of(const PagedKV& kv, int h0) {
    const unsigned u = static_cast<unsigned>(h0) >> 4;
    const unsigned b = kv.page_magic ? __umulhi(u, kv.page_magic) : u;
    return PagePlace{static_cast<int>(b), h0 - static_cast<int>(b) * kv.page};
}

__device__ __forceinline__ bf16x8 zero_frag() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.f);
    return z;
}

// The K and V operands of one 32-key block (keys t0 .. t0 + 31), as one lane holds them.
template <int HD>
struct KFrag {
    bf16x8 kf[2][(HD + 31) / 32];      // row r of each 16-key half: dims c * 32 + 8 g4 ..
};
template <int HD>
struct VFrag {
    bf16x8 vf[HD / 16];                // dim dt * 16 + r: keys 4 g4 .. 4 g4 + 3 of each half
};

// The pages of a block's two 16-key halves (a half never straddles pages: the page size is a
// multiple of 16). A half none of whose keys lies in [key_lo, key_end) is not looked up: behind
// key_end nothing is written yet (and the table may end), before key_lo (the first key any
// row of the work item may see) the pages may have been given back.
struct BlockPages {
    int pg[2];
};

__device__ __forceinline__ BlockPages lookup_pages(const PagedKV& kv, int t0, int key_lo, int key_end) {
    BlockPages b;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        const int h0 = t0 + hf * 16;
        // the same for every lane: kept in a scalar register, so that page addresses are scalar work
        b.pg[hf] = (h0 < key_end && h0 + 15 >= key_lo && h0 >= 0)
                       ? __builtin_amdgcn_readfirstlane(kv.table[page_of(kv, h0).block]) : 0;
    }
    return b;
}

// Loads a block's K operand from the pages looked up before. FULL: every key of the block lies
// in [key_lo, key_end) and nothing is checked; otherwise keys outside are not loaded (zeros).
// The full variant has no branch at all: the loop over full blocks then issues the same loads
// on every turn, so the counter of loads in flight tells exactly which have arrived, and a
// wait for this block's operand does not also wait for the next block's.
// STREAM: the loads carry the hint that the data is read once (a decoding request's keys and
// values are read by one workgroup per step): they then pass the L2 without displacing what is
// used again, which streams measurably faster from HBM.
template <int HD, bool FULL, bool STREAM = false>
__device__ __forceinline__ void load_k(const PagedKV& kv, int t0, const BlockPages& pages, int key_lo, int key_end,
                                       KFrag<HD>& f) {
    constexpr int DC = (HD + 31) / 32;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g4 = lane >> 4;
    const unsigned lane_off = r * HD + g4 * 8;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        const int h0 = t0 + hf * 16;
        const bf16* base = kv.k + static_cast<size_t>(pages.pg[hf]) * kv.page_stride + kv.head_off +
                           static_cast<size_t>(page_of(kv, h0).offset) * HD;                    // scalar
        const int t = h0 + r;
        const bool key_ok = FULL || (t >= key_lo && t < key_end);
#pragma unroll
        for (int c = 0; c < DC; ++c) {
            if (HD % 32 != 0 && c == DC - 1) {       // the last 32 dims are half there: lanes of the upper half hold zeros
                f.kf[hf][c] = (key_ok && g4 < 2) ? *reinterpret_cast<const bf16x8*>(base + lane_off + c * 32) : zero_frag();
            } else if (FULL) {
                const bf16x8* p = reinterpret_cast<const bf16x8*>(base + lane_off + c * 32);
                f.kf[hf][c] = STREAM ? __builtin_nontemporal_load(p) : *p;
            } else {
                f.kf[hf][c] = key_ok ? *reinterpret_cast<const bf16x8*>(base + lane_off + c * 32) : zero_frag();
            }
        }
    }
}

// The same for the V operand, read 4 keys (8 bytes) at a time from the transposed pages.
template <int HD, bool FULL, bool STREAM = false>
__device__ __forceinline__ void load_v(const PagedKV& kv, int t0, const BlockPages& pages, int key_lo, int key_end,
                                       VFrag<HD>& f) {
    constexpr int DT = HD / 16;
    const int lane = threadIdx.x & 63;
    const int r = lane & 15, g4 = lane >> 4;
    const unsigned lane_off = r * kv.page + g4 * 4;
    const bf16* base[2];
    bool ok[2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        const int h0 = t0 + hf * 16;
        base[hf] = kv.v + static_cast<size_t>(pages.pg[hf]) * kv.page_stride + kv.head_off + page_of(kv, h0).offset;
        const int t = h0 + g4 * 4;
        ok[hf] = FULL || (t + 3 >= key_lo && t < key_end);     // the 4 keys share a page with a visible key
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const unsigned off = lane_off + dt * 16 * kv.page;
        bf16x4 lo4, hi4;
#pragma unroll
        for (int e = 0; e < 4; ++e) lo4[e] = hi4[e] = static_cast<__bf16>(0.f);
        if (FULL && STREAM) {
            lo4 = __builtin_nontemporal_load(reinterpret_cast<const bf16x4*>(base[0] + off));
            hi4 = __builtin_nontemporal_load(reinterpret_cast<const bf16x4*>(base[1] + off));
        } else {
            if (FULL || ok[0]) lo4 = *reinterpret_cast<const bf16x4*>(base[0] + off);
            if (FULL || ok[1]) hi4 = *reinterpret_cast<const bf16x4*>(base[1] + off);
        }
        f.vf[dt] = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

// A row that has seen no key yet has this reference maximum: any visible score lies far above it,
// so the first visible key of a row always moves the reference.
constexpr float kNoMax = -1.0e30f;

// The scores of one 32-key block for QT row tiles: s[qt][hf] = K (16 keys of half hf) x Q^T.
template <int HD, int QT>
__device__ __forceinline__ void block_scores(const KFrag<HD>& f, const bf16x8 (&qf)[QT][(HD + 31) / 32],
                                             f32x4 (&s)[QT][2]) {
    constexpr int DC = (HD + 31) / 32;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            s[qt][hf] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c32 = 0; c32 < DC; ++c32)
                s[qt][hf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.kf[hf][c32], qf[qt][c32], s[qt][hf], 0, 0, 0);
        }
}

// Softmax weights of one block from its scores, as the second product's first operand. This
// lane holds row r of tile qt and the keys t0 + 16 hf + 4 g4 + e. row_pos[qt]: position of the
// lane's row, or -1 for a row that does not exist; row_lo[qt]: first key the row may see;
// tile_free[qt]: the last key every row of tile qt sees without a check (the position of its
// first row if all 16 rows exist and there is no window, else -1): blocks that end at or
// before it skip the masking. c = scale * log2(e) > 0; m is kept in units of c * score.
//
// The reference maximum m of a row moves only when a score exceeds it by more than kLazy (in
// powers of two): until then weights are at most 2^kLazy, well inside the range, and the sums
// need no rescaling; the softmax does not depend on which reference is subtracted. Whether any
// lane of the wavefront has such a score is one vote; only then are the row maxima reduced over
// the lanes and the sums rescaled, so the usual block costs per score one fused multiply-add,
// one exponential, one addition, half a conversion and half a maximum.
template <int HD, int QT>
__device__ __forceinline__ void block_weights(f32x4 (&s)[QT][2], int t0, const int (&row_pos)[QT],
                                              const int (&row_lo)[QT], const int (&tile_free)[QT], float c,
                                              float (&m)[QT], float (&l)[QT], f32x4 (&o)[QT][HD / 16],
                                              bf16x8 (&pf)[QT]) {
    constexpr int DT = HD / 16;
    const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        if (t0 + 31 > tile_free[qt]) {
            const int pos = row_pos[qt], lo = row_lo[qt];
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int t = t0 + hf * 16 + g4 * 4 + e;
                    s[qt][hf][e] = ((t <= pos) && (t >= lo)) ? s[qt][hf][e] : -INFINITY;
                }
        }
        float mx = fmaxf(fmaxf(s[qt][0][0], s[qt][0][1]), s[qt][0][2]);
        mx = fmaxf(fmaxf(mx, s[qt][0][3]), s[qt][1][0]);
        mx = fmaxf(fmaxf(mx, s[qt][1][1]), s[qt][1][2]);
        mx = fmaxf(mx, s[qt][1][3]);
        if (__any(fmaf(mx, c, -m[qt]) > kLazy)) {       // some row's maximum moves: rescale what is summed
            float mr = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mr = fmaxf(mr, __shfl_xor(mr, 32, 64));
            const float ms = mr * c;
            const float m_new = (ms > m[qt] + kLazy) ? ms : m[qt];
            const float alpha = fast_exp2(m[qt] - m_new);
            m[qt] = m_new;
            l[qt] *= alpha;
            float ar[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) ar[e] = __shfl(alpha, g4 * 4 + e, 64);     // factor of O's row 4 g4 + e
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[qt][dt][e] *= ar[e];
        }
        const float neg_m = -m[qt];
        float psum = 0.f;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const __bf16 p = static_cast<__bf16>(fast_exp2(fmaf(s[qt][hf][e], c, neg_m)));
                psum += static_cast<float>(p);          // (the sum of the weights as the product sees them)
                pf[qt][hf * 4 + e] = p;
            }
        l[qt] += psum;
    }
}

// One block on its own, loaded with checks: for the blocks at the edges of a range.
template <int HD, int QT>
__device__ __forceinline__ void attend_edge_block(const PagedKV& kv, int t0, int key_lo, int key_end,
                                                  const bf16x8 (&qf)[QT][(HD + 31) / 32], const int (&row_pos)[QT],
                                                  const int (&row_lo)[QT], const int (&tile_free)[QT],
                                                  float scale_log2, float (&m)[QT], float (&l)[QT],
                                                  f32x4 (&o)[QT][HD / 16]) {
    constexpr int DT = HD / 16;
    KFrag<HD> kf;
    VFrag<HD> vf;
    const BlockPages pg = lookup_pages(kv, t0, key_lo, key_end);
    load_k<HD, false>(kv, t0, pg, key_lo, key_end, kf);
    load_v<HD, false>(kv, t0, pg, key_lo, key_end, vf);
    f32x4 s[QT][2];
    block_scores<HD, QT>(kf, qf, s);
    bf16x8 pf[QT];
    block_weights<HD, QT>(s, t0, row_pos, row_lo, tile_free, scale_log2, m, l, o, pf);
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[qt], vf.vf[dt], o[qt][dt], 0, 0, 0);
}

// Walks the 32-key blocks t0 = first, first + stride, ... < key_end. A first block that begins
// before key_lo and a last block that ends behind key_end are taken on their own; the blocks
// between them lie inside the range whole and run in a loop without checks on the loads. There
// K and V each have one set of registers: the next block's K is asked for as soon as the scores
// are out, its V as soon as the second product is, so each load has most of a block's work to
// arrive in; page ids are looked up one block further ahead, so that no load waits for a table
// entry. The last turn asks for its own block once more instead of for nothing, and the lookups
// ahead are clamped to the table's last entry in use: the same loads on every turn.
template <int HD, int QT, bool STREAM = false>
__device__ __forceinline__ void attend_range(const PagedKV& kv, int first, int stride, int key_lo, int key_end,
                                             const bf16x8 (&qf)[QT][(HD + 31) / 32], const int (&row_pos)[QT],
                                             const int (&row_lo)[QT], const int (&tile_free)[QT], float scale_log2,
                                             float (&m)[QT], float (&l)[QT], f32x4 (&o)[QT][HD / 16]) {
    constexpr int DT = HD / 16;
    int t0 = first;
    if (t0 >= key_end) return;
    if (t0 < key_lo) {
        attend_edge_block<HD, QT>(kv, t0, key_lo, key_end, qf, row_pos, row_lo, tile_free, scale_log2, m, l, o);
        t0 += stride;
    }
    const int full_end = key_end - 31;                       // a block is full if t0 < full_end
    if (t0 < full_end) {
        const int last_half = (key_end - 1) & ~15;          // the last 16-key half that has a page
        KFrag<HD> kf;
        VFrag<HD> vf;
        BlockPages pg_cur = lookup_pages(kv, t0, key_lo, key_end);
        BlockPages pg_next;
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int h0 = min(t0 + stride + hf * 16, last_half);
            pg_next.pg[hf] = __builtin_amdgcn_readfirstlane(kv.table[page_of(kv, h0).block]);
        }
        load_k<HD, true, STREAM>(kv, t0, pg_cur, key_lo, key_end, kf);
        load_v<HD, true, STREAM>(kv, t0, pg_cur, key_lo, key_end, vf);
        for (; t0 < full_end; t0 += stride) {
            const bool more = t0 + stride < full_end;
            const int tn = more ? t0 + stride : t0;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                if (more) pg_cur.pg[hf] = pg_next.pg[hf];
                const int h0 = min(t0 + 2 * stride + hf * 16, last_half);
                pg_next.pg[hf] = __builtin_amdgcn_readfirstlane(kv.table[page_of(kv, h0).block]);
            }
            f32x4 s[QT][2];
            block_scores<HD, QT>(kf, qf, s);
            load_k<HD, true, STREAM>(kv, tn, pg_cur, key_lo, key_end, kf);
            bf16x8 pf[QT];
            block_weights<HD, QT>(s, t0, row_pos, row_lo, tile_free, scale_log2, m, l, o, pf);
#pragma unroll
            for (int qt = 0; qt < QT; ++qt)
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[qt], vf.vf[dt], o[qt][dt], 0, 0, 0);
            load_v<HD, true, STREAM>(kv, tn, pg_cur, key_lo, key_end, vf);
        }
    }
    if (t0 < key_end)                                        // one block that ends behind key_end
        attend_edge_block<HD, QT>(kv, t0, key_lo, key_end, qf, row_pos, row_lo, tile_free, scale_log2, m, l, o);
}

// Loads the query fragments of one 16-row tile: lane holds row r, dims c * 32 + 8 g4 ..
template <int HD>
__device__ __forceinline__ void load_q(const bf16* qrow, bool ok, bf16x8 (&qf)[(HD + 31) / 32]) {
    const int g4 = (threadIdx.x & 63) >> 4;
#pragma unroll
    for (int c = 0; c < (HD + 31) / 32; ++c) {
        const int d = c * 32 + g4 * 8;
        qf[c] = (ok && d < HD) ? *reinterpret_cast<const bf16x8*>(qrow + d) : zero_frag();
    }
}


// ------------------------------------------------------------------------------------------
// decode: one token per request. A workgroup's four wavefronts (the first DEC_WAVES of it) take
// one split of the keys of one (request s, kv head and tile of 16 query heads `head_tile`, split);
// they take every fourth 32-key block each and add up through LDS (sh: decode_lds_floats(HD)
// floats). A device function so that two kernels can hold it: the decode kernel, and the kernel
// that runs a step's prompt portions beside its decoded tokens in one launch.
constexpr int DEC_WAVES = 4;
__host__ __device__ constexpr int decode_lds_floats(int hd) { return DEC_WAVES * 16 * hd + 2 * DEC_WAVES * 16; }

// RAW: the step's q/k/v rows come as the projection left them, 32-bit and unrotated ([rows, (n_q + 2 n_kv)
// hd], full rotation, head size 64 or 128), and the workgroup does what the rotation kernel would have
// done for its request and kv head: it rotates its query heads into operand registers, rotates the new key,
// writes key and value into the request's page, and sets what it has read of the row to zero (the buffer
// is one that a product cut over k adds into). Only with a single split: every value of the row is then
// read by one workgroup. The cache is non-const here: the new key and value go into it.
struct RawQkv {
    float* qkv = nullptr;            // [rows, (n_q + 2 n_kv) hd]
    const float* cos_t = nullptr;    // [max_pos, hd / 2]
    const float* sin_t = nullptr;
    bf16* k_cache = nullptr;
    bf16* v_cache = nullptr;
};

// (k_cache and v_cache carry no promise that nothing else points at them: RAW writes into them)
template <int HD, bool STREAM, bool RAW = false>
__device__ __forceinline__ void decode_item(
    const bf16* __restrict__ q, const bf16* k_cache, const bf16* v_cache,
    bf16* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ q_start, const int* __restrict__ ctx_len, const int* __restrict__ block_table,
    int max_blocks, int n_q, int n_kv, int page, float scale, int window, int split_len, int nsplit, int s,
    int head_tile, int split, float* sh, const RawQkv& raw = RawQkv{}) {
    constexpr int DC = (HD + 31) / 32, DT = HD / 16;
    float (*sh_o)[16][HD] = reinterpret_cast<float (*)[16][HD]>(sh);
    float (*sh_m)[16] = reinterpret_cast<float (*)[16]>(sh + DEC_WAVES * 16 * HD);
    float (*sh_l)[16] = sh_m + DEC_WAVES;
    // What the walk over the keys needs first is asked for together, before anything depends on
    // it: the request's rows, its length, and the line of its block table that this split's first
    // page ids lie in (the walk's own lookups then find it in the cache). One after the other
    // these were three trips to memory in front of the first key.
    const int row0 = q_start[s], row1 = q_start[s + 1];
    const int pos = ctx_len[s];                         // the token's position; it sees keys lo..pos
    const long first_block = static_cast<long>(split) * split_len / page;
    const int table_line = block_table[static_cast<size_t>(s) * max_blocks +
                                       (first_block < max_blocks ? first_block : max_blocks - 1)];
    if (row1 - row0 != 1) return;                       // not a decoding request (whole workgroup)
    asm volatile("" ::"v"(table_line));                 // (the load is wanted for its effect on the cache)
    const int G = n_q / n_kv;
    const int gtiles = (G + 15) / 16;
    const int kvh = head_tile / gtiles, gt = head_tile % gtiles;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g4 = lane >> 4;

    const int lo_all = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    int k_begin = split * split_len, k_end = k_begin + split_len;
    if (k_end > pos + 1) k_end = pos + 1;
    if (k_begin < (lo_all & ~31)) k_begin = lo_all & ~31;

    const int head = kvh * G + gt * 16 + r;             // this lane's row is a query head
    const bool row_ok = (gt * 16 + r) < G;
    bf16x8 qf[1][DC];
    PagedKV kv{k_cache, v_cache, block_table + static_cast<size_t>(s) * max_blocks, page, n_kv, kvh, HD,
               page_magic_of(page), static_cast<unsigned>(n_kv) * page * HD, static_cast<unsigned>(kvh) * page * HD};
    if constexpr (RAW) {
        static_assert(!RAW || HD == 64 || HD == 128, "a lane holds a dim and its rotation partner");
        constexpr int HALF = HD / 2;
        float* qkv_row = raw.qkv + static_cast<size_t>(row0) * (n_q + 2 * n_kv) * HD;
        const float* cs = raw.cos_t + static_cast<size_t>(pos) * HALF;
        const float* sn = raw.sin_t + static_cast<size_t>(pos) * HALF;
        // a + b i -> (a c - b s) + (b c + a s) i, as the rotation kernel computes it, then rounded
        auto rotate8 = [&](const float* src, int d, bf16x8& lo, bf16x8& hi) {
            const float4 a0 = *reinterpret_cast<const float4*>(src + d), a1 = *reinterpret_cast<const float4*>(src + d + 4);
            const float4 b0 = *reinterpret_cast<const float4*>(src + d + HALF), b1 = *reinterpret_cast<const float4*>(src + d + HALF + 4);
            const float4 c0 = *reinterpret_cast<const float4*>(cs + d), c1 = *reinterpret_cast<const float4*>(cs + d + 4);
            const float4 s0 = *reinterpret_cast<const float4*>(sn + d), s1 = *reinterpret_cast<const float4*>(sn + d + 4);
            const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
            const float b[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            const float c[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
            const float sv[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                lo[j] = static_cast<__bf16>(a[j] * c[j] - b[j] * sv[j]);
                hi[j] = static_cast<__bf16>(b[j] * c[j] + a[j] * sv[j]);
            }
        };
        auto zero8 = [&](float* dst) {
            const float4 z{0.f, 0.f, 0.f, 0.f};
            reinterpret_cast<float4*>(dst)[0] = z;
            reinterpret_cast<float4*>(dst)[1] = z;
        };
        // the query heads: lane (r, g4) holds dims 32 c + 8 g4 .. of head r, c < DC / 2, and their partners
        float* qhead = qkv_row + static_cast<size_t>(row_ok ? head : 0) * HD;
#pragma unroll
        for (int c = 0; c < DC / 2; ++c) {
            bf16x8 lo, hi;
            rotate8(qhead, c * 32 + g4 * 8, lo, hi);
            qf[0][c] = row_ok ? lo : zero_frag();
            qf[0][c + DC / 2] = row_ok ? hi : zero_frag();
        }
        // the new key and value of this kv head: the first wavefront's lanes take 8 dims each
        const PagePlace at = page_of(kv, pos);
        const int pg = __builtin_amdgcn_readfirstlane(kv.table[at.block]);
        if (wave == 0) {
            float* krow = qkv_row + static_cast<size_t>(n_q + kvh) * HD;
            float* vrow = qkv_row + static_cast<size_t>(n_q + n_kv + kvh) * HD;
            if (lane < HALF / 8) {
                bf16x8 lo, hi;
                rotate8(krow, lane * 8, lo, hi);
                bf16* dst = raw.k_cache + static_cast<size_t>(pg) * kv.page_stride + kv.head_off +
                            static_cast<size_t>(at.offset) * HD + lane * 8;
                *reinterpret_cast<bf16x8*>(dst) = lo;
                *reinterpret_cast<bf16x8*>(dst + HALF) = hi;
                zero8(krow + lane * 8);
                zero8(krow + lane * 8 + HALF);
            } else if (lane >= 32 && lane < 32 + HD / 8) {
                const int d0 = (lane - 32) * 8;
                const float4 v0 = *reinterpret_cast<const float4*>(vrow + d0), v1 = *reinterpret_cast<const float4*>(vrow + d0 + 4);
                const float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                bf16* dst = raw.v_cache + static_cast<size_t>(pg) * kv.page_stride + kv.head_off +
                            static_cast<size_t>(d0) * page + at.offset;
#pragma unroll
                for (int j = 0; j < 8; ++j) dst[static_cast<size_t>(j) * page] = static_cast<__bf16>(v[j]);
                zero8(vrow + d0);
            }
        }
        __syncthreads();                                // the key and the value are in the page; every wavefront has read q
        if (wave == 0 && row_ok) {
#pragma unroll
            for (int c = 0; c < DC / 2; ++c) {
                zero8(qhead + c * 32 + g4 * 8);
                zero8(qhead + c * 32 + g4 * 8 + HALF);
            }
        }
    } else {
        load_q<HD>(q + (static_cast<size_t>(row0) * n_q + (row_ok ? head : 0)) * HD, row_ok, qf[0]);
    }
    const int row_pos[1] = {row_ok ? pos : -1};
    const int row_lo[1] = {lo_all};
    const int tile_free[1] = {-1};                      // few blocks, heads may be missing: always checked
    float m[1] = {kNoMax}, l[1] = {0.f};
    f32x4 o[1][DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[0][dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int first = k_begin + __builtin_amdgcn_readfirstlane(wave) * 32;
    attend_range<HD, 1, STREAM>(kv, first, DEC_WAVES * 32, lo_all, k_end, qf, row_pos, row_lo, tile_free,
                              scale * kLog2e, m, l, o);

    float lt = l[0];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (g4 == 0) {
        sh_m[wave][r] = m[0];
        sh_l[wave][r] = lt;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int e = 0; e < 4; ++e) sh_o[wave][g4 * 4 + e][dt * 16 + r] = o[0][dt][e];
    __syncthreads();
    // join the wavefronts: thread -> (row, dims)
    for (int item = threadIdx.x; item < 16 * HD; item += DEC_WAVES * 64) {
        const int row = item / HD, d = item % HD;
        if (gt * 16 + row >= G) continue;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) mx = fmaxf(mx, sh_m[w][row]);
        float acc = 0.f, lsum = 0.f;
#pragma unroll
        for (int w = 0; w < DEC_WAVES; ++w) {
            const float mw = sh_m[w][row];
            const float f = (mw <= kNoMax) ? 0.f : exp2f(mw - mx);
            acc += f * sh_o[w][row][d];
            lsum += f * sh_l[w][row];
        }
        const int h = kvh * G + gt * 16 + row;
        if (nsplit == 1) {
            out[(static_cast<size_t>(row0) * n_q + h) * HD + d] = static_cast<bf16>(acc / lsum);
        } else {
            const size_t pidx = (static_cast<size_t>(s) * n_q + h) * nsplit + split;
            part_o[pidx * HD + d] = acc;
            if (d == 0) {
                part_ml[pidx * 2] = mx;
                part_ml[pidx * 2 + 1] = lsum;
            }
        }
    }
}


// The prefill kernel that shares K and V blocks among a workgroup's wavefronts through LDS
// (attention_prefill.hip). rows_per_item: rows of one work item, see prefill_shared_rows; queue:
// two integers that are zero and that no other launch in flight uses. nsplit > 1: an item's keys
// are cut into key_runs(...) runs of `run` stretches; items with one run write out, the runs of
// the others go to part_o [rows, n_q, nsplit, hd] and part_ml [rows, n_q, nsplit, 2] (by batch
// row) and the caller joins them.
// beside: the same step's decoded tokens, for the launch to hold as well (blocks = 0: none): its
// first `blocks` workgroups each take one decode_item (read-once loads) and leave; the two kinds
// of work do not depend on each other, and each alone leaves most of the chip waiting for loads.
struct DecodeBeside {
    float* part_o = nullptr;
    float* part_ml = nullptr;
    int head_tiles = 0, split_len = 0, nsplit = 0;      // grid of the decode kernel: (n_seq, head_tiles, nsplit)
    int blocks = 0;                                     // n_seq * head_tiles * nsplit
};
int launch_prefill_shared(const bf16* q, const bf16* k_cache, const bf16* v_cache, bf16* out, const int* q_start,
                          const int* ctx_len, const int* block_table, int max_blocks, int n_seq, int n_q, int n_kv,
                          int hd, int page, float scale, int window, int items, int rows_per_item, int* queue,
                          int nsplit, int run, float* part_o, float* part_ml, int key_waves, const DecodeBeside& beside,
                          hipStream_t stream);

// Runs that the keys [k_begin, key_end) of a prefill work item are cut into: `run` stretches of 64
// keys each, at most max_runs (the last run then takes the rest).
__host__ __device__ __forceinline__ int key_runs(int k_begin, int key_end, int run, int max_runs) {
    const int stretches = (key_end - k_begin + 63) / 64;
    const int runs = (stretches + run - 1) / run;
    return runs < 1 ? 1 : (runs > max_runs ? max_runs : runs);
}
// Rows per work item of the shared kernel for these sizes, or 0 if it does not take them.
int prefill_shared_rows(int hd, int n_q, int n_kv);

}  // namespace llme
