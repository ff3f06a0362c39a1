// Decode-time projections fused with the RMSNorm in front of them (and, for the gated
// feed-forward, with the activation behind them), for up to 16 rows:
//
//   plain:  out[m, n]  = sum_k bf16((w_norm[k] * h[row(m), k]) * inv_m) * W[n, k]
//   gated:  out[m, j]  = silu(g) * u,  g, u = the same sums over the gate and the up row of unit j
//   inv_m = 1 / sqrt(mean_k h[row(m), k]^2 + eps)          (src/kernels.cpp:18-24, 26-31, 33-57)
//
// The activations enter the product as the norm kernel would have stored them: the normed value
// rounded to bfloat16, scale included. (Rounding bf16(w_norm * h) and scaling the 32-bit sums
// afterwards saves a pass over the row and is as accurate, but rounds other values than the norm
// kernel does: a token then gets other logits, within rounding, when it is decoded than when it
// is part of a prompt, and measured against one rounded reference the difference doubles.)
// h is the 32-bit residual stream, row(m) = rows ? rows[m] : m (the output head reads the wanted
// rows only).
//
// A workgroup first puts the normed rows into LDS, each wavefront taking its rows: sum of squares,
// scale, rounded values, while its first weight loads are already in flight. It then works
// through tiles of 16 output columns (gated: the 16 gate and the 16 up rows of 16 units, which
// lie next to each other in the interleaved weight matrix), TPR tiles at a time: NW / TPR
// wavefronts share a tile, each streaming every (NW / TPR)-th 128-element chunk of k of the
// tile's weight rows from HBM straight into MFMA operand registers, two chunks ahead (one with 16
// wavefronts), also across tiles; the partial sums are added through LDS and stored. The grid
// is sized so that the prologue is paid once per several tiles.
//
// A third form serves the attention's q/k/v projection: its epilogue rotates q and k heads at
// the rows' positions (pairs (i, i + hd/2), src/kernels.cpp:189-203) and writes q to the query
// buffer and k, v straight into the rows' cache pages, so that neither the 32-bit q/k/v rows
// nor a separate rotation kernel exist. For this form the weight rows of every q and k head
// come in another order (the caller's copy of the matrix for this kernel alone): the j-th group
// of 16 rows of a head holds dims 8 j .. 8 j + 7 and, behind them, their rotation partners
// hd/2 + 8 j .. hd/2 + 8 j + 7. A tile of 16 output columns then has both values of 8 pairs,
// a lane finds its partners in the lane 32 further on, and every tile is independent of the
// others, so the matrix is spread over as many workgroups as the plain form's.
//
// The weight matrix comes row-major ([rows, K]) or blocked: [rows / 16][K / 32] blocks of 1 KB,
// a block holding its 16 rows x 32 k in the order of the matrix instruction's operand (lane
// l = 16 q + r holds row r, k = 8 q .. 8 q + 7, so the block is [4 q][16 r][8]). A wavefront's
// load is then 1 KB of consecutive addresses instead of 16 pieces of 64 bytes a row apart, which
// streams a quarter faster from HBM (measured: 64 MB in 13.3 instead of 17.6 us).
//
// Limits (checked by the caller): M <= 16, K a multiple of 8, 16 * (K + 8) * 2 bytes of LDS;
// blocked: K a multiple of 32 and the weight rows a multiple of 16.
#include "common.h"
#include <math.h>

namespace llme {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

constexpr int kReadOnce = 2;            // a buffer load's cache policy: the non-temporal bit
constexpr int GV_U = 4;                 // 32-element k steps per chunk
constexpr int GV_CHUNK = 32 * GV_U;     // 128

__device__ __forceinline__ bf16x8 gv_zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.f);
    return z;
}

enum Epilogue : int { kPlain = 0, kGated = 1, kRope = 2 };

// Four neighbouring norm weights in one load (the entry point checks the vector's alignment),
// kept as loaded until they are used: a conversion right behind the load would wait for it.
template <typename T> struct Norm4;
template <> struct Norm4<float> {
    float4 v;
    __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
    __device__ __forceinline__ void get(float (&o)[4]) const { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
};
template <> struct Norm4<bf16> {
    bf16x4 v;
    __device__ __forceinline__ void load(const bf16* p) { v = *reinterpret_cast<const bf16x4*>(p); }
    __device__ __forceinline__ void get(float (&o)[4]) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = static_cast<float>(v[i]);
    }
};

// What the rotating epilogue needs: where rows sit in their requests and where their pages are.
struct RopeTarget {
    const int* positions;       // [M] position of each row's token
    const int* seq_idx;         // [M] request of each row (row of the block table)
    const int* block_table;     // [n_seq, max_blocks]
    int max_blocks;
    const float* cos_t;         // [max_pos, hd / 2]
    const float* sin_t;
    bf16* q_out;                // [M, n_q * hd]
    bf16* k_cache;              // [pages, n_kv, page, hd]
    bf16* v_cache;              // [pages, n_kv, hd, page]
    int n_q, n_kv, hd, page;
};

template <int NW, int TPR, int EPI, typename TNW, int PU = 8>
__global__ __launch_bounds__(NW * 64) void gemv_norm_kernel(const float* __restrict__ h, const int* __restrict__ rows,
                                                            const TNW* __restrict__ norm_w, float eps,
                                                            const bf16* __restrict__ w, void* __restrict__ out,
                                                            int M, int N, int K, int tiles, int blocked,
                                                            RopeTarget rope) {
    constexpr bool GATED = EPI == kGated;
    constexpr int NT = GATED ? 2 : 1;                   // weight fragments per k step
    constexpr int KS = NW / TPR;                        // wavefronts that share a tile, splitting k
    constexpr int GV_DEPTH = NW > 8 ? 1 : 2;             // chunks of weights a wavefront has in flight (measured: more stream more slowly)
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int XS = K + 8;                               // padded row of the activation tile (elements)
    bf16* xs = reinterpret_cast<bf16*>(lds_raw);                                    // [16][XS]
    f32x4* red = reinterpret_cast<f32x4*>(lds_raw + static_cast<size_t>(16) * XS * 2);   // [NW][NT][64]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int slot = wave / KS, kpart = wave % KS;      // which of the round's tiles, which share of k
    const int n_rows_w = GATED ? 2 * N : N;             // rows of the weight matrix
    const int n_chunks = (K + GV_CHUNK - 1) / GV_CHUNK;

    // The weights come by buffer loads: one descriptor over the whole matrix, a 32-bit byte offset
    // per lane. A tile or chunk that does not exist gets an offset behind the descriptor's end:
    // such a load returns zeros and fetches nothing, so loads can be issued without a condition.
    // (The matrix is smaller than 4 GB: the entry points check it.)
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16*>(w), 0, static_cast<unsigned>(static_cast<size_t>(n_rows_w) * K * 2), 0x00020000);
    constexpr unsigned kNowhere = 0xFFFFFFF0u;
    // GV_DEPTH sets of weight fragments, in use one after the other
    bf16x8 fw[GV_DEPTH][NT][GV_U];
    auto load_w = [&](bf16x8 (&f)[NT][GV_U], int tile, int chunk) {
        // weight rows of this lane: plain: n = 16 tile + r; gated: gate row 32 tile + r, up row 16 further
        // blocked: the 16-row group (NT t + tile's first), the 32-wide k block, 16 bytes per lane
        const int wr0 = GATED ? tile * 32 + r : tile * 16 + r;
        const int k0 = chunk * GV_CHUNK;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const bool w_ok = tile < tiles && chunk < n_chunks && (wr0 + 16 * t) < n_rows_w;
            const unsigned base = blocked
                ? (static_cast<unsigned>(tile * NT + t) * static_cast<unsigned>(K / 32)) * 1024u + lane * 16u
                : (static_cast<unsigned>(wr0 + 16 * t) * K + q * 8) * 2;
#pragma unroll
            for (int u = 0; u < GV_U; ++u) {
                const int kk = k0 + u * 32;
                // (all ones or zero, and the offset put together from both: written as a condition, the
                // compiler made two loads under a branch out of it, with a wait for everything between)
                const unsigned in = 0u - static_cast<unsigned>(w_ok && (kk + (blocked ? 0 : q * 8)) < K);
                const unsigned step = blocked ? static_cast<unsigned>(kk / 32) * 1024u : static_cast<unsigned>(kk) * 2;
                const unsigned off = ((base + step) & in) | (kNowhere & ~in);
                // (with the hint that the weights are read once: they pass the L2 without displacing
                // the activations, and stream measurably faster)
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, off, 0, kReadOnce);
                f[t][u] = __builtin_bit_cast(bf16x8, v);
            }
        }
    };
    // Which tile this wavefront works on in a round.
    const int tiles_per_head = (EPI == kRope) ? rope.hd / 16 : 1;
    auto tile_of = [&](int item) { return item * TPR + slot; };
    const int items = (tiles + TPR - 1) / TPR;
    // A wavefront's work in order: unit j is chunk kpart + (j % cpw) KS of the tile of round j / cpw.
    // Every wavefront has the same number of units (chunks past the end of k are zeros that cost
    // nothing), GV_DEPTH of them in flight: a unit's loads are issued GV_DEPTH units ahead, also
    // across rounds and before the prologue, so that the trip to memory is waited for once and not
    // once per chunk.
    const int rounds = (items + gridDim.x - 1) / gridDim.x;
    const int cpw = (n_chunks + KS - 1) / KS;
    const int units = rounds * cpw;
    auto unit_tile = [&](int j) { return j < units ? tile_of((j / cpw) * gridDim.x + blockIdx.x) : tiles; };
    auto unit_chunk = [&](int j) { return kpart + (j % cpw) * KS; };
    // ---- prologue: xs[m][k] = bf16((w_norm[k] * h[row(m)][k]) * inv_m) ----
    // Rows m >= M stay as they are: a product's row m depends on activation row m alone, and
    // the results of the rows that do not exist are never stored.
    // A row's loads are asked for eight at a time (one after the other, each trip to memory took
    // as long as the row's whole share of the products), and the first row's before the first
    // weights: loads come back in the order they were asked for, and the weights' come from far.
    // The rows are dealt out over the wavefronts: with fewer rows than wavefronts, several
    // wavefronts share a row (each takes every wpr-th group of 256 values) and add their sums of
    // squares through LDS. A wavefront's share of its row stays in registers from the sum of squares
    // to the rounding where it fits (PU loads of four values per lane); a longer share, or a second
    // row, is read again for the second pass, from the cache.
    // A row that fits one wavefront's registers is not shared: its sum of squares then needs no
    // trip through LDS and no barrier (measured at one row of 2,048: 0.9 us a kernel).
    const int Mp = M <= 1 ? 1 : M <= 2 ? 2 : M <= 4 ? 4 : M <= 8 ? 8 : 16;
    int wpr = 1;                                        // wavefronts that share a row
    while (K > 64 * 4 * PU * wpr && 2 * wpr * Mp <= NW) wpr *= 2;
    const int row_step = NW / wpr;                      // rows that the workgroup covers at a time
    const int seg = wave % wpr, m0 = wave / wpr;
    const int stride = 64 * 4 * wpr;                    // between a lane's neighbouring loads
    const int span = stride * PU;                       // values of a row that its wavefronts' registers hold
    const int kb0 = (seg * 64 + lane) * 4;
    float* ssq = reinterpret_cast<float*>(red);         // [16 rows][16 shares]; the area is free until the first round ends
    float4 hv[PU];
    Norm4<TNW> nw4[PU];
    auto ask = [&](int m, int kb) {
        const float* hrow = h + static_cast<size_t>(rows ? rows[m] : m) * K;
#pragma unroll
        for (int u = 0; u < PU; ++u) {
            const int k = kb + u * stride;
            const int ks = k < K ? k : 0;                          // past the row: a place that exists
            hv[u] = *reinterpret_cast<const float4*>(hrow + ks);
            nw4[u].load(norm_w + ks);
        }
    };
    auto squares = [&](int kb, float& ss) {
#pragma unroll
        for (int u = 0; u < PU; ++u) {
            const float4 v = hv[u];
            if (kb + u * stride < K) ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    };
    // xs = bf16((w_norm * h) * inv): the product and the order of its factors are the norm kernel's
    // (elementwise.hip), so a row is rounded to the same values whichever kernel norms it.
    auto take = [&](int m, int kb, float inv) {
        bf16* xrow = xs + static_cast<size_t>(m) * XS;
#pragma unroll
        for (int u = 0; u < PU; ++u) {
            const int k = kb + u * stride;
            if (k < K) {                                           // K % 8 == 0: whole groups of 4
                float nw[4];
                nw4[u].get(nw);
                const float4 v = hv[u];
                bf16x4 o;
                o[0] = static_cast<__bf16>((nw[0] * v.x) * inv);
                o[1] = static_cast<__bf16>((nw[1] * v.y) * inv);
                o[2] = static_cast<__bf16>((nw[2] * v.z) * inv);
                o[3] = static_cast<__bf16>((nw[3] * v.w) * inv);
                *reinterpret_cast<bf16x4*>(xrow + k) = o;
            }
        }
    };
    if (m0 < M) ask(m0, kb0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 0; d < GV_DEPTH; ++d) load_w(fw[d], unit_tile(d), unit_chunk(d));   // in flight during the prologue
    __builtin_amdgcn_sched_barrier(0);
    // (the first loads of the first row are taken apart from the loop: only straight-line code lets
    // the compiler count that the weights' loads, asked for later, may stay in flight)
    float ss_first = 0.f;
    if (m0 < M) squares(kb0, ss_first);
    const bool held = K <= span && m0 + row_step >= M;  // one row, and this wavefront's share of it is in its registers
    for (int m = m0; m < M; m += row_step) {
        float ss = m == m0 ? ss_first : 0.f;
        for (int kb = kb0 + (m == m0 ? span : 0); kb < K; kb += span) {
            ask(m, kb);
            squares(kb, ss);
        }
        ss = wave_sum(ss);
        if (lane == 0) ssq[m * 16 + seg] = ss;
    }
    if (wpr > 1) lds_barrier();                         // (the same for the whole workgroup; alone, a wavefront reads what it wrote)
    for (int m = m0; m < M; m += row_step) {
        float ss = 0.f;
        for (int i = 0; i < wpr; ++i) ss += ssq[m * 16 + i];        // (the same order in every wavefront of the row)
        const float inv = 1.0f / sqrtf(ss / static_cast<float>(K) + eps);
        for (int kb = kb0; kb < K; kb += span) {
            if (!held) ask(m, kb);
            take(m, kb, inv);
        }
    }
    lds_barrier();                                      // (waits for LDS only: the weights stay in flight)

    const bf16* xlane = xs + static_cast<size_t>(r) * XS + q * 8;      // row m = r of the activation tile
    f32x4 acc[NT];
    auto multiply = [&](const bf16x8 (&f)[NT][GV_U], int chunk) {
        const int k0 = chunk * GV_CHUNK;
#pragma unroll
        for (int u = 0; u < GV_U; ++u) {
            const int kk = k0 + u * 32;
            const bf16x8 fx = ((kk + q * 8) < K) ? *reinterpret_cast<const bf16x8*>(xlane + kk) : gv_zero8();
#pragma unroll
            for (int t = 0; t < NT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[t][u], fx, acc[t], 0, 0, 0);
        }
    };

#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    // Rotating epilogue: where this lane's row goes (its position, its page) is asked for now, and a
    // round's table values before its sums are added up: each is a trip to memory that the
    // epilogue would otherwise wait for one after the other at the kernel's very end.
    int row_pos = 0, row_page = 0;
    if (EPI == kRope && kpart == 0 && (lane & 15) < M) {
        row_pos = rope.positions[lane & 15];
        row_page = rope.block_table[static_cast<size_t>(rope.seq_idx[lane & 15]) * rope.max_blocks + row_pos / rope.page];
    }
    // the end of a round: the sums are added up, scaled and stored (further down)
    auto finish_round = [&](int round) {
        const int tile = tile_of(round * gridDim.x + blockIdx.x);
        float4 cs4 = float4{1.f, 1.f, 1.f, 1.f}, sn4 = float4{0.f, 0.f, 0.f, 0.f};
        if (EPI == kRope && kpart == 0 && tile < tiles && (lane & 15) < M &&
            tile / tiles_per_head < rope.n_q + rope.n_kv) {
            // (four neighbouring values, 16-byte aligned: hd / 2 and the index are multiples of 4)
            const size_t at = static_cast<size_t>(row_pos) * (rope.hd / 2) + (tile % tiles_per_head) * 8 + ((lane >> 4) & 1) * 4;
            cs4 = *reinterpret_cast<const float4*>(rope.cos_t + at);
            sn4 = *reinterpret_cast<const float4*>(rope.sin_t + at);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) red[(wave * NT + t) * 64 + lane] = acc[t];
        lds_barrier();
        // the first wavefront of each tile adds up: lane l holds row m = l % 16, columns 4 (l / 16) + e
        f32x4 s[NT];
        const int m = lane & 15;
        const bool leader = kpart == 0 && tile < tiles;
        if (leader) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                s[t] = acc[t];
                for (int wv = 1; wv < KS; ++wv) {
                    const f32x4 p = red[((wave + wv) * NT + t) * 64 + lane];
                    s[t][0] += p[0]; s[t][1] += p[1]; s[t][2] += p[2]; s[t][3] += p[3];
                }
            }
        }
        if (EPI == kRope) {
            // A tile of a q or k head holds dims 8 j .. 8 j + 7 of the first half in its columns 0 .. 7
            // and their partners in columns 8 .. 15: lanes 0 .. 31 hold first halves, and the lane 32
            // further on the partners of the same row. A tile of a v head holds 16 dims as they are.
            const int hd = rope.hd, half = hd / 2;
            const int head = tile < tiles ? tile / tiles_per_head : 0;      // among q heads, then k heads, then v heads
            const int j = tile % tiles_per_head, g = lane >> 4;
            const bool is_q = head < rope.n_q, is_k = !is_q && head < rope.n_q + rope.n_kv;
            float own[4], other[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                own[e] = leader ? s[0][e] : 0.f;
                other[e] = __shfl_xor(own[e], 32, 64);                       // (every lane of the wavefront takes part)
            }
            if (leader && m < M) {
                const int kvh = is_q ? 0 : (is_k ? head - rope.n_q : head - rope.n_q - rope.n_kv);
                const int off = row_pos % rope.page;
                const size_t page_off = (static_cast<size_t>(row_page) * rope.n_kv + kvh) * rope.page * hd;
                const float cs[4] = {cs4.x, cs4.y, cs4.z, cs4.w}, sns[4] = {sn4.x, sn4.y, sn4.z, sn4.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = own[e];
                    int d = j * 16 + g * 4 + e;                               // v heads: columns as they are
                    if (is_q || is_k) {
                        const int i = j * 8 + (g & 1) * 4 + e;                // index within the half
                        const float c = cs[e], sn = sns[e];
                        v = g < 2 ? own[e] * c - other[e] * sn : own[e] * c + other[e] * sn;
                        d = g < 2 ? i : half + i;
                    }
                    if (is_q) rope.q_out[(static_cast<size_t>(m) * rope.n_q + head) * hd + d] = static_cast<bf16>(v);
                    else if (is_k) rope.k_cache[page_off + static_cast<size_t>(off) * hd + d] = static_cast<bf16>(v);
                    else rope.v_cache[page_off + static_cast<size_t>(d) * rope.page + off] = static_cast<bf16>(v);
                }
            }
        } else if (leader && m < M) {
            const int c0 = tile * 16 + (lane >> 4) * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = c0 + e;
                if (c >= N) continue;
                if (GATED) {
                    const float g = s[0][e], u = s[NT - 1][e];
                    static_cast<bf16*>(out)[static_cast<size_t>(m) * N + c] =
                        static_cast<bf16>((g / (1.0f + expf(-g))) * u);
                } else {
                    static_cast<float*>(out)[static_cast<size_t>(m) * N + c] = s[0][e];
                }
            }
        }
        lds_barrier();
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    auto work = [&](int d, int j) {
        multiply(fw[d], unit_chunk(j));
        if (j % cpw == cpw - 1) finish_round(j / cpw);
    };
    // While more than GV_DEPTH units are left, every unit done is followed by the loads of the unit
    // GV_DEPTH further on (without a condition: the compiler's count of loads in flight stays exact;
    // a unit past the end reads zeros). The last GV_DEPTH units are only worked on.
    int j = 0;
    for (; j + GV_DEPTH < units; j += GV_DEPTH) {
#pragma unroll
        for (int d = 0; d < GV_DEPTH; ++d) {
            work(d, j + d);
            load_w(fw[d], unit_tile(j + d + GV_DEPTH), unit_chunk(j + d + GV_DEPTH));
        }
    }
#pragma unroll
    for (int d = 0; d < GV_DEPTH; ++d)
        if (j + d < units) work(d, j + d);                  // (the same for the whole workgroup)
}

template <int NW, int TPR, int EPI, typename TNW, int PU>
static int launch_gemv_norm_held(const float* h, const int* rows, const void* norm_w, float eps, const bf16* w, void* out,
                                 int M, int N, int K, int grid, int blocked, const RopeTarget& rope, hipStream_t stream) {
    const size_t lds = static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(NW) * (EPI == kGated ? 2 : 1) * 64 * 16 + 64;
    if (lds > 160 * 1024) return kErrUnsupported;
    auto kernel = gemv_norm_kernel<NW, TPR, EPI, TNW, PU>;
    static size_t granted = 0;                          // per instantiation
    if (lds > granted) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
        if (e != hipSuccess) return static_cast<int>(e);
        granted = lds;
    }
    const int tiles = (N + 15) / 16;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(NW * 64), lds, stream, h, rows, static_cast<const TNW*>(norm_w), eps,
                       w, out, M, N, K, tiles, blocked, rope);
    return launch_status();
}

template <int NW, int TPR, int EPI, typename TNW>
static int launch_gemv_norm(const float* h, const int* rows, const void* norm_w, float eps, const bf16* w, void* out,
                            int M, int N, int K, int grid, int blocked, const RopeTarget& rope, hipStream_t stream) {
    // Rows wider than 2,048 leave room for one workgroup per compute unit anyway (their LDS): eight
    // wavefronts then have the registers to hold twice as much of a row between the two passes of
    // the norm, and rows up to 4,096 wide are still read once.
    if (NW == 8 && K > 2048)
        return launch_gemv_norm_held<NW, TPR, EPI, TNW, NW == 8 ? 16 : 8>(h, rows, norm_w, eps, w, out, M, N, K, grid,
                                                                          blocked, rope, stream);
    return launch_gemv_norm_held<NW, TPR, EPI, TNW, 8>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, rope, stream);
}

template <int EPI, typename TNW>
static int launch_gemv_norm_shape(int tpr, const float* h, const int* rows, const void* norm_w, float eps,
                                  const bf16* w, void* out, int M, int N, int K, int grid, int blocked,
                                  hipStream_t stream) {
    const RopeTarget none{};
    // tpr: tiles at a time; 12 and 14: 2 and 4 tiles with 16 wavefronts instead of 8
    if (tpr == 11) return launch_gemv_norm<16, 1, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
    if (tpr == 12) return launch_gemv_norm<16, 2, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
    if (tpr == 14) return launch_gemv_norm<16, 4, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
    if (tpr >= 4) return launch_gemv_norm<8, 4, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
    if (tpr == 2) return launch_gemv_norm<8, 2, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
    return launch_gemv_norm<8, 1, EPI, TNW>(h, rows, norm_w, eps, w, out, M, N, K, grid, blocked, none, stream);
}

}  // namespace llme

using namespace llme;

// h [*, K] float32; rows: M indices into h or null; norm_w [K] (norm_dtype 0 float32, 1 bfloat16);
// w bfloat16: plain [N, K], gated [2 N, K] with gate and up rows interleaved in groups of 16;
// out: plain float32 [M, N], gated bfloat16 [M, N]. tpr (tiles a workgroup of 8 wavefronts works
// on at a time: 1, 2 or 4; 11, 12, 14: 1, 2, 4 tiles with 16 wavefronts) and grid (workgroups): 0 lets the
// entry point choose. blocked: w is
// stored in 1 KB blocks of 16 rows x 32 k (see the head of this file).
extern "C" int llme_gemv_norm(const float* h, const int* rows, const void* norm_w, int norm_dtype, float eps,
                              const void* w, void* out, int M, int N, int K, int gated, int tpr, int grid,
                              int blocked, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K <= 0 || K % 8 != 0) return kErrUnsupported;
    if (blocked && (K % 32 != 0 || N % 16 != 0)) return kErrUnsupported;
    if (reinterpret_cast<uintptr_t>(norm_w) % 16 != 0 || reinterpret_cast<uintptr_t>(h) % 16 != 0) return kErrUnsupported;
    if (static_cast<size_t>(16) * (K + 8) * 2 > 132 * 1024) return kErrUnsupported;
    if (gated && N % 16 != 0) return kErrUnsupported;
    const int tiles = (N + 15) / 16;
    if (static_cast<double>(gated ? 2 * N : N) * K * 2 >= 4294967296.0) return kErrUnsupported;   // 32-bit offsets
    if (tpr <= 0) {
        // few tiles: all 8 wavefronts on one tile, so that every tile has a workgroup of its own;
        // more tiles than compute units: 2 tiles at a time, 4 wavefronts each with several chunks of k
        tpr = tiles <= compute_units() ? 1 : 2;
        // (one tile per workgroup: 16 wavefronts on it where their sums fit into LDS, see the rotating form)
        if (tpr == 1 && static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(16) * 2 * 64 * 16 + 64 <= 160 * 1024) tpr = 11;
        // (measured: 16 wavefronts on 2 tiles, 14.2 against 14.8 us at 512 tiles; they need more LDS for their sums)
        const size_t lds16 = static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(16) * 2 * 64 * 16 + 64;
        if (gated && tiles > compute_units() && tiles <= 4 * compute_units() && lds16 <= 160 * 1024) tpr = 12;
    }
    if (tpr != 1 && tpr != 2 && tpr != 4 && tpr != 11 && tpr != 12 && tpr != 14) return kErrBadArgument;
    if (grid <= 0) {
        const int at_a_time = tpr > 10 ? tpr - 10 : tpr;
        grid = (tiles + at_a_time - 1) / at_a_time;
        // As many workgroups as the chip holds at once, each going through several rounds of tiles: two per
        // compute unit, or one where the activation tile leaves LDS for one only (rows of 2,560 values and
        // more). Workgroups beyond that would start when others end and pay the norm in front again (the 8B
        // sizes' gate/up, 896 tiles of k = 4,096 at 8 rows: 47.4 us with 448 workgroups, 43.2 with 256).
        const size_t lds = static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(tpr > 10 ? 16 : 8) * (gated ? 2 : 1) * 64 * 16 + 64;
        const int resident = (2 * lds <= 160 * 1024 ? 2 : 1) * compute_units();
        if (grid > resident) grid = resident;
    }
    const bf16* W = static_cast<const bf16*>(w);
    if (norm_dtype == kBF16) {
        return gated ? launch_gemv_norm_shape<kGated, bf16>(tpr, h, rows, norm_w, eps, W, out, M, N, K, grid, blocked, stream)
                     : launch_gemv_norm_shape<kPlain, bf16>(tpr, h, rows, norm_w, eps, W, out, M, N, K, grid, blocked, stream);
    }
    if (norm_dtype == kF32) {
        return gated ? launch_gemv_norm_shape<kGated, float>(tpr, h, rows, norm_w, eps, W, out, M, N, K, grid, blocked, stream)
                     : launch_gemv_norm_shape<kPlain, float>(tpr, h, rows, norm_w, eps, W, out, M, N, K, grid, blocked, stream);
    }
    return kErrBadArgument;
}

// The q/k/v projection of up to 16 rows with the norm in front and rotation plus cache write
// behind: h [M, K] float32 (row m is batch row m), w [(n_q + 2 n_kv) hd, K] bfloat16 (q heads, k
// heads, v heads; within every q and k head the rows in the order dims 0 .. 7, hd/2 .. hd/2 + 7,
// 8 .. 15, hd/2 + 8 .. hd/2 + 15, ..: see the head of this file), cos/sin [max_pos, hd / 2];
// writes q_out [M, n_q hd] and the rows' k, v into the pages that block_table[seq_idx[m]] names
// for positions[m], all in the usual order of dims. Full rotation only (all hd dimensions), hd a
// multiple of 16.
extern "C" int llme_gemv_norm_rope(const float* h, const void* norm_w, int norm_dtype, float eps, const void* w,
                                   const int* positions, const int* seq_idx, const int* block_table, int max_blocks,
                                   const float* cos_t, const float* sin_t, void* q_out, void* k_cache, void* v_cache,
                                   int M, int K, int n_q, int n_kv, int hd, int page, int grid, int blocked,
                                   hipStream_t stream) {
    if (M <= 0) return 0;
    if (blocked && K % 32 != 0) return kErrUnsupported;
    if (reinterpret_cast<uintptr_t>(norm_w) % 16 != 0 || reinterpret_cast<uintptr_t>(h) % 16 != 0) return kErrUnsupported;
    if (M > 16 || K <= 0 || K % 8 != 0 || hd <= 0 || hd % 16 != 0 || n_q <= 0 || n_kv <= 0 || page <= 0)
        return kErrUnsupported;
    if (reinterpret_cast<uintptr_t>(cos_t) % 16 != 0 || reinterpret_cast<uintptr_t>(sin_t) % 16 != 0)
        return kErrUnsupported;                        // the tables are read four values at a time
    if (static_cast<size_t>(16) * (K + 8) * 2 > 132 * 1024) return kErrUnsupported;
    const int N = (n_q + 2 * n_kv) * hd;
    if (static_cast<double>(N) * K * 2 >= 4294967296.0) return kErrUnsupported;   // 32-bit offsets into w
    const int tiles = N / 16;
    const int tpr = tiles <= compute_units() ? 1 : 2;  // as the plain form
    if (grid <= 0) {
        // (as many workgroups as the chip holds at once, as in the plain form)
        const size_t lds = static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(8) * 64 * 16 + 64;
        const int resident = (2 * lds <= 160 * 1024 ? 2 : 1) * compute_units();
        grid = (tiles + tpr - 1) / tpr > resident ? resident : (tiles + tpr - 1) / tpr;
    }
    const RopeTarget rope{positions, seq_idx, block_table, max_blocks, cos_t, sin_t, static_cast<bf16*>(q_out),
                          static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache), n_q, n_kv, hd, page};
    const bf16* W = static_cast<const bf16*>(w);
    if (norm_dtype != kBF16 && norm_dtype != kF32) return kErrBadArgument;
    if (tpr == 1) {
        // One tile per workgroup leaves a compute unit to one workgroup: 16 wavefronts then norm up to
        // 16 rows in one go (a row each) and cut k finer (measured at 192 tiles of k = 2,048, plain
        // epilogue: 4.39 against 4.61 us at 1 row, 5.75 against 5.95 at 8, 7.12 against 8.88 at 16).
        const size_t lds16 = static_cast<size_t>(16) * (K + 8) * 2 + static_cast<size_t>(16) * 64 * 16 + 64;
        if (lds16 <= 160 * 1024)
            return norm_dtype == kBF16
                ? launch_gemv_norm<16, 1, kRope, bf16>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream)
                : launch_gemv_norm<16, 1, kRope, float>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream);
        return norm_dtype == kBF16
            ? launch_gemv_norm<8, 1, kRope, bf16>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream)
            : launch_gemv_norm<8, 1, kRope, float>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream);
    }
    return norm_dtype == kBF16
        ? launch_gemv_norm<8, 2, kRope, bf16>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream)
        : launch_gemv_norm<8, 2, kRope, float>(h, nullptr, norm_w, eps, W, nullptr, M, N, K, grid, blocked, rope, stream);
}

LLME_LOAD_ENTRY(gemv_fused)
