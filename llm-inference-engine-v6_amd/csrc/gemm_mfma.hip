// out[m, n] (+)= sum_k a[m, k] * w[n, k] for bfloat16 operands on the matrix cores
// (v_mfma_f32_16x16x32_bf16), 32-bit accumulation. Reference for the operation:
// src/kernels.cpp:33-57 (W is [N, K] row-major, so both operands are contiguous in k).
//
// Two kernels:
//  * tile kernel, for many rows (prompt portions): a workgroup of four wavefronts makes a
//    128 x 128 tile, each wavefront 64 x 64 as 4 x 4 MFMA tiles; k advances in slabs of 64
//    through two LDS buffers, the next slab's global loads in flight during the products.
//  * skinny kernel, for up to 64 rows (decoding): the weight matrix is streamed once from
//    HBM straight into MFMA operand registers; a workgroup owns 16 output columns and its
//    wavefronts split k between them (interleaved 128-element chunks), then add up
//    through LDS. Many wavefronts with several 16-byte loads in flight each are what
//    keeps HBM busy when there is almost no arithmetic.
//
// Operand layout of the 16x16x32 instruction (wavefront lane l, r = l % 16, q = l / 16):
// the first operand holds row r, k = 8q..8q+7 of a 16 x 32 block; the second holds column
// r, k = 8q..8q+7 of a 32 x 16 block; the result holds column r, rows 4q..4q+3. Since both
// operands are contiguous in k, a lane's 8 values are one 16-byte load.
//
// K must be a multiple of 8 and all pointers 16-byte aligned (checked by the caller);
// M and N are arbitrary: rows and columns past the edge are loaded as zeros and not stored.
//
// W comes row-major or blocked: [N / 16][K / 32] blocks of 1 KB, a block holding its 16 rows x
// 32 k in the order of the instruction's operand, [4 q][16 r][8] (N a multiple of 16, K of 32).
// A wavefront's load of an operand is then 1 KB of consecutive addresses, which is what lets
// the skinny kernel stream weights a quarter faster; the tile kernel reads the same layout,
// a slab of a tile being whole blocks, and puts it into LDS as rows as before.
#include "common.h"

namespace llme {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 zero8() {
    bf16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = static_cast<__bf16>(0.f);
    return z;
}

__device__ __forceinline__ bf16x8 load8(const bf16* p, bool ok) {
    return ok ? *reinterpret_cast<const bf16x8*>(p) : zero8();
}
// The same with the hint that the data is read once (the weights of a product with few rows).
__device__ __forceinline__ bf16x8 load8_once(const bf16* p, bool ok) {
    return ok ? __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p)) : zero8();
}

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
// The fourth word of a buffer descriptor for raw 32-bit data on this chip.
constexpr int kBufferFlags = 0x00020000;

enum OutMode : int { kStoreF32 = 0, kAddF32 = 1, kStoreBF16 = 2, kAtomicF32 = 3, kGatedBF16 = 4, kRopeCache = 5 };

// Where the q/k/v projection's epilogue (kRopeCache) puts its result: the columns are the heads
// of q, then k, then v (hd columns each); q and k heads are rotated at the rows' positions (pairs
// (i, i + hd / 2), src/kernels.cpp:189-203), q goes to q_out [M, n_q hd], k and v into the rows'
// cache pages (k_cache [pages, n_kv, page, hd], v_cache [pages, n_kv, hd, page]), all bfloat16.
struct QkvTarget {
    const float* cos_t;         // [max_pos, hd / 2]
    const float* sin_t;
    const int* positions;       // [M]
    const int* seq_idx;         // [M] row of the block table
    const int* block_table;     // [n_seq, max_blocks]
    int max_blocks;
    bf16* q_out;
    bf16* k_cache;
    bf16* v_cache;
    int n_q, n_kv, hd, page;
};

// ----------------------------------------------------------------------------------------
// tile kernel: a workgroup of 2 x 2 wavefronts makes a (32 WMT) x (32 WNT) tile of the output,
// each wavefront WMT x WNT MFMA tiles of 16 x 16. Larger wavefront tiles read fewer LDS bytes
// per product (the 64 x 64 wavefront tile is bound by LDS reads); smaller tiles give more
// workgroups when the output is small.
constexpr int TK = 64;
constexpr int TSTRIDE = TK + 16;                     // elements; 160-byte rows measured fastest (144 had bank conflicts)

template <int WMT, int WNT>
constexpr int tile_lds_bytes() { return 2 * (32 * WMT + 32 * WNT) * TSTRIDE * 2; }   // A and W, two buffers

// Kinds of instruction for the compiler's scheduler, and a hint for it: the next COUNT matrix
// products with one instruction of KIND behind each.
constexpr int kMfma = 0x008, kVmemRead = 0x020, kDsRead = 0x100, kDsWrite = 0x200;
template <int KIND, int COUNT>
__device__ __forceinline__ void deal_between_products() {
#pragma unroll
    for (int i = 0; i < COUNT; ++i) {
        __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
        __builtin_amdgcn_sched_group_barrier(KIND, 1, 0);
    }
}

// The end of a tile kernel: the wavefronts' accumulators go to `out` in the kernel's mode. The
// result tile (i, j) of a lane is column wn + 16 j + r, rows wm + 16 i + 4 q + e: written straight
// from there, a store instruction touches 4 rows with 64 bytes each. Where the tile fits into the
// LDS that the operand slabs no longer need (LDS_BYTES of it; the caller has passed a barrier), it
// goes through LDS instead, so that every thread stores 16 contiguous bytes of a row.
// The values that an adding epilogue adds to, asked for before the tile's last products and the
// staging (a thread's pieces of four in the order in which the staged epilogue takes them): their
// trip from memory is over when the sums are staged. (Measured at 2,048 rows: the adding down-proj
// of the 1B sizes took 6 us more than the storing one, o-proj 2 us.)
template <int BM, int BN, int NT>
struct AddendsAhead {
    static constexpr int PER_ROW = BN / 4, COUNT = (BM * PER_ROW + NT - 1) / NT;
    float4 v[COUNT];
    __device__ __forceinline__ void load(const void* out, int M, int N, int m0, int n0, int tid) {
#pragma unroll
        for (int it = 0; it < COUNT; ++it) {
            const int idx = tid + it * NT;
            const int m = m0 + idx / PER_ROW, n = n0 + (idx % PER_ROW) * 4;
            const bool in = idx < BM * PER_ROW && m < M && n < N;
            // (N is a multiple of 8 here: a piece of four is in or out whole; out: a place that exists)
            v[it] = *reinterpret_cast<const float4*>(static_cast<const float*>(out) + (in ? static_cast<size_t>(m) * N + n : 0));
        }
    }
};

// Where row m0 + tid of the tile goes (rotating epilogue): its position and the page that holds it,
// looked up by thread tid while the products run (see the kernel).
struct RowPlace {
    int pos = 0, page = 0;
};

template <int WMT, int WNT, int MODE, int LDS_BYTES, int WR = 2, int WC = 2, bool AHEAD = false>
__device__ __forceinline__ void tile_epilogue(f32x4 (&acc)[WMT][WNT], unsigned char* lds_raw, void* __restrict__ out,
                                              int M, int N, int m0, int n0, int wm, int wn, int tid, int r, int q,
                                              const QkvTarget& qt = QkvTarget{},
                                              const AddendsAhead<WR * 16 * WMT, WC * 16 * WNT, 64 * WR * WC>& ahead = {},
                                              const RowPlace& place = RowPlace{}) {
    constexpr int BM = WR * 16 * WMT, BN = WC * 16 * WNT, NT = 64 * WR * WC;

    constexpr int SS = BN + 4;                           // floats per staged row
    // A tile that is larger than the LDS goes through it in 2 or 4 passes of whole wavefront rows.
    constexpr int WAVE_ROWS = 16 * WMT;
    constexpr auto fits = [](int passes) {
        return (BM / passes) % WAVE_ROWS == 0 && static_cast<size_t>(BM / passes) * SS * 4 <= static_cast<size_t>(LDS_BYTES);
    };
    constexpr int PASSES = fits(1) ? 1 : (WR % 2 == 0 && fits(2)) ? 2 : (WR % 4 == 0 && fits(4)) ? 4 : 0;
    // (Atomic adds are faster scattered than packed into the same cache lines: they stay direct.)
    constexpr bool STAGED = MODE != kAtomicF32 && PASSES > 0;
    if (STAGED && N % 8 == 0) {
        constexpr int HB = PASSES > 0 ? BM / (PASSES > 0 ? PASSES : 1) : BM;     // rows of a pass
        float* stage = reinterpret_cast<float*>(lds_raw);
        // the rows' positions and pages, behind the stage: [BM] each (the rotating epilogue has one pass)
        int* row_pos = reinterpret_cast<int*>(lds_raw + static_cast<size_t>(HB) * SS * 4);
        int* row_page = row_pos + BM;
        if (MODE == kRopeCache) {
            static_assert(MODE != kRopeCache || (PASSES == 1 && static_cast<size_t>(BM) * SS * 4 + BM * 8 <= static_cast<size_t>(LDS_BYTES)),
                          "the rows' places fit behind the stage");
            if (tid < BM) {
                row_pos[tid] = place.pos;
                row_page[tid] = place.page;
            }
        }
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
        if (pass > 0) __syncthreads();                  // the pass before has been stored
        if (wm / HB == pass) {
#pragma unroll
            for (int i = 0; i < WMT; ++i)
#pragma unroll
                for (int j = 0; j < WNT; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        stage[(wm - pass * HB + i * 16 + q * 4 + e) * SS + wn + j * 16 + r] = acc[i][j][e];
        }
        __syncthreads();
        const int mp = m0 + pass * HB;                  // the pass's first row
        if (MODE == kRopeCache) {
            // The tile holds whole heads (the entry point chose it so). q and k heads: a thread takes 8
            // dims of a head's first half and their partners in the second, of one row.
            const int hd = qt.hd, half = hd / 2, hv = half / 8, rotated = qt.n_q + qt.n_kv;
            const int per_row = (BN / hd) * hv;
            for (int idx = tid; idx < HB * per_row; idx += NT) {
                const int row = idx / per_row, e = idx % per_row;
                const int hh = e / hv, i = (e % hv) * 8;
                const int m = mp + row, head = n0 / hd + hh;
                if (m >= M || head >= rotated) continue;
                const float* sp = stage + row * SS + hh * hd + i;
                const int pos = row_pos[row];
                const float* cs = qt.cos_t + static_cast<size_t>(pos) * half + i;
                const float* sn = qt.sin_t + static_cast<size_t>(pos) * half + i;
                bf16x8 lo, hi;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float a = sp[j], b = sp[half + j], c = cs[j], sv = sn[j];
                    lo[j] = static_cast<__bf16>(a * c - b * sv);
                    hi[j] = static_cast<__bf16>(b * c + a * sv);
                }
                bf16* dst;
                if (head < qt.n_q) {
                    dst = qt.q_out + (static_cast<size_t>(m) * qt.n_q + head) * hd + i;
                } else {
                    const int pg = row_page[row];
                    dst = qt.k_cache + ((static_cast<size_t>(pg) * qt.n_kv + (head - qt.n_q)) * qt.page + pos % qt.page) * hd + i;
                }
                *reinterpret_cast<bf16x8*>(dst) = lo;
                *reinterpret_cast<bf16x8*>(dst + half) = hi;
            }
            // v heads: a thread takes one dim of 16 consecutive rows. Where these are 16 consecutive
            // positions of one request that begin at a multiple of 16 (the usual case in a prompt) they
            // lie together in the transposed page and go out as one piece; otherwise one by one.
            for (int idx = tid; idx < (HB / 16) * BN; idx += NT) {
                const int g16 = idx / BN, col = idx % BN;
                const int n = n0 + col, head = n / hd;
                const int mg = mp + g16 * 16;
                if (head < rotated || n >= N || mg >= M) continue;
                const int kvh = head - rotated, d = n % hd;
                const int nt = M - mg < 16 ? M - mg : 16;
                const float* sp = stage + (g16 * 16) * SS + col;
                // (a page belongs to one request: the same page and 15 positions further on is the same request)
                const int pos0 = row_pos[g16 * 16];
                const bool together = nt == 16 && row_page[g16 * 16] == row_page[g16 * 16 + 15] && pos0 % 16 == 0 &&
                                      qt.page % 16 == 0 && row_pos[g16 * 16 + 15] == pos0 + 15;
                if (together) {
                    const int pg = row_page[g16 * 16];
                    bf16* dst = qt.v_cache + ((static_cast<size_t>(pg) * qt.n_kv + kvh) * hd + d) * qt.page + pos0 % qt.page;
                    bf16x8 lo, hi;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        lo[j] = static_cast<__bf16>(sp[j * SS]);
                        hi[j] = static_cast<__bf16>(sp[(j + 8) * SS]);
                    }
                    *reinterpret_cast<bf16x8*>(dst) = lo;
                    *reinterpret_cast<bf16x8*>(dst + 8) = hi;
                } else {
                    for (int j = 0; j < nt; ++j) {
                        const int pos = row_pos[g16 * 16 + j];
                        const int pg = row_page[g16 * 16 + j];
                        qt.v_cache[((static_cast<size_t>(pg) * qt.n_kv + kvh) * hd + d) * qt.page + pos % qt.page] =
                            static_cast<__bf16>(sp[j * SS]);
                    }
                }
            }
        } else if (MODE == kGatedBF16) {
            // a thread makes 8 units: their gates and ups lie 16 columns apart in a group of 32
            constexpr int PER_ROW = BN / 16;             // 8-unit pieces per row
            for (int idx = tid; idx < HB * PER_ROW; idx += NT) {
                const int row = idx / PER_ROW, piece = idx % PER_ROW;
                const int col = (piece / 2) * 32 + (piece % 2) * 8;
                const int m = mp + row, n = n0 + col;
                if (m >= M || n >= N) continue;
                const float* gp = stage + row * SS + col;
                bf16x8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float gt = gp[e], up = gp[16 + e];
                    o[e] = static_cast<__bf16>((gt / (1.0f + expf(-gt))) * up);
                }
                const int unit = (n0 + (piece / 2) * 32) / 2 + (piece % 2) * 8;
                *reinterpret_cast<bf16x8*>(static_cast<bf16*>(out) + static_cast<size_t>(m) * (N / 2) + unit) = o;
            }
        } else if (MODE == kStoreBF16) {
            constexpr int PER_ROW = BN / 8;
            for (int idx = tid; idx < HB * PER_ROW; idx += NT) {
                const int row = idx / PER_ROW, col = (idx % PER_ROW) * 8;
                const int m = mp + row, n = n0 + col;
                if (m >= M || n >= N) continue;
                const float* sp = stage + row * SS + col;
                bf16x8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<__bf16>(sp[e]);
                *reinterpret_cast<bf16x8*>(static_cast<bf16*>(out) + static_cast<size_t>(m) * N + n) = o;
            }
        } else if (MODE == kAddF32 && PASSES == 1 && AHEAD) {
            constexpr int PER_ROW = BN / 4;
#pragma unroll
            for (int it = 0; it < (BM * PER_ROW + NT - 1) / NT; ++it) {
                const int idx = tid + it * NT;
                const int row = idx / PER_ROW, col = (idx % PER_ROW) * 4;
                const int m = mp + row, n = n0 + col;
                if (idx >= BM * PER_ROW || m >= M || n >= N) continue;
                const float4 v = *reinterpret_cast<const float4*>(stage + row * SS + col);
                float4 cur = ahead.v[it];
                cur.x += v.x; cur.y += v.y; cur.z += v.z; cur.w += v.w;
                *reinterpret_cast<float4*>(static_cast<float*>(out) + static_cast<size_t>(m) * N + n) = cur;
            }
        } else {
            constexpr int PER_ROW = BN / 4;
            for (int idx = tid; idx < HB * PER_ROW; idx += NT) {
                const int row = idx / PER_ROW, col = (idx % PER_ROW) * 4;
                const int m = mp + row, n = n0 + col;
                if (m >= M || n >= N) continue;
                const float4 v = *reinterpret_cast<const float4*>(stage + row * SS + col);
                float* op = static_cast<float*>(out) + static_cast<size_t>(m) * N + n;
                if (MODE == kStoreF32) {
                    *reinterpret_cast<float4*>(op) = v;
                } else if (MODE == kAddF32) {
                    float4 cur = *reinterpret_cast<const float4*>(op);
                    cur.x += v.x; cur.y += v.y; cur.z += v.z; cur.w += v.w;
                    *reinterpret_cast<float4*>(op) = cur;
                } else {
                    atomicAdd(op, v.x); atomicAdd(op + 1, v.y); atomicAdd(op + 2, v.z); atomicAdd(op + 3, v.w);
                }
            }
        }
        }
        return;
    }
    if (MODE == kRopeCache) return;                     // (always staged: its columns are whole heads of 16 dims and more)
#pragma unroll
    for (int i = 0; i < WMT; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wm + i * 16 + q * 4 + e;
            if (m >= M) continue;
            if (MODE == kGatedBF16) {
#pragma unroll
                for (int j = 0; j + 1 < WNT; j += 2) {
                    const int unit = (n0 + wn + j * 16) / 2 + r;        // tile column pair (gate, up)
                    if (2 * unit >= N) continue;
                    const float gt = acc[i][j][e], up = acc[i][j + 1][e];
                    static_cast<bf16*>(out)[static_cast<size_t>(m) * (N / 2) + unit] =
                        static_cast<bf16>((gt / (1.0f + expf(-gt))) * up);
                }
            } else {
#pragma unroll
                for (int j = 0; j < WNT; ++j) {
                    const int n = n0 + wn + j * 16 + r;
                    if (n >= N) continue;
                    const size_t idx = static_cast<size_t>(m) * N + n;
                    const float v = acc[i][j][e];
                    if (MODE == kStoreF32) static_cast<float*>(out)[idx] = v;
                    else if (MODE == kAddF32) static_cast<float*>(out)[idx] += v;
                    else if (MODE == kAtomicF32) atomicAdd(static_cast<float*>(out) + idx, v);
                    else static_cast<bf16*>(out)[idx] = static_cast<bf16>(v);
                }
            }
        }
    }
}

// kGatedBF16: w holds gate and up rows interleaved in groups of 16, so that even MFMA tile
// columns are gates and odd ones the ups of the same 16 units; out [M, N / 2] bfloat16 gets
// silu(gate) * up (src/engine.cpp:213-216).
template <int WMT, int WNT, int MODE, bool KFULL, bool BLOCKED>
__global__ __launch_bounds__(256, 2) void gemm_tile_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                        void* __restrict__ out, int M, int N, int K,
                                                        int tiles_m, int tiles_n, int ksplit, QkvTarget qt) {
    constexpr int BM = 32 * WMT, BN = 32 * WNT;
    constexpr int A_ELEMS = BM * TSTRIDE, W_ELEMS = BN * TSTRIDE;
    constexpr int CA = BM / 32, CW = BN / 32;        // 16-byte chunks per thread and slab
    // The 64 x 64 tile serves products with up to 64 rows (decoding at large batches): one row of
    // tiles, so every weight is read once, and the loads say so (the non-temporal bit).
    constexpr int W_POLICY = (WMT == 2 && WNT == 2) ? 2 : 0;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    bf16* lds = reinterpret_cast<bf16*>(lds_raw);
    // buffers: sA[b] = lds + b * A_ELEMS, sW[b] = lds + 2 * A_ELEMS + b * W_ELEMS

    // Workgroups go to the chip's 8 dies in turn, each die with an L2 of its own: renumber so
    // that a die gets consecutive tiles; then tiles in groups of 8 tile rows, columns fastest
    // inside a group, so that workgroups that run together share rows of A and of W.
    const int per_split = tiles_m * tiles_n;
    int pid = blockIdx.x % per_split;
    const int split = blockIdx.x / per_split;
    if (per_split % 8 == 0) pid = (pid % 8) * (per_split / 8) + pid / 8;
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int g = pid / per_group;
    const int first_m = g * GROUP;
    const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
    const int tm = first_m + (pid % per_group) % gsize;
    const int tn = (pid % per_group) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int wm = (wave >> 1) * (16 * WMT), wn = (wave & 1) * (16 * WNT);

    // this workgroup's share of k (whole slabs)
    const int nk_all = (K + TK - 1) / TK;
    const int nk_per = (nk_all + ksplit - 1) / ksplit;
    const int kt_begin = split * nk_per;
    const int kt_end = (kt_begin + nk_per < nk_all) ? kt_begin + nk_per : nk_all;

    // global -> LDS: a slab of a tile is rows x 8 chunks of 16 bytes; thread t takes chunks t, t + 256, ..
    // The loads are buffer loads: a descriptor per matrix that begins at the tile's first row and
    // ends behind the tile's last row that exists, a 32-bit offset per lane and chunk that never
    // changes, and the slab's k offset as a scalar. Rows past the matrix lie behind the
    // descriptor's end and read as zeros without a check; slab numbers past the end read the
    // last slab again. Every turn of the loop thus issues the same loads, none under a branch,
    // and the counter of loads in flight tells exactly which slab has arrived. (A tile's rows
    // span fewer than 2^32 bytes: the entry point checks K.)
    const int crow = tid >> 3, ckq = (tid & 7) * 8;   // chunk i of a thread: row crow + 32 i, same k offset
    const int a_rows = M - m0 < BM ? M - m0 : BM, w_rows = N - n0 < BN ? N - n0 : BN;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16*>(a + static_cast<size_t>(m0) * K), 0, a_rows * K * 2, kBufferFlags);
    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16*>(w + static_cast<size_t>(n0) * K), 0, w_rows * K * 2, kBufferFlags);
    unsigned aoff[CA], woff[CW];                      // bytes
#pragma unroll
    for (int i = 0; i < CA; ++i) aoff[i] = (static_cast<unsigned>(crow + 32 * i) * K + ckq) * 2;
#pragma unroll
    for (int i = 0; i < CW; ++i) woff[i] = (static_cast<unsigned>(crow + 32 * i) * K + ckq) * 2;
    // Blocked W: a slab of the tile is (BN / 16) row groups x 2 blocks of 1 KB; chunk c = 256 i + t of
    // the slab is piece c % 64 of block (c % 128) / 64 of row group c / 128, so that a wavefront's
    // load is one whole block. In LDS the piece goes to row 16 (c / 128) + c % 16, k 32 (block) + 8 (c % 64 / 16).
    int w_lds[CW];                                    // elements from the slab's W buffer
    if (BLOCKED) {
#pragma unroll
        for (int i = 0; i < CW; ++i) {
            const int c = 256 * i + tid, group = c / 128, kb = (c % 128) / 64, piece = c % 64;
            woff[i] = (static_cast<unsigned>(group) * (K / 32) + kb) * 1024u + piece * 16u;
            w_lds[i] = (group * 16 + piece % 16) * TSTRIDE + kb * 32 + (piece / 16) * 8;
        }
    }
    struct Slab {
        u32x4 ra[CA], rw[CW];
    };
    auto load_global = [&](int kt, Slab& s) {
        if (kt >= kt_end) kt = kt_end - 1;
        const int k = kt * TK;
#pragma unroll
        for (int i = 0; i < CA; ++i) s.ra[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, aoff[i], k * 2, 0);
#pragma unroll
        for (int i = 0; i < CW; ++i)                  // (blocked: a slab is two blocks further in every row group)
            s.rw[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, woff[i], BLOCKED ? kt * 2048 : k * 2, W_POLICY);
        if (!KFULL) {                                 // K is a multiple of 8: a chunk is in or out whole
            const bool ok = k + ckq < K;
#pragma unroll
            for (int i = 0; i < CA; ++i) s.ra[i] = ok ? s.ra[i] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int i = 0; i < CW; ++i) {
                const bool w_ok = BLOCKED ? k + ((256 * i + tid) % 128) / 64 * 32 < K : ok;   // (a block is in or out whole)
                s.rw[i] = w_ok ? s.rw[i] : u32x4{0u, 0u, 0u, 0u};
            }
        }
    };
    auto store_lds = [&](int buf, const Slab& s) {
        bf16* sA = lds + buf * A_ELEMS;
        bf16* sW = lds + 2 * A_ELEMS + buf * W_ELEMS;
#pragma unroll
        for (int i = 0; i < CA; ++i) *reinterpret_cast<u32x4*>(sA + (crow + 32 * i) * TSTRIDE + ckq) = s.ra[i];
#pragma unroll
        for (int i = 0; i < CW; ++i)
            *reinterpret_cast<u32x4*>(sW + (BLOCKED ? w_lds[i] : (crow + 32 * i) * TSTRIDE + ckq)) = s.rw[i];
    };

    f32x4 acc[WMT][WNT];
#pragma unroll
    for (int i = 0; i < WMT; ++i)
#pragma unroll
        for (int j = 0; j < WNT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Slab j is computed from LDS buffer j % 2 and travels in register set j % 2. While slab j is
    // computed, j + 1 sits in its registers and j + 2 is in flight. A turn first puts j + 1 into
    // the other buffer and asks for j + 3, reads the fragments of its second half, multiplies the
    // first half (whose fragments the turn before has read), and only then meets the others at the
    // barrier: behind it, it reads the first fragments of slab j + 1 and multiplies its own second
    // half meanwhile. So no product waits for an LDS read that was issued right in front of it,
    // and the barrier (which waits for LDS only) is met with products still in the pipe.
    static_assert(TK == 64, "a turn is two halves of 32");
    bf16x8 fa0[WMT], fw0[WNT];                        // fragments of a slab's first half
    auto read_frags = [&](int buf, int kk, bf16x8 (&fa)[WMT], bf16x8 (&fw)[WNT]) {
        const bf16* sA = lds + buf * A_ELEMS;
        const bf16* sW = lds + 2 * A_ELEMS + buf * W_ELEMS;
#pragma unroll
        for (int i = 0; i < WMT; ++i)
            fa[i] = *reinterpret_cast<const bf16x8*>(sA + (wm + i * 16 + r) * TSTRIDE + kk * 32 + q * 8);
#pragma unroll
        for (int j = 0; j < WNT; ++j)
            fw[j] = *reinterpret_cast<const bf16x8*>(sW + (wn + j * 16 + r) * TSTRIDE + kk * 32 + q * 8);
    };
    auto multiply = [&](const bf16x8 (&fa)[WMT], const bf16x8 (&fw)[WNT]) {
#pragma unroll
        for (int i = 0; i < WMT; ++i)
#pragma unroll
            for (int j = 0; j < WNT; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
    };
    // Within a half, the compiler is told to deal the memory instructions out between the
    // products, one after each: a wavefront then uses LDS, the loads' path and the matrix pipe at
    // the same time all along, instead of in phases that the two workgroups of a compute unit
    // fall into together (measured: in phases, a call took the sum of the four pipes' times).
    auto turn = [&](int kt, int buf, Slab& next) {
        // (the store and the loads also on the last turn, where nobody uses them: a turn without
        // them would make the number of loads in flight depend on the path taken)
        bf16x8 fa1[WMT], fw1[WNT];
        read_frags(buf, 1, fa1, fw1);
        store_lds(buf ^ 1, next);
        multiply(fa0, fw0);
        deal_between_products<kDsRead, (WMT * WNT) / 2>();
        deal_between_products<kDsWrite, (WMT * WNT) / 2>();
        __builtin_amdgcn_sched_barrier(0);            // (the products stay in front of the barrier)
        lds_barrier();
        read_frags(buf ^ 1, 0, fa0, fw0);
        load_global(kt + 3, next);
        multiply(fa1, fw1);
        deal_between_products<kDsRead, (WMT * WNT) / 2>();
        deal_between_products<kVmemRead, (WMT * WNT) / 2>();
        __builtin_amdgcn_sched_barrier(0);
    };
    // Rotating epilogue: where the tile's rows go is looked up while the slabs travel: thread t asks
    // for row m0 + t's position and request in front of the first slab (they come from L2 and hold
    // nothing up) and for its page behind the second; the epilogue finds them in LDS. Looked up in
    // the epilogue, row by row, the two dependent trips were a fifth of the kernel at 273 rows.
    RowPlace place;
    int place_seq = 0;
    if (MODE == kRopeCache) {
        const int mrow = m0 + tid < M ? m0 + tid : M - 1;         // (every thread loads: no load under a condition)
        place.pos = qt.positions[mrow];
        place_seq = qt.seq_idx[mrow];
        __builtin_amdgcn_sched_barrier(0);
    }
    if (kt_begin < kt_end) {
        Slab s0, s1;
        // (the scheduling barriers keep the three slabs' loads in this order: the loop's waits
        // count on slab j + 1 being older than slab j + 2)
        load_global(kt_begin, s0);
        __builtin_amdgcn_sched_barrier(0);
        load_global(kt_begin + 1, s1);
        __builtin_amdgcn_sched_barrier(0);
        if (MODE == kRopeCache) {
            place.page = qt.block_table[static_cast<size_t>(place_seq) * qt.max_blocks + place.pos / qt.page];
            __builtin_amdgcn_sched_barrier(0);
        }
        store_lds(0, s0);
        load_global(kt_begin + 2, s0);
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier();
        read_frags(0, 0, fa0, fw0);
        // pairs of turns in a loop with one way round, then the odd turn: on every path into a
        // turn the loads in flight are the same, which keeps the compiler's waits exact
        int kt = kt_begin;
        for (int pair = (kt_end - kt_begin) / 2; pair > 0; --pair, kt += 2) {
            turn(kt, 0, s1);
            turn(kt + 1, 1, s0);
        }
        if ((kt_end - kt_begin) & 1) turn(kt, 0, s1);
    }
    // (an adding epilogue that goes through LDS in one pass has its addends asked for here)
    AddendsAhead<BM, BN, 256> addends;
    constexpr bool AHEAD = MODE == kAddF32 && static_cast<size_t>(BM) * (BN + 4) * 4 <= tile_lds_bytes<WMT, WNT>();
    if (AHEAD && N % 8 == 0) addends.load(out, M, N, m0, n0, tid);
    __syncthreads();                                  // the epilogue reuses the slabs' LDS
    tile_epilogue<WMT, WNT, MODE, tile_lds_bytes<WMT, WNT>(), 2, 2, AHEAD>(acc, lds_raw, out, M, N, m0, n0, wm, wn, tid, r, q,
                                                                           qt, addends, place);
}

// ----------------------------------------------------------------------------------------
// The tile kernel for wide outputs: tiles of 256 x 256 by eight wavefronts (64 x 128 each), whose slabs go
// from memory straight into LDS. On this chip a buffer load can name LDS as its destination, 16
// bytes per lane, lane l's bytes landing at the wavefront's LDS base + 16 l. A wavefront's load is
// thus 1 KB of consecutive LDS:
//  * W in the blocked layout: one operand block of the matrix instruction ([4 q][16 r][8]: lane
//    16 q + r holds row r, k = 8 q ..), lane l loading the block's bytes 16 l ..; a wavefront reads
//    it back as an operand with 1 KB of consecutive addresses.
//  * A is row-major: a load takes 8 rows x 64 k, whole 128-byte lines (16 rows x 32 k, a block's own
//    shape, touches twice as many lines per load: measured 856 against 963 TFLOP/s). Lane
//    32 kb + 8 q + r loads row r, k = 32 kb + 8 q .., so that LDS holds the chunk as [2 kb][4 q][8 r][8]:
//    the upper or lower half of two operand blocks. An operand's two halves (rows 0 .. 7 and 8 .. 15
//    of a block) lie in neighbouring chunks, 1 KB apart, in the same banks; so the odd chunks hold
//    their k quarters in the order 1, 0, 3, 2 (a lane of an odd chunk loads the neighbouring
//    quarter's k), and the two halves of a read fall into different banks without padding.
// No staging registers, no LDS-write instructions, no padding: that is what lets 160 KB of LDS hold
// a tile that loads half the bytes per product of a 128 x 128 one. (The same kernel at 128 x 128 and
// 256 x 128 was slower than the kernel above, which has three slabs in flight in registers; measured
// 822 and 812 against 954 TFLOP/s at 16,384 x 2,048.)
// LDS is cut into three buffers for A's slabs (64 k each) and four for halves of W's slabs (32 k:
// one block per 16 rows), so that A is asked for two slabs ahead and W three half slabs: with two
// buffers of whole slabs the loads, asked for one slab ahead, arrived late (from asking for A's
// 32 KB to having them takes 1.06 us, W's 1.4 us, a slab's products 1.1 us; 1,060 against 1,111
// TFLOP/s). The price is a barrier per half slab, at which a half buffer of W changes hands. The
// loads are counted by hand (nothing else of a turn goes through the vector memory path).
// Half turn h (k = 32 h ..) has its operands in registers when it starts. It waits for half slab
// h + 1, meets the barrier, asks for W's half slab h + 4 into the buffer of h, which everybody has
// read, and, if h is odd, for A's slab (h - 1) / 2 + 3 into the buffer of the slab that ends here;
// then it reads the operands of h + 1 while it multiplies.
// Needs: W blocked (N a multiple of 16, K of 32). A slab that hangs over the end of k reads zeros
// there (the loads of A's second half get an offset behind the descriptor's end).
constexpr int DK = 64;

// Waits until at most N of this wavefront's vector memory loads are still on their way.
template <int N> __device__ __forceinline__ void wait_vm() { __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14)); }

// A buffer descriptor for raw data, as four words (what __builtin_amdgcn_make_buffer_rsrc makes).
__device__ __forceinline__ u32x4 raw_descriptor(const void* base, unsigned bytes) {
    const unsigned long long p = reinterpret_cast<unsigned long long>(base);
    return u32x4{static_cast<unsigned>(p), static_cast<unsigned>(p >> 32) & 0xFFFFu, bytes, static_cast<unsigned>(kBufferFlags)};
}
// 16 bytes per lane from rsrc at voffset (per lane) + soffset (scalar), straight into LDS: lane l's
// bytes land at lds_base + 16 l (lds_base: the same in every lane, a byte address within LDS).
// Written as assembly because the compiler, which cannot tell which LDS reads such a load may
// alias, would wait for every load in flight in front of every LDS read.
__device__ __forceinline__ void load_b128_to_lds(u32x4 rsrc, unsigned lds_base, unsigned voffset, unsigned soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_base), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory", "m0");
}
template <int WR, int WC, int WMT, int WNT, int MODE>
__global__ __launch_bounds__(64 * WR * WC, 1) void gemm_tile_direct_kernel(
    const bf16* __restrict__ a, const bf16* __restrict__ w, void* __restrict__ out, int M, int N, int K, int tiles_m,
    int tiles_n, int ksplit, QkvTarget qt) {
    constexpr int BM = WR * 16 * WMT, BN = WC * 16 * WNT, NW = WR * WC;
    constexpr int AC = BM / 8, WB = BN / 16;                    // loads: chunks of a slab of A, blocks of half a slab of W
    static_assert(AC % NW == 0 && WB % NW == 0, "every wavefront has the same loads");
    constexpr int LA = AC / NW, LW = WB / NW;
    constexpr int NSA = 3, NHW = 4;
    constexpr int A_STAGE = AC * 1024, W_STAGE = WB * 1024, W_BASE = NSA * A_STAGE;
    static_assert(W_BASE + NHW * W_STAGE <= 160 * 1024, "LDS");
    static_assert(3 * LW + 2 * LA < 64, "the count of loads in flight has six bits");
    extern __shared__ __align__(16) unsigned char lds_raw[];

    const int per_split = tiles_m * tiles_n;
    int pid = blockIdx.x % per_split;
    const int split = blockIdx.x / per_split;
    if (per_split % 8 == 0) pid = (pid % 8) * (per_split / 8) + pid / 8;      // (a die gets consecutive tiles)
    constexpr int GROUP = 8;
    const int per_group = GROUP * tiles_n;
    const int g = pid / per_group;
    const int first_m = g * GROUP;
    const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
    const int tm = first_m + (pid % per_group) % gsize;
    const int tn = (pid % per_group) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, q = lane >> 4;
    const int wm = (wave / WC) * (16 * WMT), wn = (wave % WC) * (16 * WNT);

    // this workgroup's share of k, in half slabs (the shares are whole slabs, the last may end in a half)
    const int nh_all = K / 32;
    const int nk_all = (K + DK - 1) / DK;
    const int nk_per = (nk_all + ksplit - 1) / ksplit;
    const int h_begin = 2 * split * nk_per;
    const int h_end = (h_begin + 2 * nk_per < nh_all) ? h_begin + 2 * nk_per : nh_all;

    const int a_rows = M - m0 < BM ? M - m0 : BM, w_rows = N - n0 < BN ? N - n0 : BN;
    const u32x4 a_rsrc = raw_descriptor(a + static_cast<size_t>(m0) * K, static_cast<unsigned>(a_rows) * K * 2);
    const u32x4 w_rsrc = raw_descriptor(w + static_cast<size_t>(n0) * K, static_cast<unsigned>(w_rows) * K * 2);
    const unsigned lds_origin = static_cast<unsigned>(reinterpret_cast<size_t>(
        (__attribute__((address_space(3))) unsigned char*)lds_raw));
    constexpr unsigned kNowhere = 0xFFFFFF00u;
    unsigned a_off[LA], a_tail[LA], w_off[LW];
#pragma unroll
    for (int i = 0; i < LA; ++i) {
        // chunk j: rows 8 j .. 8 j + 7; lane 32 kb + 8 q' + r' loads row r', k = 32 kb + 8 q' (odd chunks: 8 (q' ^ 1))
        const int j = wave + NW * i;
        const int kb = lane >> 5, q8 = ((lane >> 3) & 3) ^ (j & 1), r8 = lane & 7;
        a_off[i] = (static_cast<unsigned>(j * 8 + r8) * K + kb * 32 + q8 * 8) * 2;
        a_tail[i] = kb == 0 ? a_off[i] : kNowhere;              // (row-major A: k past the end is the next row's start)
    }
#pragma unroll
    for (int i = 0; i < LW; ++i) w_off[i] = static_cast<unsigned>(wave + NW * i) * (K / 32) * 1024u + lane * 16u;
    // (past the end of the share: the last one again, nobody reads it)
    auto ask_a = [&](int kt, int stage) {
        const int last = (h_end - 1) >> 1;
        if (kt > last) kt = last;
        const bool tail = 2 * kt + 1 >= nh_all;                 // the slab is half a slab: k ends in it
        const unsigned base = lds_origin + stage * A_STAGE + wave * 1024;
#pragma unroll
        for (int i = 0; i < LA; ++i) load_b128_to_lds(a_rsrc, base + i * (NW * 1024), tail ? a_tail[i] : a_off[i], kt * (DK * 2));
    };
    auto ask_w = [&](int h, int stage) {
        if (h >= h_end) h = h_end - 1;
        const unsigned base = lds_origin + W_BASE + stage * W_STAGE + wave * 1024;
#pragma unroll
        for (int i = 0; i < LW; ++i) load_b128_to_lds(w_rsrc, base + i * (NW * 1024), w_off[i], h * 1024);
    };

    f32x4 acc[WMT][WNT];
#pragma unroll
    for (int i = 0; i < WMT; ++i)
#pragma unroll
        for (int j = 0; j < WNT; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (h_begin < h_end) {
        // this lane's place in an operand of A: chunk 2 g + r / 8, then [kb][q, or q ^ 1 in odd chunks][r % 8]
        const unsigned a_lane = (wm / 8 + (r >> 3)) * 1024 + (q ^ (r >> 3)) * 128 + (r & 7) * 16;
        const unsigned w_lane = W_BASE + (wn / 16) * 1024 + lane * 16;
        auto read_frags = [&](int sa, int kk, int sw, bf16x8 (&fa)[WMT], bf16x8 (&fw)[WNT]) {
            const unsigned char* sA = lds_raw + sa * A_STAGE + a_lane + kk * 512;
            const unsigned char* sW = lds_raw + sw * W_STAGE + w_lane;
#pragma unroll
            for (int i = 0; i < WMT; ++i) fa[i] = *reinterpret_cast<const bf16x8*>(sA + i * 2048);
#pragma unroll
            for (int j = 0; j < WNT; ++j) fw[j] = *reinterpret_cast<const bf16x8*>(sW + j * 1024);
        };
        auto multiply = [&](const bf16x8 (&fa)[WMT], const bf16x8 (&fw)[WNT]) {
#pragma unroll
            for (int i = 0; i < WMT; ++i)
#pragma unroll
                for (int j = 0; j < WNT; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        };
        // In front of the loop, what the half turns -5 .. -1 would have asked for, in their order
        // (W, then A): A(0); W(0); W(1), A(1); W(2); W(3), A(2). The waits count on this order: at an
        // even half turn h the loads behind W(h + 1) are A, W(h + 2), W(h + 3), A; at an odd one
        // W(h + 2), A, W(h + 3), and A's slab (h + 1) / 2 is older than W(h + 1).
        const int kt0 = h_begin >> 1;
        ask_a(kt0, 0);
        ask_w(h_begin, 0);
        ask_w(h_begin + 1, 1);
        ask_a(kt0 + 1, 1);
        ask_w(h_begin + 2, 2);
        ask_w(h_begin + 3, 3);
        ask_a(kt0 + 2, 2);
        wait_vm<3 * LW + 2 * LA>();
        lds_barrier();
        bf16x8 fa0[WMT], fw0[WNT];
        read_frags(0, 0, 0, fa0, fw0);
        int sa = 0, pair = 0;                           // A's buffer of this slab; W's buffers of it are 2 pair and 2 pair + 1
        for (int h = h_begin; h < h_end; h += 2) {
            bf16x8 fa1[WMT], fw1[WNT];
            wait_vm<2 * LW + 2 * LA>();                 // half slab h + 1 has landed (the later ones may be on their way)
            lds_barrier();                              // .. everybody's share of it, and everybody has read half slab h
            ask_w(h + 4, 2 * pair);
            read_frags(sa, 1, 2 * pair + 1, fa1, fw1);
            multiply(fa0, fw0);
            deal_between_products<kDsRead, WMT + WNT>();
            __builtin_amdgcn_sched_barrier(0);
            wait_vm<2 * LW + LA>();
            lds_barrier();
            ask_w(h + 5, 2 * pair + 1);
            ask_a((h >> 1) + 3, sa);
            sa = sa + 1 == NSA ? 0 : sa + 1;
            pair ^= 1;
            read_frags(sa, 0, 2 * pair, fa0, fw0);
            if (h + 1 < h_end) multiply(fa1, fw1);      // (a share that ends in half a slab: k ends there)
            deal_between_products<kDsRead, WMT + WNT>();
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    wait_vm<0>();                                       // (loads past the end are still on their way into LDS)
    __syncthreads();                                    // the epilogue reuses the slabs' LDS
    tile_epilogue<WMT, WNT, MODE, 160 * 1024, WR, WC>(acc, lds_raw, out, M, N, m0, n0, wm, wn, tid, r, q, qt);
}

template <auto KERNEL, int THREADS = 256>
static int launch_tile_kernel(int LDS, int BM, int BN, const bf16* A, const bf16* W, void* out, int M, int N, int K,
                              int ksplit, hipStream_t stream, const QkvTarget& qt = QkvTarget{}) {
    static bool attr_set = false;                      // per kernel
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(KERNEL),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set = true;
    }
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    hipLaunchKernelGGL(KERNEL, dim3(tiles_m * tiles_n * ksplit), dim3(THREADS), LDS, stream, A, W, out, M, N, K, tiles_m,
                       tiles_n, ksplit, qt);
    return launch_status();
}

template <int WMT, int WNT, int MODE, bool BLOCKED>
static int launch_tile_layout(const bf16* A, const bf16* W, void* out, int M, int N, int K, int ksplit,
                              hipStream_t stream) {
    constexpr int LDS = tile_lds_bytes<WMT, WNT>();
    if (K % TK != 0)
        return launch_tile_kernel<gemm_tile_kernel<WMT, WNT, MODE, false, BLOCKED>>(LDS, 32 * WMT, 32 * WNT, A, W, out,
                                                                                    M, N, K, ksplit, stream);
    return launch_tile_kernel<gemm_tile_kernel<WMT, WNT, MODE, true, BLOCKED>>(LDS, 32 * WMT, 32 * WNT, A, W, out, M,
                                                                               N, K, ksplit, stream);
}

template <int WMT, int WNT, int MODE>
static int launch_tile_mode(const bf16* A, const bf16* W, void* out, int M, int N, int K, int ksplit, int blocked,
                            hipStream_t stream) {
    if (blocked) return launch_tile_layout<WMT, WNT, MODE, true>(A, W, out, M, N, K, ksplit, stream);
    return launch_tile_layout<WMT, WNT, MODE, false>(A, W, out, M, N, K, ksplit, stream);
}

template <int WMT, int WNT>
static int launch_tile(const bf16* A, const bf16* W, void* out, int M, int N, int K, int mode, int ksplit,
                       int blocked, hipStream_t stream) {
    switch (mode) {
        case kStoreF32: return launch_tile_mode<WMT, WNT, kStoreF32>(A, W, out, M, N, K, 1, blocked, stream);
        case kAddF32: return launch_tile_mode<WMT, WNT, kAddF32>(A, W, out, M, N, K, 1, blocked, stream);
        case kAtomicF32: return launch_tile_mode<WMT, WNT, kAtomicF32>(A, W, out, M, N, K, ksplit, blocked, stream);
        case kGatedBF16: return launch_tile_mode<WMT, WNT, kGatedBF16>(A, W, out, M, N, K, 1, blocked, stream);
        default: return launch_tile_mode<WMT, WNT, kStoreBF16>(A, W, out, M, N, K, 1, blocked, stream);
    }
}

template <int WR, int WC, int WMT, int WNT>
static int launch_tile_direct(const bf16* A, const bf16* W, void* out, int M, int N, int K, int mode, int ksplit,
                                    hipStream_t stream) {
    constexpr int LDS = 160 * 1024;
    constexpr int BM = WR * 16 * WMT, BN = WC * 16 * WNT;
#define LLME_DIRECT(MODE) \
    launch_tile_kernel<gemm_tile_direct_kernel<WR, WC, WMT, WNT, MODE>, 64 * WR * WC>( \
        LDS, BM, BN, A, W, out, M, N, K, MODE == kAtomicF32 ? ksplit : 1, stream)
    switch (mode) {
        case kStoreF32: return LLME_DIRECT(kStoreF32);
        case kAddF32: return LLME_DIRECT(kAddF32);
        case kAtomicF32: return LLME_DIRECT(kAtomicF32);
        case kGatedBF16: return LLME_DIRECT(kGatedBF16);
        default: return LLME_DIRECT(kStoreBF16);
    }
#undef LLME_DIRECT
}

// ----------------------------------------------------------------------------------------
// skinny kernel: MT row tiles of 16 (M <= 16 MT), NW wavefronts per workgroup splitting k
template <int WMT, int WNT>
static int launch_tile_rope(const bf16* A, const bf16* W, int M, int N, int K, int blocked, const QkvTarget& qt,
                            hipStream_t stream) {
    constexpr int LDS = tile_lds_bytes<WMT, WNT>();
#define LLME_ROPE_TILE(KFULL, BLOCKED) \
    launch_tile_kernel<gemm_tile_kernel<WMT, WNT, kRopeCache, KFULL, BLOCKED>>(LDS, 32 * WMT, 32 * WNT, A, W, nullptr, M, N, \
                                                                                K, 1, stream, qt)
    if (K % TK != 0) return blocked ? LLME_ROPE_TILE(false, true) : LLME_ROPE_TILE(false, false);
    return blocked ? LLME_ROPE_TILE(true, true) : LLME_ROPE_TILE(true, false);
#undef LLME_ROPE_TILE
}

constexpr int SK_U = 4;                  // 32-element k steps per wavefront iteration
constexpr int SK_CHUNK = 32 * SK_U;      // 128 elements

template <int MT, int NW, int MODE>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                              void* __restrict__ out, int M, int N, int K,
                                                              int k_per_block, int blocked) {
    __shared__ f32x4 red[NW * MT * 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int k_begin = blockIdx.y * k_per_block;
    const int k_end = (k_begin + k_per_block < K) ? k_begin + k_per_block : K;

    // this lane's weights at k: row-major, row n0 + r from k + 8 q on; blocked, piece `lane` of block k / 32
    // of row group n0 / 16 (K is a multiple of 32 then: a block is in or out whole)
    const bool wrow_ok = (n0 + r) < N;
    const bf16* wrow = blocked ? w + static_cast<size_t>(blockIdx.x) * 16 * K + lane * 8
                               : w + static_cast<size_t>(wrow_ok ? n0 + r : 0) * K + q * 8;
    const int wstep = blocked ? 16 : 1;                 // elements of w per element of k
    const bf16* xrow[MT];
    bool xrow_ok[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xrow_ok[t] = (t * 16 + r) < M;
        xrow[t] = x + static_cast<size_t>(xrow_ok[t] ? t * 16 + r : 0) * K + q * 8;
    }
    f32x4 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k = k_begin + wave * SK_CHUNK; k < k_end; k += NW * SK_CHUNK) {
        bf16x8 fw[SK_U];
        bf16x8 fx[MT][SK_U];
#pragma unroll
        for (int u = 0; u < SK_U; ++u) {
            const int kk = k + u * 32;
            const bool k_ok = (kk + q * 8) < k_end;
            fw[u] = load8_once(wrow + static_cast<size_t>(kk) * wstep, wrow_ok && (blocked ? kk < k_end : k_ok));
#pragma unroll
            for (int t = 0; t < MT; ++t) fx[t][u] = load8(xrow[t] + kk, xrow_ok[t] && k_ok);
        }
#pragma unroll
        for (int u = 0; u < SK_U; ++u)
#pragma unroll
            for (int t = 0; t < MT; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[u], fx[t][u], acc[t], 0, 0, 0);
    }
    // add up the wavefronts' partial sums
#pragma unroll
    for (int t = 0; t < MT; ++t) red[(wave * MT + t) * 64 + lane] = acc[t];
    __syncthreads();
    // result of tile t in lane l: row m = 16 t + r (the x row), columns n = n0 + 4 q + e
    for (int item = tid; item < MT * 64; item += NW * 64) {
        const int t = item >> 6, l = item & 63;
        f32x4 s = red[t * 64 + l];
        for (int wv = 1; wv < NW; ++wv) {
            const f32x4 p = red[(wv * MT + t) * 64 + l];
            s[0] += p[0]; s[1] += p[1]; s[2] += p[2]; s[3] += p[3];
        }
        const int m = t * 16 + (l & 15);
        if (m >= M) continue;
        const int nb = n0 + (l >> 4) * 4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = nb + e;
            if (n >= N) continue;
            const size_t idx = static_cast<size_t>(m) * N + n;
            if (MODE == kStoreF32) static_cast<float*>(out)[idx] = s[e];
            else if (MODE == kAddF32) static_cast<float*>(out)[idx] += s[e];
            else if (MODE == kAtomicF32) atomicAdd(static_cast<float*>(out) + idx, s[e]);
            else static_cast<bf16*>(out)[idx] = static_cast<bf16>(s[e]);
        }
    }
}

template <int MT, int NW>
static void launch_skinny(const bf16* x, const bf16* w, void* out, int M, int N, int K, int mode, int ksplit,
                          int blocked, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    int k_per_block = (K + ksplit - 1) / ksplit;
    k_per_block = ((k_per_block + SK_CHUNK - 1) / SK_CHUNK) * SK_CHUNK;
    const dim3 grid(tiles, (K + k_per_block - 1) / k_per_block), block(NW * 64);
#define LLME_SK(MODE)                                                                            \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NW, MODE>), grid, block, 0, stream, x, w, out, M, N, K, k_per_block, \
                       blocked)
    if (mode == kStoreF32) LLME_SK(kStoreF32);
    else if (mode == kAddF32) LLME_SK(kAddF32);
    else if (mode == kAtomicF32) LLME_SK(kAtomicF32);
    else LLME_SK(kStoreBF16);
#undef LLME_SK
}

template <int MT>
static void launch_skinny_nw(const bf16* x, const bf16* w, void* out, int M, int N, int K, int mode, int nw,
                             int ksplit, int blocked, hipStream_t stream) {
    if (nw >= 16 && MT <= 2) launch_skinny<MT, 16>(x, w, out, M, N, K, mode, ksplit, blocked, stream);
    else if (nw >= 8) launch_skinny<MT, 8>(x, w, out, M, N, K, mode, ksplit, blocked, stream);
    else launch_skinny<MT, 4>(x, w, out, M, N, K, mode, ksplit, blocked, stream);
}

}  // namespace llme

using namespace llme;

// a [M, K], w [N, K] bfloat16; out [M, N] float32 (out_dtype 0) or bfloat16 (1).
// accumulate (float32 only) adds into out. gated: w holds gate and up rows interleaved in
// groups of 16 and out is bfloat16 [M, N / 2] = silu(gate) * up (tile kernel only).
// nw, ksplit: 0 lets the entry point choose the skinny kernel's wavefronts per workgroup and
// the split over k; tile_shape: 0 chooses, 64 / 128 force the tile kernel with that tile
// edge also for small M (for tests and measurements), 128096, 128064, 96128, 96064 tiles of 128 x 96 and so on. blocked: w is stored in 1 KB blocks of
// 16 rows x 32 k (see the head of this file; N a multiple of 16, K of 32). direct: the tile kernel
// of 256 x 256 whose slabs go from memory straight into LDS (needs blocked): -1 where the entry point
// finds it faster, 0 never, 1 it must (with tile_shape 256256).
extern "C" int llme_gemm_bf16(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K,
                              int accumulate, int gated, int nw, int ksplit, int tile_shape, int blocked, int direct,
                              hipStream_t stream) {
    if (direct < -1 || direct > 1 || (direct == 1 && !blocked)) return kErrBadArgument;
    if (M <= 0 || N <= 0) return 0;
    if (blocked && (N % 16 != 0 || K % 32 != 0)) return kErrUnsupported;
    if (K <= 0 || K % 8 != 0 || K >= (1 << 23)) return kErrUnsupported;   // 256 rows of K must stay below 2^32 bytes
    if (out_dtype != kF32 && out_dtype != kBF16) return kErrBadArgument;
    if (accumulate && out_dtype != kF32) return kErrBadArgument;
    if (gated && (out_dtype != kBF16 || N % 32 != 0 || accumulate)) return kErrBadArgument;
    const bf16* A = static_cast<const bf16*>(a);
    const bf16* W = static_cast<const bf16*>(w);
    int mode = out_dtype == kBF16 ? kStoreBF16 : (accumulate ? kAddF32 : kStoreF32);
    // Up to 16 rows: the skinny kernel (one row tile). 17 to 64 rows: the skinny kernel re-reads
    // the activations from L2 once per 16 output columns, which costs more than the weights
    // themselves, so wide outputs and sums that can be cut over k go to the 64 x 64 tile kernel.
    // (measured at 64 rows: 3,072 columns 12.7 us skinny against 13.8 with tiles, 5,120 columns 31.9
    // against 20.7, 6,144 columns of k = 4,096 40.5 against 27.2)
    const bool skinny = M <= 16 || (M <= 64 && !accumulate && N < 4096);
    const int cus = compute_units();
    if (skinny && tile_shape <= 0 && !gated) {
        const int tiles = (N + 15) / 16;
        if (nw <= 0 && ksplit <= 0 && accumulate && out_dtype == kF32 && tiles < 2 * cus) {
            // Few output columns and a sum to join anyway (the residual stream): cut k over
            // several workgroups that add their parts with atomics, so that the whole chip
            // streams the matrix. (The order of these additions is not fixed.)
            // (measured at 128 tiles: k = 2,048: 512 workgroups of 4 wavefronts 4.0 us, 256 of 8 4.1 us;
            // k = 8,192: 8.9 against 8.3 us)
            const bool long_k = K >= 4096 && tiles <= cus;
            ksplit = (long_k ? cus : 2 * cus) / tiles;
            if (ksplit > K / 512) ksplit = K / 512;
            if (ksplit < 1) ksplit = 1;
            nw = long_k ? 8 : 4;
        }
        if (nw <= 0) {
            // enough wavefronts to cover the chip several times, each with at least one chunk of k
            const int chunks = (K + SK_CHUNK - 1) / SK_CHUNK;
            nw = 4;
            while (nw < 16 && tiles * nw < 4096 && chunks >= nw * 2) nw *= 2;
        }
        if (ksplit <= 0) ksplit = 1;
        if (ksplit > 1) {
            if (out_dtype != kF32 || !accumulate) return kErrBadArgument;   // partial sums need a sum to join
            mode = kAtomicF32;
        }
        const int mt = (M + 15) / 16;
        switch (mt) {
            case 1: launch_skinny_nw<1>(A, W, out, M, N, K, mode, nw, ksplit, blocked, stream); break;
            case 2: launch_skinny_nw<2>(A, W, out, M, N, K, mode, nw, ksplit, blocked, stream); break;
            case 3: launch_skinny_nw<3>(A, W, out, M, N, K, mode, nw, ksplit, blocked, stream); break;
            default: launch_skinny_nw<4>(A, W, out, M, N, K, mode, nw, ksplit, blocked, stream); break;
        }
        return launch_status();
    }
    // tile shape: 0 lets the entry point choose: the largest tile that still gives about one
    // workgroup per compute unit; a small output with a long k is cut over k instead (the
    // parts are added with atomics, so this needs an accumulating float32 output).
    if (gated) mode = kGatedBF16;
    const bool auto_shape = tile_shape <= 0;
    float tiles_cost = -1.f;                           // of the chosen tile, in the units of the estimate below
    if (tile_shape <= 0) {
        const long wg128 = static_cast<long>((M + 127) / 128) * ((N + 127) / 128);
        // (a stored output with fewer than 96 tiles of 128 x 128 fills the chip better in 64 x 64 tiles:
        // q/k/v of the 1B sizes at 273 rows 12.6 against 16.0 us; sums that are cut over k keep the larger tiles)
        const long enough = (mode == kStoreF32 || mode == kStoreBF16) ? 96 : 64;
        tile_shape = (M > 64 && wg128 >= enough) ? 128 : 64;
        if (tile_shape == 128 && wg128 < 4 * cus && !(mode == kAddF32 && wg128 <= cus && K >= 4096)) {
            // Medium outputs: narrower tiles can fill the compute units (two workgroups
            // each) more evenly. Estimated time: rounds of one workgroup per compute unit x tile area / measured
            // efficiency of the shape; a workgroup alone on its compute unit overlaps nothing.
            // (tiles of 96 rows where they cover the rows with less to spare: 273 rows are three row
            // tiles either way; measured at the 1B sizes, gate/up 39.5 -> 32.6 us at 273 rows, 24.5 -> 21.7 at 192)
            const int shapes[5] = {128, 128096, 128064, 96128, 96064};
            const int heights[5] = {128, 128, 128, 96, 96};
            const int widths[5] = {128, 96, 64, 128, 64};
            // (efficiencies: sums that are added, from sweeps at 96 to 512 rows; stored and gated outputs, from the
            // gate/up shapes of the 1B, 3B and 8B sizes at 100 to 1,536 rows, e.g. at 320 rows of the 1B sizes
            // 36 / 44 / 38 / 34 / 39 us in the order of the shapes)
            const float eff_added[5] = {1.0f, 0.9f, 0.85f, 0.84f, 0.78f};
            const float eff_stored[5] = {1.0f, 0.9f, 0.70f, 0.83f, 0.67f};
            const float* eff = mode == kAddF32 ? eff_added : eff_stored;
            float best = 0.f;
            for (int c = 0; c < 5; ++c) {
                const long wgs = static_cast<long>((M + heights[c] - 1) / heights[c]) * ((N + widths[c] - 1) / widths[c]);
                const long rounds = (wgs + cus - 1) / cus;
                float cost = static_cast<float>(rounds) * heights[c] * widths[c] / eff[c];
                // (less so for the gated product, whose epilogue is long: measured at 129 to 256 rows,
                // 128 x 128 tiles 26.5 against 31 us at the 1B sizes, 36.6 against 43.7 at the 3B sizes)
                if (wgs <= cus) cost *= (mode == kGatedBF16 ? 1.1f : 1.25f);
                if (c == 0 || cost < best) {
                    best = cost;
                    tile_shape = shapes[c];
                }
            }
            tiles_cost = best;
        } else if (tile_shape == 128) {
            tiles_cost = static_cast<float>((wg128 + cus - 1) / cus) * 16384.f;
        }
        // A long sum into an output of few tiles (down-proj at 65 to 288 rows): tiles of 64 columns whose
        // 64, 96 or 128 rows leave the fewest rows to spare (the taller on a tie), cut over k in 2, 4 or 8
        // up to three workgroups per compute unit. Measured (us, against tiles of 64 x 64 or the estimate
        // above): down-proj of the 1B sizes at 273 rows 23.7 against 29.3, at 192 rows 18.4 against 21.3, at
        // 81 rows 13.5 against 14.7; of the 3B sizes at 200 and 256 rows 27.5 and 29.7 against 37.0 and 39.6, at 81
        // rows 16.6 against 21.1; of the 8B sizes at 273 rows 53 against 66, at 100 and 128 rows 28.9 and 30.6
        // against 40.9.
        bool tall = false;
        if (mode == kAddF32 && ksplit <= 0 && M > 64 && M <= 288 && K >= 4096 && wg128 <= cus) {
            const int rows64 = (M + 63) / 64 * 64, rows96 = (M + 95) / 96 * 96, rows128 = (M + 127) / 128 * 128;
            if (rows128 <= rows96 && rows128 <= rows64) tile_shape = 128064;
            else if (rows96 <= rows64) tile_shape = 96064;
            else tile_shape = 64;
            tall = tile_shape != 64;
        }
        if (mode == kAddF32 && ksplit <= 0) {
            // A sum that is joined anyway (the residual stream) is cut over k until the tiles fill
            // the chip: 64 x 64 tiles to about two workgroups per compute unit, the larger ones to
            // about one. (Measured at 96 to 512 rows, where the output has few tiles: down-proj of
            // the 1B sizes 48 us uncut against 15 to 33 us, o-proj 13.5 against 7.5 to 14 us.)
            const int bm = tile_shape == 64 ? 64 : (tile_shape == 96064 || tile_shape == 96128) ? 96 : 128;
            const int bn = (tile_shape == 128 || tile_shape == 96128) ? 128 : tile_shape == 128096 ? 96 : 64;
            const long wgs = static_cast<long>((M + bm - 1) / bm) * ((N + bn - 1) / bn);
            long ks = (tile_shape == 64 ? 2 * cus : cus) / wgs;
            if (tall) ks = (K >= 8192 && (M <= 96 || 8 * wgs <= cus) && 3 * cus / wgs >= 8) ? 8 : 3 * cus / wgs >= 4 ? 4 : 3 * cus / wgs >= 2 ? 2 : 1;
            // (a long sum in 128 x 128 tiles that leave compute units idle is cut in two: down-proj of the 1B sizes
            // at 1,024 rows 49 against 73 us, at 1,792 rows 75 against 79; with a tile for every compute unit it
            // is not: 84 against 87 us at 2,048 rows)
            if (tile_shape == 128 && wg128 < cus && K >= 4096 && ks < 2) ks = 2;
            if (ks > K / 512) ks = K / 512;
            if (ks > 8) ks = 8;
            ksplit = ks < 1 ? 1 : static_cast<int>(ks);
        }
    }
    if (ksplit <= 0) ksplit = 1;
    if (ksplit > 1) {
        if (mode != kAddF32) return kErrBadArgument;
        mode = kAtomicF32;
    }
    if (auto_shape && blocked && direct != 0 && mode != kAddF32 && mode != kAtomicF32 && tiles_cost > 0.f) {
        // Wide outputs that are stored, not added (gate/up, q/k/v of long prompts): tiles of 256 x 256
        // by eight wavefronts, their slabs straight into LDS, load half the bytes per product; one
        // workgroup fills a compute unit. In the units of the estimate above a round of them costs
        // 65,536 / 1.15 (measured: 1.07 to 1.16 times the 128 x 128 tiles' speed where whole rounds cover
        // the output; 8B gate/up at 448 rows, one round against 3.5 of 128 x 128: 105 against 129 us).
        const long rounds = (static_cast<long>((M + 255) / 256) * ((N + 255) / 256) + cus - 1) / cus;
        if (static_cast<float>(rounds) * 65536.f / 1.15f < tiles_cost)
            return launch_tile_direct<4, 2, 4, 8>(A, W, out, M, N, K, mode, ksplit, stream);
    }
    if (blocked && direct == 1 && tile_shape == 256256)
        return launch_tile_direct<4, 2, 4, 8>(A, W, out, M, N, K, mode, ksplit, stream);
    if (direct == 1) return kErrUnsupported;
    if (tile_shape == 96064) return launch_tile<3, 2>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    if (tile_shape == 96128) return launch_tile<3, 4>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    if (tile_shape == 128096) return launch_tile<4, 3>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    if (tile_shape == 128064) return launch_tile<4, 2>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    if (tile_shape == 128) return launch_tile<4, 4>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    if (tile_shape == 64) return launch_tile<2, 2>(A, W, out, M, N, K, mode, ksplit, blocked, stream);
    return kErrBadArgument;
}

// The q/k/v projection of many rows (prompts) with rotation and cache write in its epilogue:
// a [M, K] (the normed activations), w [(n_q + 2 n_kv) hd, K] (q heads, k heads, v heads), both
// bfloat16; writes q_out [M, n_q hd] (rotated) and the rows' k (rotated) and v into the pages that
// block_table[seq_idx[m]] names for positions[m]; cos/sin [max_pos, hd / 2] float32. Full rotation
// only; hd 16, 32, 64 or 128 (a tile of 128 or 64 columns must hold whole heads). What the separate
// kernels would store in between, the 32-bit q/k/v rows, never exists. tile_shape 0, 64, 96064, 128064, 96128 or 128.
extern "C" int llme_gemm_bf16_qkv_rope(const void* a, const void* w, int M, int K, int blocked, const float* cos_t,
                                       const float* sin_t, const int* positions, const int* seq_idx,
                                       const int* block_table, int max_blocks, void* q_out, void* k_cache,
                                       void* v_cache, int n_q, int n_kv, int hd, int page, int tile_shape,
                                       hipStream_t stream) {
    if (M <= 0) return 0;
    if (n_q <= 0 || n_kv <= 0 || page <= 0 || max_blocks <= 0) return kErrBadArgument;
    if (hd != 16 && hd != 32 && hd != 64 && hd != 128) return kErrUnsupported;
    if (K <= 0 || K % 8 != 0 || K >= (1 << 23)) return kErrUnsupported;
    if (blocked && K % 32 != 0) return kErrUnsupported;
    if (!cos_t || !sin_t || !positions || !seq_idx || !block_table || !q_out || !k_cache || !v_cache) return kErrBadArgument;
    if (reinterpret_cast<uintptr_t>(q_out) % 16 != 0 || reinterpret_cast<uintptr_t>(k_cache) % 16 != 0 ||
        reinterpret_cast<uintptr_t>(v_cache) % 16 != 0)
        return kErrUnsupported;
    const int N = (n_q + 2 * n_kv) * hd;
    const QkvTarget qt{cos_t, sin_t, positions, seq_idx, block_table, max_blocks, static_cast<bf16*>(q_out),
                       static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache), n_q, n_kv, hd, page};
    const bf16* A = static_cast<const bf16*>(a);
    const bf16* W = static_cast<const bf16*>(w);
    if (tile_shape <= 0) {
        // The tile with the least rounds of workgroups over the compute units x (a round's fixed cost,
        // which grows with k, + the tile's area): fitted to measurements at 80 to 1,024 rows. 1B sizes
        // (us with 64 x 64 / 96 x 64 / 128 x 64 / 128 x 128 tiles): 273 rows 12.1 / 13.8 / 16.0 / 22.8,
        // 384 rows 17.8 / 14.1 / 16.2 / 22.8, 512 rows 18.6 / 20.9 / 16.6 / 23.6, 1,024 rows 28.0 / 29.1 /
        // 25.8 / 25.5. A head of 128 needs the full width: 96 x 128 / 128 x 128 at the 3B sizes 26.3 / 31.4
        // at 256 rows, 44.3 / 49.2 at 1,024; at the 8B sizes 33.0 / 40.1 at 384 rows, 52.7 / 40.8 at 512.
        const int shapes[5] = {64, 96064, 128064, 96128, 128};
        const int heights[5] = {64, 96, 128, 96, 128};
        const int widths[5] = {64, 64, 64, 128, 128};
        const int cus = compute_units();
        const double fixed = 4.3 * K;
        double best = 0.0;
        for (int c = 0; c < 5; ++c) {
            if (hd > widths[c]) continue;
            const long wgs = static_cast<long>((M + heights[c] - 1) / heights[c]) * ((N + widths[c] - 1) / widths[c]);
            const double cost = static_cast<double>((wgs + cus - 1) / cus) * (fixed + heights[c] * widths[c]);
            if (tile_shape <= 0 || cost < best) {
                best = cost;
                tile_shape = shapes[c];
            }
        }
    }
    if (tile_shape == 128) return launch_tile_rope<4, 4>(A, W, M, N, K, blocked, qt, stream);
    if (tile_shape == 64 && hd <= 64) return launch_tile_rope<2, 2>(A, W, M, N, K, blocked, qt, stream);
    if (tile_shape == 128064 && hd <= 64) return launch_tile_rope<4, 2>(A, W, M, N, K, blocked, qt, stream);
    if (tile_shape == 96064 && hd <= 64) return launch_tile_rope<3, 2>(A, W, M, N, K, blocked, qt, stream);
    if (tile_shape == 96128) return launch_tile_rope<3, 4>(A, W, M, N, K, blocked, qt, stream);
    return kErrBadArgument;
}

LLME_LOAD_ENTRY(gemm_mfma)
