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

enum OutMode : int { kStoreF32 = 0, kAddF32 = 1, kStoreBF16 = 2, kAtomicF32 = 3 };

// ----------------------------------------------------------------------------------------
// tile kernel
constexpr int TM = 128, TN = 128, TK = 64;
constexpr int TSTRIDE = TK + 8;                      // elements; 144 bytes: conflict-free 16-byte reads
constexpr int TILE_ELEMS = TM * TSTRIDE;             // one operand tile in LDS
constexpr int TILE_LDS_BYTES = 4 * TILE_ELEMS * 2;   // A and W, two buffers each

template <int MODE>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const bf16* __restrict__ a, const bf16* __restrict__ w,
                                                        void* __restrict__ out, int M, int N, int K,
                                                        int tiles_m, int tiles_n) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    bf16* lds = reinterpret_cast<bf16*>(lds_raw);
    // buffers: sA[b] = lds + b * TILE_ELEMS, sW[b] = lds + (2 + b) * TILE_ELEMS

    // Tile order: groups of 8 tile rows, columns fastest inside a group, so that workgroups
    // that run together share rows of A and of W in L2.
    constexpr int GROUP = 8;
    const int pid = blockIdx.x;
    const int per_group = GROUP * tiles_n;
    const int g = pid / per_group;
    const int first_m = g * GROUP;
    const int gsize = (tiles_m - first_m < GROUP) ? tiles_m - first_m : GROUP;
    const int tm = first_m + (pid % per_group) % gsize;
    const int tn = (pid % per_group) / gsize;
    const int m0 = tm * TM, n0 = tn * TN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;

    // global -> LDS mapping: a tile is 128 rows x 8 chunks of 16 bytes; 4 chunks per thread
    int crow[4], ckq[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        crow[i] = c >> 3;
        ckq[i] = c & 7;
    }
    bf16x8 ra[4], rw[4];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + ckq[i] * 8;
            const int am = m0 + crow[i], wr = n0 + crow[i];
            ra[i] = load8(a + static_cast<size_t>(am) * K + k, am < M && k < K);
            rw[i] = load8(w + static_cast<size_t>(wr) * K + k, wr < N && k < K);
        }
    };
    auto store_lds = [&](int buf) {
        bf16* sA = lds + buf * TILE_ELEMS;
        bf16* sW = lds + (2 + buf) * TILE_ELEMS;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<bf16x8*>(sA + crow[i] * TSTRIDE + ckq[i] * 8) = ra[i];
            *reinterpret_cast<bf16x8*>(sW + crow[i] * TSTRIDE + ckq[i] * 8) = rw[i];
        }
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int nk = (K + TK - 1) / TK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * TK);
        const bf16* sA = lds + buf * TILE_ELEMS;
        const bf16* sW = lds + (2 + buf) * TILE_ELEMS;
#pragma unroll
        for (int kk = 0; kk < TK / 32; ++kk) {
            bf16x8 fa[4], fw[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                fa[i] = *reinterpret_cast<const bf16x8*>(sA + (wm + i * 16 + r) * TSTRIDE + kk * 32 + q * 8);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                fw[j] = *reinterpret_cast<const bf16x8*>(sW + (wn + j * 16 + r) * TSTRIDE + kk * 32 + q * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // result tile (i, j): column n = wn + 16 j + r, rows m = wm + 16 i + 4 q + e
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int m = m0 + wm + i * 16 + q * 4 + e;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn + j * 16 + r;
                if (n >= N) continue;
                const size_t idx = static_cast<size_t>(m) * N + n;
                const float v = acc[i][j][e];
                if (MODE == kStoreF32) static_cast<float*>(out)[idx] = v;
                else if (MODE == kAddF32) static_cast<float*>(out)[idx] += v;
                else static_cast<bf16*>(out)[idx] = static_cast<bf16>(v);
            }
        }
    }
}

// ----------------------------------------------------------------------------------------
// skinny kernel: MT row tiles of 16 (M <= 16 MT), NW wavefronts per workgroup splitting k
constexpr int SK_U = 4;                  // 32-element k steps per wavefront iteration
constexpr int SK_CHUNK = 32 * SK_U;      // 128 elements

template <int MT, int NW, int MODE>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                              void* __restrict__ out, int M, int N, int K,
                                                              int k_per_block) {
    __shared__ f32x4 red[NW * MT * 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int k_begin = blockIdx.y * k_per_block;
    const int k_end = (k_begin + k_per_block < K) ? k_begin + k_per_block : K;

    const bool wrow_ok = (n0 + r) < N;
    const bf16* wrow = w + static_cast<size_t>(wrow_ok ? n0 + r : 0) * K + q * 8;
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
            fw[u] = load8(wrow + kk, wrow_ok && k_ok);
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
                          hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    int k_per_block = (K + ksplit - 1) / ksplit;
    k_per_block = ((k_per_block + SK_CHUNK - 1) / SK_CHUNK) * SK_CHUNK;
    const dim3 grid(tiles, (K + k_per_block - 1) / k_per_block), block(NW * 64);
#define LLME_SK(MODE)                                                                            \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, NW, MODE>), grid, block, 0, stream, x, w, out, M, N, K, k_per_block)
    if (mode == kStoreF32) LLME_SK(kStoreF32);
    else if (mode == kAddF32) LLME_SK(kAddF32);
    else if (mode == kAtomicF32) LLME_SK(kAtomicF32);
    else LLME_SK(kStoreBF16);
#undef LLME_SK
}

template <int MT>
static void launch_skinny_nw(const bf16* x, const bf16* w, void* out, int M, int N, int K, int mode, int nw,
                             int ksplit, hipStream_t stream) {
    if (nw >= 16 && MT <= 2) launch_skinny<MT, 16>(x, w, out, M, N, K, mode, ksplit, stream);
    else if (nw >= 8) launch_skinny<MT, 8>(x, w, out, M, N, K, mode, ksplit, stream);
    else launch_skinny<MT, 4>(x, w, out, M, N, K, mode, ksplit, stream);
}

}  // namespace llme

using namespace llme;

// a [M, K], w [N, K] bfloat16; out [M, N] float32 (out_dtype 0) or bfloat16 (1).
// accumulate (float32 only) adds into out. nw, ksplit: 0 lets the entry point choose the
// skinny kernel's wavefronts per workgroup and grid split over k; force_tile != 0 sends
// small M to the tile kernel too (for tests).
extern "C" int llme_gemm_bf16(const void* a, const void* w, void* out, int out_dtype, int M, int N, int K,
                              int accumulate, int nw, int ksplit, int force_tile, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || K % 8 != 0) return kErrUnsupported;
    if (out_dtype != kF32 && out_dtype != kBF16) return kErrBadArgument;
    if (accumulate && out_dtype != kF32) return kErrBadArgument;
    const bf16* A = static_cast<const bf16*>(a);
    const bf16* W = static_cast<const bf16*>(w);
    int mode = out_dtype == kBF16 ? kStoreBF16 : (accumulate ? kAddF32 : kStoreF32);
    if (M <= 64 && !force_tile) {
        const int tiles = (N + 15) / 16;
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
            case 1: launch_skinny_nw<1>(A, W, out, M, N, K, mode, nw, ksplit, stream); break;
            case 2: launch_skinny_nw<2>(A, W, out, M, N, K, mode, nw, ksplit, stream); break;
            case 3: launch_skinny_nw<3>(A, W, out, M, N, K, mode, nw, ksplit, stream); break;
            default: launch_skinny_nw<4>(A, W, out, M, N, K, mode, nw, ksplit, stream); break;
        }
        return launch_status();
    }
    const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
    const dim3 grid(tiles_m * tiles_n), block(256);
    static bool attr_set[3] = {false, false, false};
#define LLME_TILE(MODE, SLOT)                                                                              \
    do {                                                                                                   \
        if (!attr_set[SLOT]) {                                                                             \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_tile_kernel<MODE>),     \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, TILE_LDS_BYTES); \
            if (e != hipSuccess) return static_cast<int>(e);                                               \
            attr_set[SLOT] = true;                                                                         \
        }                                                                                                  \
        hipLaunchKernelGGL((gemm_tile_kernel<MODE>), grid, block, TILE_LDS_BYTES, stream, A, W, out, M, N, \
                           K, tiles_m, tiles_n);                                                           \
    } while (0)
    if (mode == kStoreF32) LLME_TILE(kStoreF32, 0);
    else if (mode == kAddF32) LLME_TILE(kAddF32, 1);
    else LLME_TILE(kStoreBF16, 2);
#undef LLME_TILE
    return launch_status();
}
