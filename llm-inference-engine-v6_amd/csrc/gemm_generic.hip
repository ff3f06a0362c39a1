// out[m, n] (+)= sum_k a[m, k] * w[n, k]     (src/kernels.cpp:33-57: W is [N, K] row-major)
//
// The plain-precision matrix product: every element is widened to 32-bit, multiplied
// and accumulated with 32-bit FMA, whatever the storage types. It is the whole
// matrix path of the 32-bit model and the fallback of the bfloat16 model for
// operand types or shapes that the MFMA kernels refuse. Any M, N, K. W may also come in the
// MFMA kernels' blocked layout ([N / 16][K / 32] blocks of [4][16][8]; N % 16 == 0, K % 32 == 0).
//
// Up to 16 rows (decoding) go to a kernel of their own that streams the weights once (further
// down). Tiling otherwise: a workgroup of 256 threads makes a 64 x 64 tile of the output, 4 x 4 per
// thread, stepping through K in slabs of 16 staged in LDS (stored k-major so that
// the inner loop reads consecutive addresses).
#include "common.h"

namespace llme {

constexpr int GB = 64;   // tile edge in m and n
constexpr int GK = 16;   // k slab

template <typename TA, typename TW, typename TO, bool ACC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                           TO* __restrict__ out, int M, int N, int K, int blocked) {
    __shared__ float As[GK][GB + 4];
    __shared__ float Ws[GK][GB + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * GB;
    const int n0 = blockIdx.x * GB;
    const int tx = tid % 16;      // n direction
    const int ty = tid / 16;      // m direction
    // loader mapping: 64 rows x 16 k per slab = 1024 elements, 4 per thread
    const int lrow = tid / 4;          // 0..63
    const int lk = (tid % 4) * 4;      // 0,4,8,12

    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + lk + j;
            const int am = m0 + lrow;
            const int wn = n0 + lrow;
            As[lk + j][lrow] = (am < M && k < K) ? to_float(a[static_cast<size_t>(am) * K + k]) : 0.f;
            const size_t widx = blocked
                ? (static_cast<size_t>(wn / 16) * (K / 32) + k / 32) * 512 + ((k % 32) / 8 * 16 + wn % 16) * 8 + k % 8
                : static_cast<size_t>(wn) * K + k;
            Ws[lk + j][lrow] = (wn < N && k < K) ? to_float(w[widx]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < GK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            TO* o = out + static_cast<size_t>(m) * N + n;
            if (ACC) *o = from_float<TO>(to_float(*o) + acc[i][j]);
            else *o = from_float<TO>(acc[i][j]);
        }
    }
}

// The same product for up to 16 rows (decoding): nothing to tile, the weight matrix is streamed
// once. A wavefront takes GV_COLS output columns at a time; its lanes split k in groups of four
// (16- or 8-byte loads), each lane keeps a partial sum per row and column, and the lanes' sums are
// added at the end. The rows of a come from the cache (they are read once per GV_COLS columns).
// K a multiple of 4, a and w 16-byte aligned, w row-major.
constexpr int GV_COLS = 4;
constexpr int GV_MAX_ROWS = 16;

template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&v)[4]);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <>
__device__ __forceinline__ void load4<bf16>(const bf16* p, float (&v)[4]) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(x[i]);
}

template <typename TA, typename TW, typename TO, bool ACC, int MR>
__global__ __launch_bounds__(256) void gemv_generic_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                           TO* __restrict__ out, int M, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int wave_id = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int n0 = wave_id * GV_COLS;
    if (n0 >= N) return;                                  // (whole wavefronts)
    float acc[MR][GV_COLS];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int c = 0; c < GV_COLS; ++c) acc[m][c] = 0.f;
    for (int k = lane * 4; k < K; k += 64 * 4) {
        float wv[GV_COLS][4];
#pragma unroll
        for (int c = 0; c < GV_COLS; ++c) {
            const int n = n0 + c < N ? n0 + c : N - 1;     // past the edge: the last column again, not stored
            load4<TW>(w + static_cast<size_t>(n) * K + k, wv[c]);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            float av[4];
            load4<TA>(a + static_cast<size_t>(m < M ? m : M - 1) * K + k, av);
#pragma unroll
            for (int c = 0; c < GV_COLS; ++c)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[m][c] = fmaf(av[i], wv[c][i], acc[m][c]);
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int c = 0; c < GV_COLS; ++c) {
            const float s = wave_sum(acc[m][c]);
            if (lane == 0 && m < M && n0 + c < N) {
                TO* o = out + static_cast<size_t>(m) * N + n0 + c;
                *o = from_float<TO>(ACC ? to_float(*o) + s : s);
            }
        }
}

template <typename TA, typename TW, typename TO>
static int launch_gemv_generic(const void* a, const void* w, void* out, int M, int N, int K, int accumulate,
                               hipStream_t stream) {
    const int waves = (N + GV_COLS - 1) / GV_COLS;
    const dim3 grid((waves + 3) / 4);
#define LLME_GEMV(ACC, MR)                                                                          \
    hipLaunchKernelGGL((gemv_generic_kernel<TA, TW, TO, ACC, MR>), grid, dim3(256), 0, stream,     \
                       static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out), M, N, K)
    // (rows in steps: the partial sums live in registers, 4 per row)
    if (accumulate) {
        if (M <= 1) LLME_GEMV(true, 1);
        else if (M <= 4) LLME_GEMV(true, 4);
        else if (M <= 8) LLME_GEMV(true, 8);
        else LLME_GEMV(true, 16);
    } else {
        if (M <= 1) LLME_GEMV(false, 1);
        else if (M <= 4) LLME_GEMV(false, 4);
        else if (M <= 8) LLME_GEMV(false, 8);
        else LLME_GEMV(false, 16);
    }
#undef LLME_GEMV
    return launch_status();
}

template <typename TA, typename TW, typename TO>
static int launch_generic(const void* a, const void* w, void* out, int M, int N, int K, int accumulate,
                          int blocked, hipStream_t stream) {
    if (M <= GV_MAX_ROWS && !blocked && K % 4 == 0 && reinterpret_cast<uintptr_t>(a) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(w) % 16 == 0)
        return launch_gemv_generic<TA, TW, TO>(a, w, out, M, N, K, accumulate, stream);
    const dim3 grid((N + GB - 1) / GB, (M + GB - 1) / GB);
    if (accumulate)
        hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TO, true>), grid, dim3(256), 0, stream,
                           static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out), M, N, K, blocked);
    else
        hipLaunchKernelGGL((gemm_generic_kernel<TA, TW, TO, false>), grid, dim3(256), 0, stream,
                           static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out), M, N, K, blocked);
    return launch_status();
}

}  // namespace llme

using namespace llme;

// a [M, K], w [N, K], out [M, N]; each of f32 or bf16; accumulate adds into out.
extern "C" int llme_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, void* out,
                                 int out_dtype, int M, int N, int K, int accumulate, int blocked,
                                 hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return kErrBadArgument;
    if (blocked && (N % 16 != 0 || K % 32 != 0)) return kErrUnsupported;
    const int key = a_dtype * 4 + w_dtype * 2 + out_dtype;
    switch (key) {
        case 0: return launch_generic<float, float, float>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 1: return launch_generic<float, float, bf16>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 2: return launch_generic<float, bf16, float>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 3: return launch_generic<float, bf16, bf16>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 4: return launch_generic<bf16, float, float>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 5: return launch_generic<bf16, float, bf16>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 6: return launch_generic<bf16, bf16, float>(a, w, out, M, N, K, accumulate, blocked, stream);
        case 7: return launch_generic<bf16, bf16, bf16>(a, w, out, M, N, K, accumulate, blocked, stream);
        default: return kErrBadArgument;
    }
}

LLME_LOAD_ENTRY(gemm_generic)
