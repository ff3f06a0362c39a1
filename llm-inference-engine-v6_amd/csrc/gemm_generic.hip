// out[m, n] (+)= sum_k a[m, k] * w[n, k]     (src/kernels.cpp:33-57: W is [N, K] row-major)
//
// The plain-precision matrix product: every element is widened to 32-bit, multiplied
// and accumulated with 32-bit FMA, whatever the storage types. It is the whole
// matrix path of the 32-bit model and the fallback of the bfloat16 model for
// operand types or shapes that the MFMA kernels refuse. Any M, N, K. W may also come in the
// MFMA kernels' blocked layout ([N / 16][K / 32] blocks of [4][16][8]; N % 16 == 0, K % 32 == 0).
//
// Tiling: a workgroup of 256 threads makes a 64 x 64 tile of the output, 4 x 4 per
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

template <typename TA, typename TW, typename TO>
static int launch_generic(const void* a, const void* w, void* out, int M, int N, int K, int accumulate,
                          int blocked, hipStream_t stream) {
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
