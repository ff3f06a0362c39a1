// Token choice on the device, one workgroup per row of logits [R, V].
//
// Greedy: the first index of the maximum (ties go to the lowest id), as the
// reference's argmax (src/engine.cpp:52-58, src/scheduler.cpp:10-16).
// Temperature: p = softmax(logits / T) in 32-bit; the token is the first id whose
// cumulative probability, summed in ascending id order, exceeds u * sum(p) for a
// uniform draw u in [0, 1) that the host supplies for the row.
#include "common.h"
#include <math.h>

namespace llme {

constexpr int kSampleThreads = 256;

__device__ __forceinline__ void argmax_combine(float& bv, int& bi, float ov, int oi) {
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

// Block-wide argmax with the lowest-index tie rule; result valid in every thread.
__device__ __forceinline__ void block_argmax(float& bv, int& bi, float* sv, int* si) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        argmax_combine(bv, bi, ov, oi);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) { sv[wave] = bv; si[wave] = bi; }
    __syncthreads();
    bv = sv[0]; bi = si[0];
    for (int i = 1; i < kSampleThreads / kWave; ++i) argmax_combine(bv, bi, sv[i], si[i]);
}

// Greedy choice in two stages, so that a few rows of a large vocabulary still fill the chip:
// grid (row, part): each workgroup takes a contiguous part of the row and writes its
// (maximum, first index); a second small kernel joins the parts.
__global__ __launch_bounds__(kSampleThreads) void argmax_part_kernel(const float* __restrict__ logits,
                                                                     float* __restrict__ part_val,
                                                                     int* __restrict__ part_idx, int V, int chunk) {
    __shared__ float sv[kSampleThreads / kWave];
    __shared__ int si[kSampleThreads / kWave];
    const float* row = logits + static_cast<size_t>(blockIdx.x) * V;
    const int begin = blockIdx.y * chunk;
    const int end = (begin + chunk < V) ? begin + chunk : V;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    // eight loads at a time (asked for one by one, each waits for its own trip to memory)
    constexpr int U = 8;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kSampleThreads * U) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * kSampleThreads;
            v[u] = row[i < end ? i : end - 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * kSampleThreads;
            if (i < end) argmax_combine(bv, bi, v[u], i);
        }
    }
    block_argmax(bv, bi, sv, si);
    if (threadIdx.x == 0) {
        part_val[blockIdx.x * gridDim.y + blockIdx.y] = bv;
        part_idx[blockIdx.x * gridDim.y + blockIdx.y] = bi;
    }
}

__global__ __launch_bounds__(kWave) void argmax_join_kernel(const float* __restrict__ part_val,
                                                            const int* __restrict__ part_idx, int* __restrict__ out,
                                                            int parts) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int p = threadIdx.x; p < parts; p += kWave)
        argmax_combine(bv, bi, part_val[blockIdx.x * parts + p], part_idx[blockIdx.x * parts + p]);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        argmax_combine(bv, bi, ov, oi);
    }
    if (threadIdx.x == 0) out[blockIdx.x] = (bi == 0x7fffffff) ? 0 : bi;
}

// Rows with temperature <= 0 are greedy.
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits,
                                                                const float* __restrict__ temperature,
                                                                const float* __restrict__ uniform,
                                                                int* __restrict__ out, int V) {
    __shared__ float sv[kSampleThreads / kWave];
    __shared__ int si[kSampleThreads / kWave];
    __shared__ float seg_sum[kSampleThreads];
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const float* row = logits + static_cast<size_t>(r) * V;
    const float temp = temperature[r];

    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += kSampleThreads) argmax_combine(bv, bi, row[i], i);
    block_argmax(bv, bi, sv, si);
    if (bi == 0x7fffffff) bi = 0;
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[r] = bi;
        return;
    }
    // Each thread owns a run of consecutive ids, so that segment sums added in
    // thread order are the cumulative sums in ascending id order.
    const float inv_t = 1.0f / temp;
    const float mx = bv * inv_t;
    const int seg = (V + kSampleThreads - 1) / kSampleThreads;
    const int begin = threadIdx.x * seg;
    const int end = (begin + seg < V) ? begin + seg : V;
    float mine = 0.f;
    for (int i = begin; i < end; ++i) mine += expf(row[i] * inv_t - mx);
    seg_sum[threadIdx.x] = mine;
    const float total = block_sum(mine, scratch, kSampleThreads / kWave);
    if (threadIdx.x == 0) {
        const float target = uniform[r] * total;
        float cum = 0.f;
        int s = 0;
        while (s < kSampleThreads - 1 && cum + seg_sum[s] <= target) { cum += seg_sum[s]; ++s; }
        const int b = s * seg;
        const int e = (b + seg < V) ? b + seg : V;
        int pick = -1;
        for (int i = b; i < e; ++i) {
            cum += expf(row[i] * inv_t - mx);
            if (cum > target) { pick = i; break; }
        }
        if (pick < 0) {
            // Rounding left the target beyond the last partial sum: take the last id with mass.
            pick = (e > b) ? e - 1 : bi;
        }
        out[r] = pick;
    }
}

}  // namespace llme

using namespace llme;

// Parts per row that llme_argmax uses for a vocabulary size: the caller provides scratch for
// R * parts floats and ints.
extern "C" int llme_argmax_parts(int V) {
    const int parts = (V + 2047) / 2048;
    return parts < 1 ? 1 : (parts > 64 ? 64 : parts);
}

extern "C" int llme_argmax(const float* logits, int* out, float* part_val, int* part_idx, int R, int V,
                           hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0) return kErrBadArgument;
    const int parts = llme_argmax_parts(V);
    const int chunk = (V + parts - 1) / parts;
    hipLaunchKernelGGL(argmax_part_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, part_val,
                       part_idx, V, chunk);
    hipLaunchKernelGGL(argmax_join_kernel, dim3(R), dim3(kWave), 0, stream, part_val, part_idx, out, parts);
    return launch_status();
}

extern "C" int llme_sample(const float* logits, const float* temperature, const float* uniform, int* out,
                           int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0) return kErrBadArgument;
    hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(kSampleThreads), 0, stream, logits, temperature, uniform,
                       out, V);
    return launch_status();
}
