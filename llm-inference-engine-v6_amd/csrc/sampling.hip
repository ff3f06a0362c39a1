// Token choice on the device for rows of logits [R, V]; a row is cut into parts so that a few
// rows of a large vocabulary still fill the chip.
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

// out[slot R + row] (slot: a number the device holds, 0 without one), and also[row] where that is given:
// a recorded decode step leaves its choice for the host in one of two places in turn, and for its own
// next replay among its integer arrays.
__global__ __launch_bounds__(kWave) void argmax_join_kernel(const float* __restrict__ part_val,
                                                            const int* __restrict__ part_idx, int* __restrict__ out,
                                                            int parts, int* __restrict__ also = nullptr,
                                                            const int* __restrict__ slot = nullptr) {
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
    if (threadIdx.x == 0) {
        const int token = (bi == 0x7fffffff) ? 0 : bi;
        out[(slot ? *slot * static_cast<int>(gridDim.x) : 0) + blockIdx.x] = token;
        if (also) also[blockIdx.x] = token;
    }
}

// Temperature sampling in three stages over the same parts as the greedy choice. The first is
// argmax_part_kernel: the row's maximum is the maximum of its parts. The second sums
// exp(x / T - max / T) over each part. The third adds the parts' sums in ascending order, finds
// the part in which the cumulative sum passes u * total, and walks that part alone: every thread
// owns a run of consecutive ids there, the runs' sums are scanned in thread order, and the
// lowest id whose cumulative sum exceeds the target wins. Rows with temperature <= 0 are greedy.
__device__ __forceinline__ float row_maximum(const float* __restrict__ part_val, int parts) {
    float m = -INFINITY;
    for (int p = 0; p < parts; ++p) m = fmaxf(m, part_val[p]);
    return m;
}

__global__ __launch_bounds__(kSampleThreads) void sample_sum_kernel(const float* __restrict__ logits,
                                                                    const float* __restrict__ temperature,
                                                                    const float* __restrict__ part_val,
                                                                    float* __restrict__ part_sum, int V, int chunk) {
    __shared__ float scratch[kSampleThreads / kWave];
    const int r = blockIdx.x, parts = gridDim.y;
    const float temp = temperature[r];
    if (!(temp > 0.f)) return;
    const float inv_t = 1.0f / temp;
    const float mx = row_maximum(part_val + r * parts, parts) * inv_t;
    const float* row = logits + static_cast<size_t>(r) * V;
    const int begin = blockIdx.y * chunk;
    const int end = (begin + chunk < V) ? begin + chunk : V;
    float mine = 0.f;
    constexpr int U = 8;
    for (int i0 = begin + threadIdx.x; i0 < end; i0 += kSampleThreads * U) {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * kSampleThreads;
            v[u] = row[i < end ? i : end - 1];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (i0 + u * kSampleThreads < end) mine += expf(v[u] * inv_t - mx);
    }
    const float total = block_sum(mine, scratch, kSampleThreads / kWave);
    if (threadIdx.x == 0) part_sum[r * parts + blockIdx.y] = total;
}

__global__ __launch_bounds__(kSampleThreads) void sample_pick_kernel(const float* __restrict__ logits,
                                                                     const float* __restrict__ temperature,
                                                                     const float* __restrict__ uniform,
                                                                     const float* __restrict__ part_val,
                                                                     const int* __restrict__ part_idx,
                                                                     const float* __restrict__ part_sum,
                                                                     int* __restrict__ out, int V, int chunk,
                                                                     int parts, int* __restrict__ also = nullptr,
                                                                     const int* __restrict__ slot = nullptr) {
    __shared__ float wave_total[kSampleThreads / kWave];
    __shared__ int pick;
    const int r = blockIdx.x;
    const float temp = temperature[r];
    // (the choice goes to out[slot R + row] and, where given, to also[row], as in argmax_join_kernel)
    const int out_at = (slot ? *slot * static_cast<int>(gridDim.x) : 0) + r;
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int p = 0; p < parts; ++p) argmax_combine(bv, bi, part_val[r * parts + p], part_idx[r * parts + p]);
            const int token = (bi == 0x7fffffff) ? 0 : bi;
            out[out_at] = token;
            if (also) also[r] = token;
        }
        return;
    }
    // every thread walks the parts' sums alike: the part in which the cumulative sum passes
    // the target (the last one if rounding leaves none), and the sum before it
    float total = 0.f;
    for (int p = 0; p < parts; ++p) total += part_sum[r * parts + p];
    const float target = uniform[r] * total;
    float before = 0.f;
    int part = 0;
    while (part < parts - 1 && before + part_sum[r * parts + part] <= target) {
        before += part_sum[r * parts + part];
        ++part;
    }
    const float inv_t = 1.0f / temp;
    const float mx = row_maximum(part_val + r * parts, parts) * inv_t;
    const float* row = logits + static_cast<size_t>(r) * V;
    const int begin = part * chunk;
    const int end = (begin + chunk < V) ? begin + chunk : V;
    const int run = (end - begin + kSampleThreads - 1) / kSampleThreads;
    const int mine_begin = begin + threadIdx.x * run;
    const int mine_end = (mine_begin + run < end) ? mine_begin + run : end;
    float mine = 0.f;
    for (int i = mine_begin; i < mine_end; ++i) mine += expf(row[i] * inv_t - mx);
    // sums of the runs before this thread's: within the wave, then over the waves before it
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    float inclusive = mine;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const float other = __shfl_up(inclusive, off, kWave);
        if (lane >= off) inclusive += other;
    }
    if (threadIdx.x == 0) pick = 0x7fffffff;
    if (lane == kWave - 1) wave_total[wave] = inclusive;
    __syncthreads();
    float cum = before + (inclusive - mine);
    for (int w = 0; w < wave; ++w) cum += wave_total[w];
    for (int i = mine_begin; i < mine_end; ++i) {
        cum += expf(row[i] * inv_t - mx);
        if (cum > target) {
            atomicMin(&pick, i);
            break;
        }
    }
    __syncthreads();
    // Rounding left the target beyond the last cumulative sum: the last id of the part.
    if (threadIdx.x == 0) {
        const int token = (pick == 0x7fffffff) ? end - 1 : pick;
        out[out_at] = token;
        if (also) also[r] = token;
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
    hipLaunchKernelGGL(argmax_join_kernel, dim3(R), dim3(kWave), 0, stream, part_val, part_idx, out, parts,
                       static_cast<int*>(nullptr), static_cast<const int*>(nullptr));
    return launch_status();
}

// The same with the choice left in two places: out[*slot * R + row] (slot: an int in device memory that is 0
// or 1; out holds 2 R ints) and also[row]. For a recorded step whose next replay reads the tokens it chose.
extern "C" int llme_argmax_to(const float* logits, int* out, int* also, const int* slot, float* part_val,
                              int* part_idx, int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0 || !out) return kErrBadArgument;
    const int parts = llme_argmax_parts(V);
    const int chunk = (V + parts - 1) / parts;
    hipLaunchKernelGGL(argmax_part_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, part_val,
                       part_idx, V, chunk);
    hipLaunchKernelGGL(argmax_join_kernel, dim3(R), dim3(kWave), 0, stream, part_val, part_idx, out, parts, also, slot);
    return launch_status();
}

// part_val, part_idx and part_sum: scratch for R * llme_argmax_parts(V) values each.
extern "C" int llme_sample(const float* logits, const float* temperature, const float* uniform, int* out,
                           float* part_val, int* part_idx, float* part_sum, int R, int V, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0) return kErrBadArgument;
    const int parts = llme_argmax_parts(V);
    const int chunk = (V + parts - 1) / parts;
    hipLaunchKernelGGL(argmax_part_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, part_val,
                       part_idx, V, chunk);
    hipLaunchKernelGGL(sample_sum_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, temperature,
                       part_val, part_sum, V, chunk);
    hipLaunchKernelGGL(sample_pick_kernel, dim3(R), dim3(kSampleThreads), 0, stream, logits, temperature, uniform,
                       part_val, part_idx, part_sum, out, V, chunk, parts, static_cast<int*>(nullptr),
                       static_cast<const int*>(nullptr));
    return launch_status();
}

// The same with the choice left in two places, as llme_argmax_to leaves it: out[*slot * R + row] (out holds
// 2 R ints; slot may be null: then out[row]) and also[row] (may be null).
extern "C" int llme_sample_to(const float* logits, const float* temperature, const float* uniform, int* out,
                              int* also, const int* slot, float* part_val, int* part_idx, float* part_sum, int R,
                              int V, hipStream_t stream) {
    if (R <= 0) return 0;
    if (V <= 0 || !out || !temperature || !uniform) return kErrBadArgument;
    const int parts = llme_argmax_parts(V);
    const int chunk = (V + parts - 1) / parts;
    hipLaunchKernelGGL(argmax_part_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, part_val,
                       part_idx, V, chunk);
    hipLaunchKernelGGL(sample_sum_kernel, dim3(R, parts), dim3(kSampleThreads), 0, stream, logits, temperature,
                       part_val, part_sum, V, chunk);
    hipLaunchKernelGGL(sample_pick_kernel, dim3(R), dim3(kSampleThreads), 0, stream, logits, temperature, uniform,
                       part_val, part_idx, part_sum, out, V, chunk, parts, also, slot);
    return launch_status();
}

LLME_LOAD_ENTRY(sampling)
