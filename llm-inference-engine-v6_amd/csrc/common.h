// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wavefront (64-lane) reductions and the launch-error convention.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llme {

constexpr int kWave = 64;

// dtype codes shared with the Python side (ops/lib.py)
enum DType : int { kF32 = 0, kBF16 = 1 };

using bf16 = __bf16;

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16>(bf16 v) { return static_cast<float>(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
// float -> bf16 rounds to nearest, ties to even (the compiler's conversion).
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return static_cast<bf16>(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Sum over a whole workgroup of `nwaves` wavefronts; `scratch` holds >= nwaves floats.
// Every thread gets the result. Contains two barriers.
__device__ __forceinline__ float block_sum(float v, float* scratch, int nwaves) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < nwaves; ++i) total += scratch[i];
    return total;
}

// A workgroup barrier for data exchanged through LDS only: this wavefront's LDS traffic is
// complete before it and LDS reads start after it, but loads from global memory that are in
// flight stay in flight (__syncthreads also waits for those, which puts their whole latency
// in front of every barrier of a loop that prefetches).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// Compute units of the current device, asked once per process: launch heuristics are sized by
// it (how many workgroups fill the chip once, when a sum is worth cutting over k). 256 on the
// MI355X that the measurements quoted beside those heuristics were taken on.
inline int compute_units() {
    static int cached = 0;
    if (cached > 0) return cached;
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
        cus = 256;
    cached = cus;
    return cus;
}

// Every entry point returns hipGetLastError() after its launches: 0 on success.
inline int launch_status() { return static_cast<int>(hipGetLastError()); }

// Error codes of our own, above HIP's range, for arguments a kernel refuses.
constexpr int kErrBadArgument = 10001;
constexpr int kErrUnsupported = 10002;

}  // namespace llme

// The runtime loads a source file's device code when one of its kernels is first launched (or asked
// about). LLME_LOAD_ENTRY(name) gives the file an entry point llme_load_<name> that makes this happen,
// so that a caller can have every file's code on the device before it records launches into a graph.
#define LLME_LOAD_ENTRY(name)                                                                        \
    namespace { __global__ void load_probe_##name() {} }                                            \
    extern "C" int llme_load_##name(void) {                                                          \
        hipFuncAttributes attr;                                                                      \
        return static_cast<int>(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(&load_probe_##name))); \
    }
