// Row-wise kernels of the step: embedding gather, RMSNorm (optionally on chosen
// rows), the SiLU-gated product, rotary position encoding fused with the write
// of keys and values into cache pages.
//
// Formulas follow the reference's scalar kernels (src/kernels.cpp:18-31,59-66,
// 189-203 and the page addressing of src/paged_kv.cpp:88-111); statistics,
// rotation and activation are evaluated in 32-bit whatever the storage type.
#include "common.h"

namespace llme {

// ---------------------------------------------------------------------------------
// Zeros for a buffer that a product cut over k adds its parts into. n4 groups of four floats.
__global__ __launch_bounds__(256) void clear_kernel(float4* __restrict__ p, size_t n4) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n4; i += static_cast<size_t>(gridDim.x) * 256)
        p[i] = float4{0.f, 0.f, 0.f, 0.f};
}

// ---------------------------------------------------------------------------------
// out[t, :] = table[tokens[t], :]        (src/kernels.cpp:59-66; no scaling)
template <typename TW>
__global__ void embed_gather_kernel(const TW* __restrict__ table, const int* __restrict__ tokens,
                                    float* __restrict__ out, int H) {
    const int t = blockIdx.x;
    const TW* row = table + static_cast<size_t>(tokens[t]) * H;
    float* o = out + static_cast<size_t>(t) * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_float(row[i]);
}
// The same with eight elements per thread and load (H a multiple of 8, 16-byte aligned rows).
template <typename TW>
__global__ void embed_gather_vec_kernel(const TW* __restrict__ table, const int* __restrict__ tokens,
                                        float* __restrict__ out, int H) {
    const int t = blockIdx.x;
    const TW* row = table + static_cast<size_t>(tokens[t]) * H;
    float* o = out + static_cast<size_t>(t) * H;
    for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
        float v[8];
        if constexpr (sizeof(TW) == 2) {
            typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
            const bf16x8 x = *reinterpret_cast<const bf16x8*>(row + i);
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = static_cast<float>(x[j]);
        } else {
            const float4 a = *reinterpret_cast<const float4*>(row + i), b = *reinterpret_cast<const float4*>(row + i + 4);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        }
        *reinterpret_cast<float4*>(o + i) = float4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<float4*>(o + i + 4) = float4{v[4], v[5], v[6], v[7]};
    }
}

// The same from a bfloat16 table in the matrix kernels' blocked layout ([V / 16][H / 32] blocks of
// [4][16][8], V a multiple of 16 and H of 32): the head that is tied to the embedding reads the
// table as a weight matrix. A row's eight values of k = 8 j .. 8 j + 7 lie together.
__global__ void embed_gather_blocked_kernel(const bf16* __restrict__ table, const int* __restrict__ tokens,
                                            float* __restrict__ out, int H) {
    typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
    const int t = blockIdx.x;
    const int row = tokens[t];
    const bf16* group = table + static_cast<size_t>(row / 16) * 16 * H + (row % 16) * 8;
    float* o = out + static_cast<size_t>(t) * H;
    for (int j = threadIdx.x; j < H / 8; j += blockDim.x) {
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(group + static_cast<size_t>(j / 4) * 512 + (j % 4) * 128);
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = static_cast<float>(x[e]);
        *reinterpret_cast<float4*>(o + j * 8) = float4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<float4*>(o + j * 8 + 4) = float4{v[4], v[5], v[6], v[7]};
    }
}

// ---------------------------------------------------------------------------------
// out[r, i] = w[i] * x[row(r), i] * rsqrt(mean_i x^2 + eps)   (src/kernels.cpp:18-24)
// row(r) = rows ? rows[r] : r. The product is evaluated (w*x)*inv as the reference does.
// Four neighbouring values of a weight vector or of an output row in one load or store.
template <typename T>
__device__ __forceinline__ void norm_load4(const T* p, float (&v)[4]);
template <>
__device__ __forceinline__ void norm_load4<float>(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <>
__device__ __forceinline__ void norm_load4<bf16>(const bf16* p, float (&v)[4]) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(x[i]);
}
template <typename T>
__device__ __forceinline__ void norm_store4(T* p, const float (&v)[4]);
template <>
__device__ __forceinline__ void norm_store4<float>(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void norm_store4<bf16>(bf16* p, const float (&v)[4]) {
    typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
    bf16x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = static_cast<__bf16>(v[i]);
    *reinterpret_cast<bf16x4*>(p) = o;
}

// NV > 0: the row's length is a multiple of 4, at most 4 NV blockDim, and x, w and out are aligned
// for 16-byte (bfloat16: 8-byte) accesses: a thread then keeps its up to NV groups of four values
// and their weights in registers between the two passes, all asked for at once, and stores four
// values at a time. NV = 0: the row is read twice, value by value.
template <typename TW, typename TO, int NVEC>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                               TO* __restrict__ out, const int* __restrict__ rows, int H, float eps) {
    __shared__ float scratch[16];
    constexpr bool VEC = NVEC > 0;
    constexpr int NV = VEC ? NVEC : 1;
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + static_cast<size_t>(src) * H;
    TO* o = out + static_cast<size_t>(r) * H;
    float v[NV][4], wv[NV][4];
    float ss = 0.f;
    if (VEC) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = (threadIdx.x + j * blockDim.x) * 4;
            if (i < H) {
                norm_load4<float>(xr + i, v[j]);
                norm_load4<TW>(w + i, wv[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = (threadIdx.x + j * blockDim.x) * 4;
            if (i < H) ss += v[j][0] * v[j][0] + v[j][1] * v[j][1] + v[j][2] * v[j][2] + v[j][3] * v[j][3];
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x) {
            const float t = xr[i];
            ss += t * t;
        }
    }
    ss = block_sum(ss, scratch, blockDim.x / kWave);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps);
    if (VEC) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int i = (threadIdx.x + j * blockDim.x) * 4;
            if (i >= H) continue;
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = (wv[j][e] * v[j][e]) * inv;
            norm_store4<TO>(o + i, y);
        }
    } else {
        for (int i = threadIdx.x; i < H; i += blockDim.x)
            o[i] = from_float<TO>((to_float(w[i]) * xr[i]) * inv);
    }
}

// ---------------------------------------------------------------------------------
// out[t, j] = silu(gate[t, j]) * up[t, j]      (src/kernels.cpp:26-31, src/engine.cpp:215-216)
// gu is [T, 2*FF]; gate and up alternate in groups of `group` columns:
// gate j sits at (j / group) * 2 * group + j % group, up `group` columns later.
// group == FF is the plain "all gates, then all ups" layout.
template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gu, TO* __restrict__ out, int FF, int group, size_t total) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const size_t t = idx / FF;
    const int j = static_cast<int>(idx % FF);
    const size_t base = t * 2 * static_cast<size_t>(FF) + static_cast<size_t>(j / group) * 2 * group + (j % group);
    const float g = to_float(gu[base]);
    const float u = to_float(gu[base + group]);
    out[idx] = from_float<TO>((g / (1.0f + expf(-g))) * u);
}

// ---------------------------------------------------------------------------------
// Rotary encoding of q and k heads (pairs (i, i + rot/2), src/kernels.cpp:189-203),
// q written to q_out, rotated k and plain v written into the token's cache page.
//   qkv     [T, (n_q + 2 n_kv) * hd] 32-bit: q heads, then k heads, then v heads
//   cos,sin [max_pos, rot/2] 32-bit (null: no rotation)
//   k_cache [pages, n_kv, page, hd]      v_cache [pages, n_kv, hd, page]
//   block_table [n_seq, max_blocks]; the token's page is block_table[seq][pos / page]
template <typename TQ, typename TC>
__global__ void rope_kv_write_kernel(const float* __restrict__ qkv, const float* __restrict__ cos_t,
                                     const float* __restrict__ sin_t, const int* __restrict__ positions,
                                     const int* __restrict__ seq_idx, const int* __restrict__ block_table,
                                     int max_blocks, TQ* __restrict__ q_out, TC* __restrict__ k_cache,
                                     TC* __restrict__ v_cache, int n_q, int n_kv, int hd, int rot,
                                     int page, int write_cache) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    const int half = rot / 2;
    const float* row = qkv + static_cast<size_t>(t) * (n_q + 2 * n_kv) * hd;
    const float* cs = cos_t ? cos_t + static_cast<size_t>(pos) * half : nullptr;
    const float* sn = sin_t ? sin_t + static_cast<size_t>(pos) * half : nullptr;

    // q heads: pairs inside the rotated span, plain copy behind it
    TQ* qo = q_out + static_cast<size_t>(t) * n_q * hd;
    const int pairs_q = n_q * half;
    for (int e = threadIdx.x; e < pairs_q; e += blockDim.x) {
        const int h = e / half, i = e % half;
        const float a = row[h * hd + i], b = row[h * hd + i + half];
        const float c = cs ? cs[i] : 1.f, s = sn ? sn[i] : 0.f;
        qo[h * hd + i] = from_float<TQ>(a * c - b * s);
        qo[h * hd + i + half] = from_float<TQ>(b * c + a * s);
    }
    const int tail = hd - rot;
    for (int e = threadIdx.x; e < n_q * tail; e += blockDim.x) {
        const int h = e / tail, i = rot + e % tail;
        qo[h * hd + i] = from_float<TQ>(row[h * hd + i]);
    }
    if (!write_cache) return;

    const int s_idx = seq_idx[t];
    const int pg = block_table[static_cast<size_t>(s_idx) * max_blocks + pos / page];
    const int off = pos % page;
    const float* krow = row + n_q * hd;
    const float* vrow = krow + n_kv * hd;
    for (int e = threadIdx.x; e < n_kv * half; e += blockDim.x) {
        const int h = e / half, i = e % half;
        const float a = krow[h * hd + i], b = krow[h * hd + i + half];
        const float c = cs ? cs[i] : 1.f, s = sn ? sn[i] : 0.f;
        TC* kd = k_cache + ((static_cast<size_t>(pg) * n_kv + h) * page + off) * hd;
        kd[i] = from_float<TC>(a * c - b * s);
        kd[i + half] = from_float<TC>(b * c + a * s);
    }
    for (int e = threadIdx.x; e < n_kv * tail; e += blockDim.x) {
        const int h = e / tail, i = rot + e % tail;
        k_cache[((static_cast<size_t>(pg) * n_kv + h) * page + off) * hd + i] = from_float<TC>(krow[h * hd + i]);
    }
    for (int e = threadIdx.x; e < n_kv * hd; e += blockDim.x) {
        const int h = e / hd, d = e % hd;
        v_cache[((static_cast<size_t>(pg) * n_kv + h) * hd + d) * page + off] = from_float<TC>(vrow[e]);
    }
}

// The same for the usual case (all of a head's dims rotated, head size a multiple of 16), eight
// dims per thread: 32-byte loads of the projection's row and of the tables, 16-byte stores of q
// and k. One workgroup per token; a thread takes 8 dims of one half of a q or k head together
// with their partners in the other half, or 8 dims of a v head.
template <typename T>
__device__ __forceinline__ void store8(T* dst, const float (&v)[8]);
template <>
__device__ __forceinline__ void store8<float>(float* dst, const float (&v)[8]) {
    *reinterpret_cast<float4*>(dst) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4*>(dst + 4) = float4{v[4], v[5], v[6], v[7]};
}
template <>
__device__ __forceinline__ void store8<bf16>(bf16* dst, const float (&v)[8]) {
    typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = static_cast<__bf16>(v[j]);
    *reinterpret_cast<bf16x8*>(dst) = o;
}
__device__ __forceinline__ void load8(const float* src, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// ZERO: every value of qkv is set to zero once it has been read (each is read by one thread, once, when
// the cache is written too): a buffer that a product cut over k adds its parts into is then ready
// for the next layer's product without a kernel that clears it.
template <typename TQ, typename TC, bool ZERO>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(
    float* qkv, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ seq_idx, const int* __restrict__ block_table,
    int max_blocks, TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache, int n_q, int n_kv,
    int hd, int page, int write_cache) {
    const int t = blockIdx.x;
    const int pos = positions[t];
    int pg = 0, off = 0;
    if (write_cache) {
        pg = block_table[static_cast<size_t>(seq_idx[t]) * max_blocks + pos / page];
        off = pos % page;
    }
    const int half = hd / 2, hv = half / 8, dv = hd / 8;
    float* row = qkv + static_cast<size_t>(t) * (n_q + 2 * n_kv) * hd;
    const float* cs = cos_t + static_cast<size_t>(pos) * half;
    const float* sn = sin_t + static_cast<size_t>(pos) * half;
    const int q_items = n_q * hv, k_items = n_kv * hv, v_items = n_kv * dv;
    const int items = q_items + (write_cache ? k_items + v_items : 0);
    const float4 zero4{0.f, 0.f, 0.f, 0.f};
    for (int it = threadIdx.x; it < items; it += blockDim.x) {
        if (it < q_items + k_items) {
            const bool is_q = it < q_items;
            const int e = is_q ? it : it - q_items;
            const int h = e / hv, i = (e % hv) * 8;
            float* src = row + (is_q ? 0 : n_q * hd) + h * hd + i;
            float a[8], b[8], c[8], sv[8], lo[8], hi[8];
            load8(src, a);
            load8(src + half, b);
            if (ZERO) {
                reinterpret_cast<float4*>(src)[0] = zero4;
                reinterpret_cast<float4*>(src)[1] = zero4;
                reinterpret_cast<float4*>(src + half)[0] = zero4;
                reinterpret_cast<float4*>(src + half)[1] = zero4;
            }
            load8(cs + i, c);
            load8(sn + i, sv);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                lo[j] = a[j] * c[j] - b[j] * sv[j];
                hi[j] = b[j] * c[j] + a[j] * sv[j];
            }
            if (is_q) {
                TQ* dst = q_out + (static_cast<size_t>(t) * n_q + h) * hd + i;
                store8<TQ>(dst, lo);
                store8<TQ>(dst + half, hi);
            } else {
                TC* dst = k_cache + ((static_cast<size_t>(pg) * n_kv + h) * page + off) * hd + i;
                store8<TC>(dst, lo);
                store8<TC>(dst + half, hi);
            }
        } else {
            const int e = it - q_items - k_items;
            const int h = e / dv, d0 = (e % dv) * 8;
            float v[8];
            float* src = row + (n_q + n_kv) * hd + h * hd + d0;
            load8(src, v);
            if (ZERO) {
                reinterpret_cast<float4*>(src)[0] = zero4;
                reinterpret_cast<float4*>(src)[1] = zero4;
            }
            TC* dst = v_cache + ((static_cast<size_t>(pg) * n_kv + h) * hd + d0) * page + off;
#pragma unroll
            for (int j = 0; j < 8; ++j) dst[static_cast<size_t>(j) * page] = from_float<TC>(v[j]);
        }
    }
}

// The same for many tokens (prompts): a workgroup takes 16 consecutive tokens. Where they are 16
// consecutive positions of one request that begin at a multiple of 16 (the usual case in a
// prompt: they then lie in one page, whose size is a multiple of 16), a thread writes the 16
// values of one v dim as one contiguous piece; otherwise value by value as above. ROPE_PARTS
// workgroups share a group's work so that a prompt of a few thousand tokens fills the chip.
constexpr int ROPE_GROUP = 16, ROPE_PARTS = 4;
template <typename TQ, typename TC>
__global__ __launch_bounds__(256) void rope_kv_write_group_kernel(
    const float* __restrict__ qkv, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
    const int* __restrict__ positions, const int* __restrict__ seq_idx, const int* __restrict__ block_table,
    int max_blocks, TQ* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache, int n_q, int n_kv,
    int hd, int page, int write_cache, int T) {
    const int t0 = blockIdx.x * ROPE_GROUP;
    const int nt = T - t0 < ROPE_GROUP ? T - t0 : ROPE_GROUP;
    const int first = blockIdx.y * blockDim.x + threadIdx.x, stride = gridDim.y * blockDim.x;   // the group's work is dealt to gridDim.y workgroups
    const int half = hd / 2, hv = half / 8;
    const size_t row_len = static_cast<size_t>(n_q + 2 * n_kv) * hd;
    const int q_items = n_q * hv, k_items = write_cache ? n_kv * hv : 0;
    const int per_token = q_items + k_items;
    for (int it = first; it < nt * per_token; it += stride) {
        const int t = t0 + it / per_token, e0 = it % per_token;
        const bool is_q = e0 < q_items;
        const int e = is_q ? e0 : e0 - q_items;
        const int h = e / hv, i = (e % hv) * 8;
        const int pos = positions[t];
        const float* src = qkv + t * row_len + (is_q ? 0 : n_q * hd) + h * hd + i;
        float a[8], b[8], c[8], sv[8], lo[8], hi[8];
        load8(src, a);
        load8(src + half, b);
        load8(cos_t + static_cast<size_t>(pos) * half + i, c);
        load8(sin_t + static_cast<size_t>(pos) * half + i, sv);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            lo[j] = a[j] * c[j] - b[j] * sv[j];
            hi[j] = b[j] * c[j] + a[j] * sv[j];
        }
        if (is_q) {
            TQ* dst = q_out + (static_cast<size_t>(t) * n_q + h) * hd + i;
            store8<TQ>(dst, lo);
            store8<TQ>(dst + half, hi);
        } else {
            const int pg = block_table[static_cast<size_t>(seq_idx[t]) * max_blocks + pos / page];
            TC* dst = k_cache + ((static_cast<size_t>(pg) * n_kv + h) * page + pos % page) * hd + i;
            store8<TC>(dst, lo);
            store8<TC>(dst + half, hi);
        }
    }
    if (!write_cache) return;
    const int v_dims = n_kv * hd;
    const float* vsrc = qkv + t0 * row_len + static_cast<size_t>(n_q + n_kv) * hd;
    const int pos0 = positions[t0];
    const bool together = nt == ROPE_GROUP && seq_idx[t0] == seq_idx[t0 + ROPE_GROUP - 1] &&
                          pos0 % ROPE_GROUP == 0 && page % ROPE_GROUP == 0;    // the same for the whole workgroup
    if (together) {
        const int pg = block_table[static_cast<size_t>(seq_idx[t0]) * max_blocks + pos0 / page];
        const int off0 = pos0 % page;
        for (int e = first; e < v_dims; e += stride) {
            float lo[8], hi[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                lo[j] = vsrc[j * row_len + e];
                hi[j] = vsrc[(j + 8) * row_len + e];
            }
            TC* dst = v_cache + ((static_cast<size_t>(pg) * n_kv + e / hd) * hd + e % hd) * page + off0;
            store8<TC>(dst, lo);
            store8<TC>(dst + 8, hi);
        }
    } else {
        for (int it = first; it < nt * v_dims; it += stride) {
            const int tt = it / v_dims, e = it % v_dims;
            const int pos = positions[t0 + tt];
            const int pg = block_table[static_cast<size_t>(seq_idx[t0 + tt]) * max_blocks + pos / page];
            v_cache[((static_cast<size_t>(pg) * n_kv + e / hd) * hd + e % hd) * page + pos % page] =
                from_float<TC>(vsrc[tt * row_len + e]);
        }
    }
}

}  // namespace llme

using namespace llme;

// n floats, a multiple of 4, at a 16-byte aligned address.
extern "C" int llme_clear_f32(float* p, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    if (n % 4 != 0 || reinterpret_cast<uintptr_t>(p) % 16 != 0) return kErrUnsupported;
    const size_t n4 = n / 4;
    const unsigned grid = static_cast<unsigned>(n4 / 256 + 1 < 1024 ? n4 / 256 + 1 : 1024);
    hipLaunchKernelGGL(clear_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<float4*>(p), n4);
    return launch_status();
}

extern "C" int llme_embed_gather(const void* table, int table_dtype, const int* tokens, float* out, int T,
                                 int H, int blocked, hipStream_t stream) {
    if (T <= 0) return 0;
    if (blocked) {
        if (table_dtype != kBF16 || H % 32 != 0 || reinterpret_cast<uintptr_t>(table) % 16 != 0 ||
            reinterpret_cast<uintptr_t>(out) % 16 != 0)
            return kErrUnsupported;
        hipLaunchKernelGGL(embed_gather_blocked_kernel, dim3(T), dim3(256), 0, stream, static_cast<const bf16*>(table),
                           tokens, out, H);
        return launch_status();
    }
    const bool vec = H % 8 == 0 && reinterpret_cast<uintptr_t>(table) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
#define LLME_EMBED(TW)                                                                                     \
    do {                                                                                                   \
        if (vec)                                                                                           \
            hipLaunchKernelGGL(embed_gather_vec_kernel<TW>, dim3(T), dim3(256), 0, stream,                 \
                               static_cast<const TW*>(table), tokens, out, H);                             \
        else                                                                                               \
            hipLaunchKernelGGL(embed_gather_kernel<TW>, dim3(T), dim3(256), 0, stream,                     \
                               static_cast<const TW*>(table), tokens, out, H);                             \
    } while (0)
    if (table_dtype == kF32) LLME_EMBED(float);
    else if (table_dtype == kBF16) LLME_EMBED(bf16);
    else return kErrBadArgument;
#undef LLME_EMBED
    return launch_status();
}

extern "C" int llme_compute_units(void) { return compute_units(); }

extern "C" int llme_rmsnorm(const float* x, const void* w, int w_dtype, void* out, int out_dtype,
                            const int* rows, int R, int H, float eps, hipStream_t stream) {
    if (R <= 0) return 0;
    const bool vec = H % 4 == 0 && H <= 32 * 256 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    const int nv = !vec ? 0 : H <= 8 * 256 ? 2 : H <= 16 * 256 ? 4 : 8;      // groups of four per thread
#define LLME_NORM_NV(TW, TO, NV)                                                                  \
    hipLaunchKernelGGL((rmsnorm_kernel<TW, TO, NV>), dim3(R), dim3(256), 0, stream, x,            \
                       static_cast<const TW*>(w), static_cast<TO*>(out), rows, H, eps)
#define LLME_NORM(TW, TO)                                                                         \
    do {                                                                                          \
        if (nv == 2) LLME_NORM_NV(TW, TO, 2);                                                     \
        else if (nv == 4) LLME_NORM_NV(TW, TO, 4);                                                \
        else if (nv == 8) LLME_NORM_NV(TW, TO, 8);                                                \
        else LLME_NORM_NV(TW, TO, 0);                                                             \
    } while (0)
    if (w_dtype == kF32 && out_dtype == kF32) LLME_NORM(float, float);
    else if (w_dtype == kF32 && out_dtype == kBF16) LLME_NORM(float, bf16);
    else if (w_dtype == kBF16 && out_dtype == kF32) LLME_NORM(bf16, float);
    else if (w_dtype == kBF16 && out_dtype == kBF16) LLME_NORM(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_NORM
#undef LLME_NORM_NV
    return launch_status();
}

extern "C" int llme_swiglu(const void* gu, int in_dtype, void* out, int out_dtype, int T, int FF, int group,
                           hipStream_t stream) {
    if (T <= 0) return 0;
    if (group <= 0 || FF % group != 0) return kErrBadArgument;
    const size_t total = static_cast<size_t>(T) * FF;
    const dim3 grid(static_cast<unsigned>((total + 255) / 256));
#define LLME_SWIGLU(TI, TO)                                                                      \
    hipLaunchKernelGGL((swiglu_kernel<TI, TO>), grid, dim3(256), 0, stream,                      \
                       static_cast<const TI*>(gu), static_cast<TO*>(out), FF, group, total)
    if (in_dtype == kF32 && out_dtype == kF32) LLME_SWIGLU(float, float);
    else if (in_dtype == kF32 && out_dtype == kBF16) LLME_SWIGLU(float, bf16);
    else if (in_dtype == kBF16 && out_dtype == kBF16) LLME_SWIGLU(bf16, bf16);
    else return kErrBadArgument;
#undef LLME_SWIGLU
    return launch_status();
}

// zero_input (with write_cache): qkv is all zeros afterwards (by the kernel itself where one thread
// reads each value once, else by the clearing kernel behind it).
extern "C" int llme_rope_kv_write(float* qkv, const float* cos_t, const float* sin_t,
                                  const int* positions, const int* seq_idx, const int* block_table,
                                  int max_blocks, void* q_out, int q_dtype, void* k_cache, void* v_cache,
                                  int cache_dtype, int T, int n_q, int n_kv, int hd, int rot, int page,
                                  int write_cache, int zero_input, hipStream_t stream) {
    if (T <= 0) return 0;
    if (zero_input && !write_cache) return kErrBadArgument;
    if (rot < 0 || rot > hd || rot % 2 != 0 || page <= 0) return kErrBadArgument;
    // all dims rotated and head sizes in steps of 16: the kernel that moves 8 dims per thread
    const bool vec = rot == hd && hd % 16 == 0 && cos_t != nullptr && sin_t != nullptr &&
                     reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(q_out) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 && reinterpret_cast<uintptr_t>(cos_t) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(sin_t) % 16 == 0;
    // many tokens: 16 per workgroup, v written in pieces of 16 positions where they lie together
    // (up to 256 tokens, which may be as many decoding requests with a page each, a workgroup per
    // token is faster: 5.2 against 9.5 us for 64 single tokens)
    const bool grouped = vec && T > 16 * ROPE_GROUP && reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
#define LLME_ROPE(TQ, TC)                                                                                   \
    do {                                                                                                    \
        if (grouped)                                                                                        \
            hipLaunchKernelGGL((rope_kv_write_group_kernel<TQ, TC>),                                       \
                               dim3((T + ROPE_GROUP - 1) / ROPE_GROUP, ROPE_PARTS),                         \
                               dim3(256), 0, stream, qkv, cos_t, sin_t, positions, seq_idx, block_table,    \
                               max_blocks, static_cast<TQ*>(q_out), static_cast<TC*>(k_cache),              \
                               static_cast<TC*>(v_cache), n_q, n_kv, hd, page, write_cache, T);             \
        else if (vec && zero_input)                                                                         \
            hipLaunchKernelGGL((rope_kv_write_vec_kernel<TQ, TC, true>), dim3(T), dim3(256), 0, stream, qkv, \
                               cos_t, sin_t, positions, seq_idx, block_table, max_blocks,                  \
                               static_cast<TQ*>(q_out), static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), \
                               n_q, n_kv, hd, page, write_cache);                                           \
        else if (vec)                                                                                       \
            hipLaunchKernelGGL((rope_kv_write_vec_kernel<TQ, TC, false>), dim3(T), dim3(256), 0, stream, qkv, \
                               cos_t, sin_t, positions, seq_idx, block_table, max_blocks,                  \
                               static_cast<TQ*>(q_out), static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), \
                               n_q, n_kv, hd, page, write_cache);                                           \
        else                                                                                                \
            hipLaunchKernelGGL((rope_kv_write_kernel<TQ, TC>), dim3(T), dim3(256), 0, stream, qkv, cos_t,   \
                               sin_t, positions, seq_idx, block_table, max_blocks, static_cast<TQ*>(q_out), \
                               static_cast<TC*>(k_cache), static_cast<TC*>(v_cache), n_q, n_kv, hd, rot,    \
                               page, write_cache);                                                          \
    } while (0)
    if (q_dtype == kF32 && cache_dtype == kF32) LLME_ROPE(float, float);
    else if (q_dtype == kBF16 && cache_dtype == kBF16) LLME_ROPE(bf16, bf16);
    else if (q_dtype == kF32 && cache_dtype == kBF16) LLME_ROPE(float, bf16);
    else if (q_dtype == kBF16 && cache_dtype == kF32) LLME_ROPE(bf16, float);
    else return kErrBadArgument;
#undef LLME_ROPE
    if (zero_input && !(vec && !grouped)) {
        const int status = launch_status();
        if (status != 0) return status;
        const size_t n = static_cast<size_t>(T) * (n_q + 2 * n_kv) * hd;
        if (n % 4 != 0 || reinterpret_cast<uintptr_t>(qkv) % 16 != 0) return kErrUnsupported;
        const size_t n4 = n / 4;
        const unsigned grid = static_cast<unsigned>(n4 / 256 + 1 < 1024 ? n4 / 256 + 1 : 1024);
        hipLaunchKernelGGL(clear_kernel, dim3(grid), dim3(256), 0, stream, reinterpret_cast<float4*>(qkv), n4);
    }
    return launch_status();
}

LLME_LOAD_ENTRY(elementwise)
