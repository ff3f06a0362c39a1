// Prefill attention over bfloat16 cache pages with K and V shared through LDS.
// Formula as in the plain-precision kernel (src/kernels.cpp:413-474); tile arithmetic as in
// attention_tiles.h. What differs from the kernel that loads straight into registers is where
// the operands come from: a workgroup's four wavefronts need the same keys (heads of one kv
// head over the same rows, or neighbouring rows of one head), so the workgroup fetches every
// 64-key stretch of K and V once, 16 bytes per thread and load, into LDS, and each wavefront
// reads its operands from there. Global loads per key drop fourfold, and a thread holds only
// a few registers of data in flight, so the next stretch travels while this one is computed.
//
// Work item = (request, span of rows, group of HPW query heads of one kv head): wavefront w
// takes head w % HPW of the group and the row group w / HPW of the span, each row group being
// QT tiles of 16 rows. HPW is the largest of 4, 2, 1 that divides the heads per kv head.
// Stretches run from the first key the span's first row sees to the last row's own key; a
// wavefront skips the 32-key blocks that none of its rows sees and masks the rest by position.
//
// LDS: two stages of K [64 keys][hd + 8] (rows 16 bytes longer than the data, so that the
// 16-byte operand reads of 8 neighbouring keys fall into different banks) and V [hd][64 + 4]
// (8 bytes longer: the 8-byte reads of 16 neighbouring dims fall into different banks).
// Per stretch one barrier: after it the stage written during the last stretch is read, and
// the other, which everybody has finished reading, is written from the registers.
//
// Takes head sizes that are multiples of 32 up to 128 and pages that are multiples of 16; other
// sizes go to the kernel without LDS.
#include "attention_tiles.h"

namespace llme {

constexpr int KB = 64;                     // keys per stretch

template <int HD>
struct StageLayout {
    static constexpr int KS = HD + 8;      // K row stride (elements)
    static constexpr int VS = KB + 4;      // V row stride (elements)
    static constexpr int K_ELEMS = KB * KS;
    static constexpr int V_ELEMS = HD * VS;
    static constexpr int STAGE = K_ELEMS + V_ELEMS;
    static constexpr int BYTES = 2 * STAGE * 2;
};

// What one thread fetches of a stretch: NC chunks of 16 bytes of K and as many of V.
template <int HD>
struct Fetched {
    static constexpr int NC = HD / 32;     // 64 keys x hd / 8 chunks over 256 threads
    bf16x8 k[NC];
    bf16x8 v[NC];
};

// K chunk i of thread tid: key (0..63) and first dim; V chunk: 16-key half, dim and which 8 keys.
template <int HD>
__device__ __forceinline__ void k_chunk(int tid, int i, int& key, int& dim) {
    constexpr int CK = HD / 8;
    const int idx = tid + 256 * i;
    key = idx / CK;
    dim = (idx % CK) * 8;
}
template <int HD>
__device__ __forceinline__ void v_chunk(int tid, int i, int& half, int& dim, int& c2) {
    const int idx = tid + 256 * i;
    half = idx / (2 * HD);
    const int rem = idx % (2 * HD);
    dim = rem / 2;
    c2 = rem % 2;
}

// The page ids a thread's chunks of the stretch at t0 need (-1: the 16-key half has no key in
// [key_lo, key_end): nothing is read for it).
template <int HD>
__device__ __forceinline__ void lookup_stretch(const PagedKV& kv, int t0, int key_lo, int key_end, int tid,
                                               int (&pgk)[HD / 32], int (&pgv)[HD / 32]) {
#pragma unroll
    for (int i = 0; i < HD / 32; ++i) {
        int key, dim, half, c2;
        k_chunk<HD>(tid, i, key, dim);
        v_chunk<HD>(tid, i, half, dim, c2);
        const int hk = (t0 + key) & ~15, hv = t0 + 16 * half;
        pgk[i] = (hk < key_end && hk + 15 >= key_lo) ? kv.table[page_of(kv, hk).block] : -1;
        pgv[i] = (hv < key_end && hv + 15 >= key_lo) ? kv.table[page_of(kv, hv).block] : -1;
    }
}

template <int HD>
__device__ __forceinline__ void fetch_stretch(const PagedKV& kv, int t0, int tid, const int (&pgk)[HD / 32],
                                              const int (&pgv)[HD / 32], Fetched<HD>& f) {
#pragma unroll
    for (int i = 0; i < HD / 32; ++i) {
        int key, dim;
        k_chunk<HD>(tid, i, key, dim);
        const int t = t0 + key;
        const bool ok = pgk[i] >= 0;
        const bf16* src = kv.k + static_cast<size_t>(ok ? pgk[i] : 0) * kv.page_stride + kv.head_off +
                          static_cast<size_t>(page_of(kv, t & ~15).offset + (t & 15)) * HD + dim;
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(ok ? src : kv.k);
        f.k[i] = ok ? x : zero_frag();
    }
#pragma unroll
    for (int i = 0; i < HD / 32; ++i) {
        int half, dim, c2;
        v_chunk<HD>(tid, i, half, dim, c2);
        const int h0 = t0 + 16 * half;
        const bool ok = pgv[i] >= 0;
        const bf16* src = kv.v + static_cast<size_t>(ok ? pgv[i] : 0) * kv.page_stride + kv.head_off +
                          static_cast<size_t>(dim) * kv.page + page_of(kv, h0).offset + 8 * c2;
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(ok ? src : kv.v);
        f.v[i] = ok ? x : zero_frag();
    }
}

template <int HD>
__device__ __forceinline__ void store_stretch(bf16* stage, int tid, const Fetched<HD>& f) {
    using L = StageLayout<HD>;
#pragma unroll
    for (int i = 0; i < HD / 32; ++i) {
        int key, dim;
        k_chunk<HD>(tid, i, key, dim);
        *reinterpret_cast<bf16x8*>(stage + key * L::KS + dim) = f.k[i];
    }
    bf16* vs = stage + L::K_ELEMS;
#pragma unroll
    for (int i = 0; i < HD / 32; ++i) {
        int half, dim, c2;
        v_chunk<HD>(tid, i, half, dim, c2);
        bf16* dst = vs + dim * L::VS + 16 * half + 8 * c2;            // 8-byte aligned
        const bf16x4 lo = __builtin_shufflevector(f.v[i], f.v[i], 0, 1, 2, 3);
        const bf16x4 hi = __builtin_shufflevector(f.v[i], f.v[i], 4, 5, 6, 7);
        *reinterpret_cast<bf16x4*>(dst) = lo;
        *reinterpret_cast<bf16x4*>(dst + 4) = hi;
    }
}

// The operands of the 32-key block `sb` (0 or 1) of a stage, as attention_tiles.h lays them out.
template <int HD>
__device__ __forceinline__ void read_block(const bf16* stage, int sb, KFrag<HD>& kf, VFrag<HD>& vf) {
    using L = StageLayout<HD>;
    const int lane = threadIdx.x & 63, r = lane & 15, g4 = lane >> 4;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int c = 0; c < HD / 32; ++c)
            kf.kf[hf][c] = *reinterpret_cast<const bf16x8*>(stage + (32 * sb + 16 * hf + r) * L::KS + c * 32 + g4 * 8);
    const bf16* vs = stage + L::K_ELEMS;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
        const bf16* p = vs + (dt * 16 + r) * L::VS + 32 * sb + 4 * g4;
        const bf16x4 lo4 = *reinterpret_cast<const bf16x4*>(p);
        const bf16x4 hi4 = *reinterpret_cast<const bf16x4*>(p + 16);
        vf.vf[dt] = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
    }
}

template <int HD, int QT, int HPW>
__global__ __launch_bounds__(256) void attention_prefill_shared_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int max_blocks, int n_seq, int n_q, int n_kv, int page, float scale,
    int window) {
    constexpr int DC = HD / 32, DT = HD / 16, ROWS = 16 * QT, RG = 4 / HPW, SPAN = RG * ROWS;
    using L = StageLayout<HD>;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    bf16* lds = reinterpret_cast<bf16*>(lds_raw);

    // which request and which of its spans this workgroup has
    int s = 0, first = 0, n_span = 0, acc = 0;
    bool found = false;
    for (int i = 0; i < n_seq; ++i) {
        const int a = q_start[i], n = q_start[i + 1] - a;
        const int nt = (n >= 2) ? (n + SPAN - 1) / SPAN : 0;
        if (!found && static_cast<int>(blockIdx.x) < acc + nt) {
            s = i;
            first = (nt - 1 - (blockIdx.x - acc)) * SPAN;  // the last spans see the most keys and start first
            n_span = n - first < SPAN ? n - first : SPAN;
            first += a;                                    // as a batch row
            found = true;
        }
        acc += nt;
    }
    if (!found) return;                                    // the whole workgroup
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, r = lane & 15, g4 = lane >> 4;
    const int G = n_q / n_kv;
    const int head = blockIdx.y * HPW + wave % HPW;        // HPW divides G: one kv head per workgroup
    const int kvh = (blockIdx.y * HPW) / G;
    const int rg = wave / HPW;
    const int pos_span = ctx_len[s] + (first - q_start[s]); // position of the span's first row

    // this wavefront's rows
    const int first_w = first + rg * ROWS;
    int n_rows = n_span - rg * ROWS;
    n_rows = n_rows < 0 ? 0 : (n_rows > ROWS ? ROWS : n_rows);
    const int pos0 = pos_span + rg * ROWS;
    bf16x8 qf[QT][DC];
    int row_pos[QT], row_lo[QT], tile_free[QT];
    float m[QT], l[QT];
    f32x4 o[QT][DT];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        const int rr = qt * 16 + r;
        const bool ok = rr < n_rows;
        load_q<HD>(q + (static_cast<size_t>(ok ? first_w + rr : first) * n_q + head) * HD, ok, qf[qt]);
        row_pos[qt] = ok ? pos0 + rr : -1;
        row_lo[qt] = (window > 0 && pos0 + rr - window + 1 > 0) ? pos0 + rr - window + 1 : 0;
        tile_free[qt] = (window == 0 && qt * 16 + 16 <= n_rows) ? pos0 + qt * 16 : -1;
        m[qt] = kNoMax;
        l[qt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o[qt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int my_end = n_rows > 0 ? pos0 + n_rows : 0;      // this wavefront's rows see keys < my_end
    const int my_lo = (window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;

    // the workgroup's keys
    const int key_end = pos_span + n_span;
    const int key_lo = (window > 0 && pos_span - window + 1 > 0) ? pos_span - window + 1 : 0;
    const int k_begin = key_lo & ~(KB - 1);
    PagedKV kv{k_cache, v_cache, block_table + static_cast<size_t>(s) * max_blocks, page, n_kv, kvh, HD,
               page_magic_of(page), static_cast<size_t>(n_kv) * page * HD, static_cast<size_t>(kvh) * page * HD};
    const float scale_log2 = scale * kLog2e;

    Fetched<HD> fetched;
    int pgk[DC], pgv[DC];
    lookup_stretch<HD>(kv, k_begin, key_lo, key_end, tid, pgk, pgv);
    fetch_stretch<HD>(kv, k_begin, tid, pgk, pgv, fetched);
    lookup_stretch<HD>(kv, k_begin + KB, key_lo, key_end, tid, pgk, pgv);
    store_stretch<HD>(lds, tid, fetched);
    fetch_stretch<HD>(kv, k_begin + KB, tid, pgk, pgv, fetched);      // past key_end: page ids are -1, zeros
    lookup_stretch<HD>(kv, k_begin + 2 * KB, key_lo, key_end, tid, pgk, pgv);
    __syncthreads();
    int st = 0;
    for (int t0 = k_begin; t0 < key_end; t0 += KB, st ^= 1) {
        const bf16* stage = lds + st * L::STAGE;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
            const int tb = t0 + 32 * sb;
            if (tb < my_end && tb + 32 > my_lo) {           // the same for the whole wavefront
                KFrag<HD> kf;
                VFrag<HD> vf;
                read_block<HD>(stage, sb, kf, vf);
                f32x4 sc[QT][2];
                block_scores<HD, QT>(kf, qf, sc);
                bf16x8 pf[QT];
                block_weights<HD, QT>(sc, tb, row_pos, row_lo, tile_free, scale_log2, m, l, o, pf);
#pragma unroll
                for (int qt = 0; qt < QT; ++qt)
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt)
                        o[qt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[qt], vf.vf[dt], o[qt][dt], 0, 0, 0);
            }
        }
        if (t0 + KB < key_end) {                            // the same for the whole workgroup
            store_stretch<HD>(lds + (st ^ 1) * L::STAGE, tid, fetched);
            fetch_stretch<HD>(kv, t0 + 2 * KB, tid, pgk, pgv, fetched);
            lookup_stretch<HD>(kv, t0 + 3 * KB, key_lo, key_end, tid, pgk, pgv);
            __syncthreads();
        }
    }

#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float lt = l[qt];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int rr = g4 * 4 + e;
            const float l_row = __shfl(lt, rr, 64);
            const int row = qt * 16 + rr;
            if (row >= n_rows) continue;
            const float inv = 1.0f / l_row;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                out[(static_cast<size_t>(first_w + row) * n_q + head) * HD + dt * 16 + r] =
                    static_cast<bf16>(o[qt][dt][e] * inv);
        }
    }
}

static int heads_per_workgroup(int n_q, int n_kv) {
    const int G = n_q / n_kv;
    return G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);
}

// Rows per row group (16 QT) by head size; `wanted` rows per work item override it when they fit.
int prefill_shared_rows(int hd, int n_q, int n_kv, int wanted) {
    if (hd % 32 != 0 || hd <= 0 || hd > 128 || n_kv <= 0 || n_q % n_kv != 0) return 0;
    if (hd != 64 && hd != 128) return 0;
    const int rg = 4 / heads_per_workgroup(n_q, n_kv);
    int rows = 32;
    if (wanted > 0 && wanted % rg == 0 && (wanted / rg == 32 || (wanted / rg == 64 && hd <= 64))) rows = wanted / rg;
    return rows * rg;
}

template <int HD, int QT, int HPW>
static int launch_shared(const bf16* q, const bf16* kc, const bf16* vc, bf16* out, const int* q_start,
                         const int* ctx_len, const int* table, int max_blocks, int n_seq, int n_q, int n_kv, int page,
                         float scale, int window, int items, hipStream_t stream) {
    constexpr int LDS = StageLayout<HD>::BYTES;
    auto kernel = attention_prefill_shared_kernel<HD, QT, HPW>;
    static bool attr_set = false;                      // per instantiation
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set = true;
    }
    hipLaunchKernelGGL(kernel, dim3(items, n_q / HPW), dim3(256), LDS, stream, q, kc, vc, out, q_start, ctx_len, table,
                       max_blocks, n_seq, n_q, n_kv, page, scale, window);
    return launch_status();
}

int launch_prefill_shared(const bf16* q, const bf16* kc, const bf16* vc, bf16* out, const int* q_start,
                          const int* ctx_len, const int* table, int max_blocks, int n_seq, int n_q, int n_kv, int hd,
                          int page, float scale, int window, int items, int rows_per_item, hipStream_t stream) {
    const int hpw = heads_per_workgroup(n_q, n_kv);
    const int rows = rows_per_item / (4 / hpw);            // per row group
#define LLME_SHARED(HD, QT, HPW)                                                                               \
    if (hd == HD && rows == 16 * QT && hpw == HPW)                                                             \
        return launch_shared<HD, QT, HPW>(q, kc, vc, out, q_start, ctx_len, table, max_blocks, n_seq, n_q, n_kv, \
                                          page, scale, window, items, stream)
    LLME_SHARED(64, 2, 4); LLME_SHARED(64, 2, 2); LLME_SHARED(64, 2, 1);
    LLME_SHARED(64, 4, 4); LLME_SHARED(64, 4, 2); LLME_SHARED(64, 4, 1);
    LLME_SHARED(128, 2, 4); LLME_SHARED(128, 2, 2); LLME_SHARED(128, 2, 1);
#undef LLME_SHARED
    return kErrUnsupported;
}

}  // namespace llme
