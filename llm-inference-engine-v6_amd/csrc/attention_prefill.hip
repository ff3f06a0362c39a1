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
// LDS: two stages of K [64 keys][hd + 16] and V [hd][64 + 8]. The paddings are measured: LDS
// has 64 banks of 4 bytes; the 16-byte operand reads (lane = key l % 16, dims 8 (l / 16) ..) run
// at full rate with rows of 2 hd + 32 bytes and at half rate with 2 hd + 16, the 8-byte reads
// of V (lane = dim l % 16, keys 4 (l / 16) ..) at full rate with rows of 144 bytes.
// Per stretch one barrier: after it the stage written during the last stretch is read, and
// the other, which everybody has finished reading, is written from the registers.
//
// Takes head sizes 64 and 128 and pages that are multiples of 16; other sizes go to the kernel
// without LDS.
//
// Few rows over a long context (a portion of a prompt far into it) are few work items that each
// walk many keys, and in a prompt of a few thousand tokens the items of the last rows take twice
// the average while the chip has room left. Then an item's keys are cut into up to `nsplit` runs of
// `run` stretches, one work item each, which leave their rows' maxima, sums and unscaled outputs
// in 32-bit scratch indexed by batch row; a second kernel joins them, as it joins the splits of
// the decode kernel. Items with few keys have one run and write their output themselves.
#include "attention_tiles.h"

namespace llme {

constexpr int KB = 64;                     // keys per stretch

template <int HD>
struct StageLayout {
    static constexpr int KS = HD + 16;     // K row stride (elements)
    static constexpr int VS = KB + 8;      // V row stride (elements)
    static constexpr int K_ELEMS = KB * KS;
    static constexpr int V_ELEMS = HD * VS;
    static constexpr int STAGE = K_ELEMS + V_ELEMS;
    static constexpr int BYTES = 2 * STAGE * 2;
};

// What one thread fetches of a stretch: NC chunks of 16 bytes of K and as many of V. Chunk i
// of thread tid has the running number tid + threads i; of K it is key idx / (hd / 8), dims
// 8 (idx % (hd / 8)) ..; of V the 16-key half idx / (2 hd), dim (idx % (2 hd)) / 2, keys
// 8 (idx % 2) .. of the half. For head sizes 64 and 128 the 64 chunks of a wavefront then lie
// in one 16-key half, the same for K and V: (64 wave + threads i) / (2 hd). A half has one page,
// so the page's id, whether the half is to be read at all and the page's address are the
// same for the whole wavefront: scalar work, and the loads take a scalar base and a 32-bit
// offset per lane that never changes.
template <int HD, int THREADS>
struct Fetched {
    static constexpr int NC = HD * 8 / THREADS;    // 64 keys x hd / 8 chunks over the workgroup's threads
    bf16x8 k[NC];
    bf16x8 v[NC];
};

template <int HD, int THREADS>
__device__ __forceinline__ int chunk_half(int wave, int i) { return (64 * wave + THREADS * i) / (2 * HD); }

// Per lane and chunk, fixed for the kernel: offsets (elements) from the start of the half's
// keys in its page (K) or of the kv head's part of the page (V), and the places in a stage.
template <int HD, int THREADS>
struct ChunkPlaces {
    static constexpr int NC = HD * 8 / THREADS;
    unsigned k_off[NC], v_off[NC];         // global, in elements
    unsigned k_lds[NC], v_lds[NC];         // in a stage, in elements
};

template <int HD, int THREADS>
__device__ __forceinline__ ChunkPlaces<HD, THREADS> chunk_places(int tid, int page) {
    using L = StageLayout<HD>;
    constexpr int CK = HD / 8;
    ChunkPlaces<HD, THREADS> c;
#pragma unroll
    for (int i = 0; i < HD * 8 / THREADS; ++i) {
        const int idx = tid + THREADS * i;
        const int key = idx / CK, dim = (idx % CK) * 8;
        c.k_off[i] = (key & 15) * HD + dim;
        c.k_lds[i] = key * L::KS + dim;
        const int half = idx / (2 * HD), rem = idx % (2 * HD);
        const int vdim = rem / 2, c2 = rem % 2;
        c.v_off[i] = vdim * page + 8 * c2;
        c.v_lds[i] = L::K_ELEMS + vdim * L::VS + 16 * half + 8 * c2;
    }
    return c;
}

// The pages of the NC halves that this wavefront fetches of the stretch at t0: page id (or -1:
// the half has no key in [key_lo, key_end), nothing is read for it) and the first key's place
// in the page. All scalar.
template <int HD, int THREADS>
struct StretchPages {
    int pg[HD * 8 / THREADS];
    int off[HD * 8 / THREADS];
};

template <int HD, int THREADS>
__device__ __forceinline__ StretchPages<HD, THREADS> lookup_stretch(const PagedKV& kv, int t0, int key_lo, int key_end,
                                                                    int wave) {
    StretchPages<HD, THREADS> p;
#pragma unroll
    for (int i = 0; i < HD * 8 / THREADS; ++i) {
        const int h0 = t0 + 16 * chunk_half<HD, THREADS>(wave, i);
        const PagePlace pl = page_of(kv, h0);
        p.off[i] = pl.offset;
        p.pg[i] = (h0 < key_end && h0 + 15 >= key_lo) ? __builtin_amdgcn_readfirstlane(kv.table[pl.block]) : -1;
    }
    return p;
}

// Every turn issues the same loads: a half that is not to be read reads the pool's first page
// instead and counts as zeros.
template <int HD, int THREADS>
__device__ __forceinline__ void fetch_stretch(const PagedKV& kv, const StretchPages<HD, THREADS>& p,
                                              const ChunkPlaces<HD, THREADS>& c, Fetched<HD, THREADS>& f) {
#pragma unroll
    for (int i = 0; i < HD * 8 / THREADS; ++i) {
        const bool ok = p.pg[i] >= 0;                                                     // scalar
        const size_t base = static_cast<size_t>(ok ? p.pg[i] : 0) * kv.page_stride + kv.head_off;   // scalar
        const bf16* ksrc = kv.k + base + static_cast<size_t>(ok ? p.off[i] : 0) * HD;
        const bf16* vsrc = kv.v + base + (ok ? p.off[i] : 0);
        const bf16x8 xk = *reinterpret_cast<const bf16x8*>(ksrc + c.k_off[i]);
        const bf16x8 xv = *reinterpret_cast<const bf16x8*>(vsrc + c.v_off[i]);
        f.k[i] = ok ? xk : zero_frag();
        f.v[i] = ok ? xv : zero_frag();
    }
}

template <int HD, int THREADS>
__device__ __forceinline__ void store_stretch(bf16* stage, const ChunkPlaces<HD, THREADS>& c,
                                              const Fetched<HD, THREADS>& f) {
#pragma unroll
    for (int i = 0; i < HD * 8 / THREADS; ++i) {
        *reinterpret_cast<bf16x8*>(stage + c.k_lds[i]) = f.k[i];
        *reinterpret_cast<bf16x8*>(stage + c.v_lds[i]) = f.v[i];
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

// One work item: span `bx` (counted over the requests with two or more tokens, the last spans of
// a request first) for head group `by`, run `z` of its keys (SPLIT; else all keys).
template <int HD, int QT, int HPW, int KW, bool SPLIT>
__device__ __forceinline__ void prefill_item(int bx, int by, int z, int nsplit, int run, float* __restrict__ part_o,
                                             float* __restrict__ part_ml, bf16* lds, const bf16* __restrict__ q,
                                             const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
                                             bf16* __restrict__ out, const int* __restrict__ q_start,
                                             const int* __restrict__ ctx_len, const int* __restrict__ block_table,
                                             int max_blocks, int n_seq, int n_q, int n_kv, int page, float scale,
                                             int window) {
    constexpr int DC = HD / 32, DT = HD / 16, ROWS = 16 * QT, RG = 4 / HPW, SPAN = RG * ROWS;
    constexpr int THREADS = 256 * KW;
    using L = StageLayout<HD>;

    // which request and which of its spans this workgroup has
    int s = 0, first = 0, n_span = 0, acc = 0;
    bool found = false;
    for (int i = 0; i < n_seq; ++i) {
        const int a = q_start[i], n = q_start[i + 1] - a;
        const int nt = (n >= 2) ? (n + SPAN - 1) / SPAN : 0;
        if (!found && bx < acc + nt) {
            s = i;
            first = (nt - 1 - (bx - acc)) * SPAN;          // the last spans see the most keys and start first
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
    const int tile = wave % 4;                             // which rows and head; KW wavefronts share a tile
    const int ks = wave / 4;                               // and take the 32-key blocks sb with sb % KW == ks
    const int head = by * HPW + tile % HPW;                // HPW divides G: one kv head per workgroup
    const int kvh = (by * HPW) / G;
    const int rg = tile / HPW;
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
    int key_end = pos_span + n_span;
    const int key_lo = (window > 0 && pos_span - window + 1 > 0) ? pos_span - window + 1 : 0;
    int k_begin = key_lo & ~(KB - 1);
    int runs = 1;
    if (SPLIT) {
        runs = key_runs(k_begin, key_end, run, nsplit);
        if (z >= runs) return;                             // (the whole workgroup: no such run)
        k_begin += z * run * KB;
        if (z < runs - 1) key_end = k_begin + run * KB;    // (the last run takes the rest)
    }
    PagedKV kv{k_cache, v_cache, block_table + static_cast<size_t>(s) * max_blocks, page, n_kv, kvh, HD,
               page_magic_of(page), static_cast<unsigned>(n_kv) * page * HD, static_cast<unsigned>(kvh) * page * HD};
    const float scale_log2 = scale * kLog2e;

    const ChunkPlaces<HD, THREADS> places = chunk_places<HD, THREADS>(tid, page);
    Fetched<HD, THREADS> fetched;
    StretchPages<HD, THREADS> pages = lookup_stretch<HD, THREADS>(kv, k_begin, key_lo, key_end, wave);
    fetch_stretch<HD, THREADS>(kv, pages, places, fetched);
    pages = lookup_stretch<HD, THREADS>(kv, k_begin + KB, key_lo, key_end, wave);
    store_stretch<HD, THREADS>(lds, places, fetched);
    fetch_stretch<HD, THREADS>(kv, pages, places, fetched);           // past key_end: no page ids, zeros
    pages = lookup_stretch<HD, THREADS>(kv, k_begin + 2 * KB, key_lo, key_end, wave);
    lds_barrier();
    int st = 0;
    for (int t0 = k_begin; t0 < key_end; t0 += KB, st ^= 1) {
        const bf16* stage = lds + st * L::STAGE;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
            const int tb = t0 + 32 * sb;
            if (sb % KW == ks && tb < my_end && tb + 32 > my_lo) {         // the same for the whole wavefront
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
            store_stretch<HD, THREADS>(lds + (st ^ 1) * L::STAGE, places, fetched);
            fetch_stretch<HD, THREADS>(kv, pages, places, fetched);
            pages = lookup_stretch<HD, THREADS>(kv, t0 + 3 * KB, key_lo, key_end, wave);
            lds_barrier();
        }
    }

    if (KW == 2) {
        // The two wavefronts of a tile have seen every other 32-key block each: the second hands
        // its maxima, sums and accumulators over through LDS (the stages are done with), the
        // first brings both to the common maximum and adds them.
        constexpr int PER_QT = 2 + DT * 4;                 // floats per lane and row tile
        float* hand = reinterpret_cast<float*>(lds) + tile * (QT * PER_QT * 64);
        static_assert(4 * QT * PER_QT * 64 * 4 <= L::BYTES, "the hand-over must fit into the stages");
        __syncthreads();                                   // everybody has read its last stage
        if (ks == 1) {
#pragma unroll
            for (int qt = 0; qt < QT; ++qt) {
                float* p = hand + qt * PER_QT * 64 + lane;
                p[0] = m[qt];
                p[64] = l[qt];
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int e = 0; e < 4; ++e) p[(2 + dt * 4 + e) * 64] = o[qt][dt][e];
            }
        }
        __syncthreads();
        if (ks == 1) return;
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
            const float* p = hand + qt * PER_QT * 64 + lane;
            const float m1 = p[0], l1 = p[64];
            const float mx = fmaxf(m[qt], m1);
            const float a0 = fast_exp2(m[qt] - mx), a1 = fast_exp2(m1 - mx);
            m[qt] = mx;
            l[qt] = l[qt] * a0 + l1 * a1;
            float ar0[4], ar1[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {                   // factors of O's row 4 g4 + e
                ar0[e] = __shfl(a0, g4 * 4 + e, 64);
                ar1[e] = __shfl(a1, g4 * 4 + e, 64);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int e = 0; e < 4; ++e) o[qt][dt][e] = o[qt][dt][e] * ar0[e] + p[(2 + dt * 4 + e) * 64] * ar1[e];
        }
    }

#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
        float lt = l[qt];
        lt += __shfl_xor(lt, 16, 64);
        lt += __shfl_xor(lt, 32, 64);
        if (SPLIT && runs > 1) {
            // this run's part of row `row`, head `head`: statistics from the lanes of the row's
            // first quarter, outputs unscaled (the join divides)
            if (g4 == 0 && qt * 16 + r < n_rows) {
                const size_t pidx = (static_cast<size_t>(first_w + qt * 16 + r) * n_q + head) * nsplit + z;
                part_ml[pidx * 2] = m[qt];
                part_ml[pidx * 2 + 1] = lt;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = qt * 16 + g4 * 4 + e;
                if (row >= n_rows) continue;
                const size_t pidx = (static_cast<size_t>(first_w + row) * n_q + head) * nsplit + z;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) part_o[pidx * HD + dt * 16 + r] = o[qt][dt][e];
            }
            continue;
        }
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

// With many items per workgroup, the workgroups take work items from a counter, heaviest first, until none is left: spans differ
// in the keys they see by the length of the context, and a grid with one workgroup per item
// leaves most of the chip idle while the few longest finish. queue[0] counts the items taken,
// queue[1] the workgroups that have left; both are zero before and after the kernel (the last
// workgroup to leave clears them), so the same two integers serve every launch on a stream.
// KW = 2: eight wavefronts, two per tile, each taking every other 32-key block: half the time
// for a work item, for batches with too few items to fill the chip.
template <int HD, int QT, int HPW, int KW, bool SPLIT>
__global__ __launch_bounds__(256 * KW) void attention_prefill_shared_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, const int* __restrict__ q_start, const int* __restrict__ ctx_len,
    const int* __restrict__ block_table, int max_blocks, int n_seq, int n_q, int n_kv, int page, float scale,
    int window, int spans, int* __restrict__ queue, int nsplit, int run, float* __restrict__ part_o,
    float* __restrict__ part_ml, DecodeBeside beside) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    __shared__ int next_item;
    bf16* lds = reinterpret_cast<bf16*>(lds_raw);
    if (static_cast<int>(blockIdx.x) < beside.blocks) {
        // one of the step's decode work items: the workgroup's first four wavefronts, the stages' LDS
        static_assert(decode_lds_floats(HD) * 4 <= StageLayout<HD>::BYTES, "the decode item's sums must fit into the stages");
        if (threadIdx.x >= DEC_WAVES * 64) return;
        const int b = blockIdx.x, per_seq = beside.head_tiles * beside.nsplit;
        decode_item<HD, true>(q, k_cache, v_cache, out, beside.part_o, beside.part_ml, q_start, ctx_len, block_table,
                              max_blocks, n_q, n_kv, page, scale, window, beside.split_len, beside.nsplit, b / per_seq,
                              (b % per_seq) / beside.nsplit, b % beside.nsplit, reinterpret_cast<float*>(lds_raw));
        return;
    }
    const int head_groups = n_q / HPW;
    const int n_items = spans * head_groups * (SPLIT ? nsplit : 1);
    if (queue == nullptr) {
        // Few items per workgroup: a fixed order, to and fro over the workgroups (the items are
        // sorted, heaviest first: workgroup w of G takes w, 2 G - 1 - w, 2 G + w, ..), so that every
        // workgroup's items add up to about the same number of keys. The counter's answer is a trip
        // to memory per item, with two barriers around it, and costs more than its evening-out
        // wins until a workgroup has several items to take.
        const int G = static_cast<int>(gridDim.x) - beside.blocks, w = static_cast<int>(blockIdx.x) - beside.blocks;
        for (int round = 0; round * G < n_items; ++round) {
            const int item = round * G + ((round & 1) ? G - 1 - w : w);
            if (item >= n_items) continue;                 // (only in the last round)
            if (round > 0) __syncthreads();                // everybody is done with the last item's LDS
            const int whole = SPLIT ? item / nsplit : item;
            prefill_item<HD, QT, HPW, KW, SPLIT>(whole / head_groups, whole % head_groups, SPLIT ? item % nsplit : 0, nsplit,
                                                 run, part_o, part_ml, lds, q, k_cache, v_cache, out, q_start, ctx_len,
                                                 block_table, max_blocks, n_seq, n_q, n_kv, page, scale, window);
        }
        return;
    }
    for (;;) {
        __syncthreads();                                   // everybody is done with the last item's LDS
        if (threadIdx.x == 0) next_item = atomicAdd(queue, 1);
        __syncthreads();
        const int item = __builtin_amdgcn_readfirstlane(next_item);
        if (item >= n_items) break;                        // the counter only grows: every workgroup gets here
        const int whole = SPLIT ? item / nsplit : item;     // (an item's runs are neighbours in the queue)
        prefill_item<HD, QT, HPW, KW, SPLIT>(whole / head_groups, whole % head_groups, SPLIT ? item % nsplit : 0, nsplit,
                                             run, part_o, part_ml, lds, q, k_cache, v_cache, out, q_start, ctx_len,
                                             block_table, max_blocks, n_seq, n_q, n_kv, page, scale, window);
    }
    if (threadIdx.x == 0) {
        // whoever leaves last has seen every other workgroup take its final number: nobody touches
        // the counter any more
        if (atomicAdd(queue + 1, 1) == static_cast<int>(gridDim.x) - beside.blocks - 1) {
            atomicExch(queue, 0);
            atomicExch(queue + 1, 0);
        }
    }
}

constexpr long kSplitBelowItems = 768;

static int heads_per_workgroup(int n_q, int n_kv) {
    const int G = n_q / n_kv;
    return G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);
}

// Rows per work item: 32 per row group (measured: 64 are no faster at any length, and leave
// fewer items to spread over the chip), times the row groups of a workgroup. The caller may halve
// them (16 per row group) where a step has few items: an item's time is set by its walk over the
// keys, a stretch after the other, and a stretch of 16 rows is shorter than one of 32. Measured on
// whole prompts (us, 32 / 16 rows; 32 query and 8 kv heads): heads of 64, 256 tokens 9.6 / 7.2, 1,024
// 20.7 / 17.1, 2,048 40.0 / 39.1, 3,072 80.8 / 73.6, 4,096 96.8 / 121; heads of 128, 512 tokens 19.0 /
// 15.4, 1,024 30.0 / 29.0, 2,048 57.8 / 71.7: half the rows win until the items of 32 rows number
// one workgroup less per compute unit than LDS lets it hold (four with heads of 64, two with 128).
int prefill_shared_rows(int hd, int n_q, int n_kv) {
    if ((hd != 64 && hd != 128) || n_kv <= 0 || n_q % n_kv != 0) return 0;
    return 32 * (4 / heads_per_workgroup(n_q, n_kv));
}

template <int HD, int QT, int HPW, int KW, bool SPLIT>
static int launch_shared(const bf16* q, const bf16* kc, const bf16* vc, bf16* out, const int* q_start,
                         const int* ctx_len, const int* table, int max_blocks, int n_seq, int n_q, int n_kv, int page,
                         float scale, int window, int items, int* queue, int nsplit, int run, float* part_o,
                         float* part_ml, const DecodeBeside& beside, hipStream_t stream) {
    constexpr int LDS = StageLayout<HD>::BYTES;
    auto kernel = attention_prefill_shared_kernel<HD, QT, HPW, KW, SPLIT>;
    static bool attr_set = false;                      // per instantiation
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (e != hipSuccess) return static_cast<int>(e);
        attr_set = true;
    }
    static int resident = 0;                           // workgroups the chip holds at a time
    if (resident == 0) {
        int dev = 0, cus = 0, per_cu = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        if (e == hipSuccess)
            e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel), 256 * KW,
                                                             LDS);
        if (e != hipSuccess) return static_cast<int>(e);
        resident = cus * (per_cu > 0 ? per_cu : 1);
    }
    const int n_items = items * (n_q / HPW) * (SPLIT ? nsplit : 1);
    // (measured, 32/8 heads of 64: 2,048 tokens, 512 items on 256 workgroups, 40.8 us in the fixed order
    // against 47.5 with the counter; 4,096 tokens, 1,024 items on 768, 101.8 against 115.6; 8,192 tokens,
    // 2,048 items on 768, 359 against 340)
    int* counter = n_items <= 2 * resident ? nullptr : queue;
    hipLaunchKernelGGL(kernel, dim3(beside.blocks + (n_items < resident ? n_items : resident)), dim3(256 * KW), LDS, stream,
                       q, kc, vc, out, q_start, ctx_len, table, max_blocks, n_seq, n_q, n_kv, page, scale, window, items,
                       counter, nsplit, run, part_o, part_ml, beside);
    return launch_status();
}

int launch_prefill_shared(const bf16* q, const bf16* kc, const bf16* vc, bf16* out, const int* q_start,
                          const int* ctx_len, const int* table, int max_blocks, int n_seq, int n_q, int n_kv, int hd,
                          int page, float scale, int window, int items, int rows_per_item, int* queue, int nsplit,
                          int run, float* part_o, float* part_ml, int key_waves, const DecodeBeside& beside,
                          hipStream_t stream) {
    if (queue == nullptr) return kErrBadArgument;
    if (nsplit < 1 || (nsplit > 1 && (run < 1 || part_o == nullptr || part_ml == nullptr))) return kErrBadArgument;
    const int hpw = heads_per_workgroup(n_q, n_kv);
    const int rows = rows_per_item / (4 / hpw);            // per row group
    // Two wavefronts per tile while the items are too few to keep three workgroups of four
    // wavefronts on every compute unit: then an item's length, not the chip, sets the time.
    int kw = static_cast<long>(items) * (n_q / hpw) <= kSplitBelowItems ? 2 : 1;
    if (key_waves == 1 || key_waves == 2) kw = key_waves;  // (forced by the caller: tests, measurements)
#define LLME_SHARED_ARGS q, kc, vc, out, q_start, ctx_len, table, max_blocks, n_seq, n_q, n_kv, page, scale, window, \
                         items, queue, nsplit, run, part_o, part_ml, beside, stream
#define LLME_SHARED(HD, QT, HPW)                                                       \
    if (hd == HD && rows == 16 * QT && hpw == HPW) {                                   \
        if (nsplit > 1)                                                                \
            return kw == 2 ? launch_shared<HD, QT, HPW, 2, true>(LLME_SHARED_ARGS)     \
                           : launch_shared<HD, QT, HPW, 1, true>(LLME_SHARED_ARGS);    \
        return kw == 2 ? launch_shared<HD, QT, HPW, 2, false>(LLME_SHARED_ARGS)        \
                       : launch_shared<HD, QT, HPW, 1, false>(LLME_SHARED_ARGS);       \
    }
    LLME_SHARED(64, 2, 4) LLME_SHARED(64, 2, 2) LLME_SHARED(64, 2, 1)
    LLME_SHARED(128, 2, 4) LLME_SHARED(128, 2, 2) LLME_SHARED(128, 2, 1)
    LLME_SHARED(64, 1, 4) LLME_SHARED(64, 1, 2) LLME_SHARED(64, 1, 1)
    LLME_SHARED(128, 1, 4) LLME_SHARED(128, 1, 2) LLME_SHARED(128, 1, 1)
#undef LLME_SHARED
#undef LLME_SHARED_ARGS
    return kErrUnsupported;
}

}  // namespace llme

LLME_LOAD_ENTRY(attention_prefill)
