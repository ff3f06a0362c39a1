// The join of the decode kernel's key splits and the output projection behind it, as one kernel
// for a step of up to 16 decoded tokens:
//   o[m, h, :]   = sum_i weight_i part_o[m, h, i, :]        (the join, as attention_mfma.hip's join kernel)
//   out[m, n]   += sum_k bf16(o[m, k]) w[n, k]              (o_proj + residual, src/model.cpp's attention block)
// Apart, each is a few microseconds of launch and trips to memory around very little work (the
// joined rows are 32 KB at 8 requests of the 1B sizes, the projection's matrix 8 MB): at 8 requests
// and a context of 4,096 the join took 4.7 us and the projection 4.4 us a layer.
//
// A workgroup takes a stretch of k (the dims of a few heads, at most 256) and a block of output
// columns: it asks for its weights first, joins its heads' splits for all rows meanwhile (every
// workgroup of the same heads does the same join: the parts are small and come from L2), rounds
// the joined rows to bfloat16 into LDS as the join kernel rounds them into memory, multiplies,
// and adds its part of the sum over k into the 32-bit output with atomics, like the projection
// that is cut over k (the order of these additions is not fixed).
// Weights: blocked [N / 16][K / 32] blocks of 1 KB in the matrix instruction's operand order.
#include "attention_tiles.h"

namespace llme {

constexpr int JP_WAVES = 4;
constexpr int JP_MAX_KP = 256;                       // dims of a workgroup's heads at most
constexpr int JP_KB = JP_MAX_KP / 32;                // 32-wide k blocks of a stretch at most
constexpr int JP_XS = JP_MAX_KP + 8;                 // padded row of the joined tile (elements)
constexpr int JP_MAX_SPLITS = 64;
constexpr int JP_READ_ONCE = 2;                      // a buffer load's cache policy: the non-temporal bit

// grid: parts x column blocks, the part fastest (workgroups go to the chip's dies in turn: with 8
// parts each die joins one part's heads). part p: heads p hpk .. p hpk + hpk - 1; column block c:
// tiles c JP_WAVES tpw .., wavefront w taking tpw of them one after the other.
// Every index below is taken apart by shifts: hpk, the padded number d4p of 4-dim pieces of a head
// and the number of shares of a row's splits are powers of two (2^lg_hpk, 2^lg_d4p, 2^lg_g). Divisions
// by sizes only known at run time took longer than the trips to memory they stood in front of.
struct JoinShape {
    int lg_hpk, lg_d4p, lg_g;
    int nb;                      // batches of splits per unit
    int n_seq;                   // (unit, batch) pairs per thread, in order: batch b of unit tid + 256 it
    int first_it[4], first_b[4]; // the first four of them
};

// LP: lanes that share a (row, head)'s statistics: 4 (a split each; up to 4 splits, 64 pairs to a pass
// of the workgroup) or 16 (up to 4 splits each; 16 pairs to a pass). BW: splits of a batch of partial
// outputs (2, 4 or 8: the least that holds a unit's splits, so that few loads are asked for in vain).
// SA passes of statistics and UA batches are asked for in front of the weights; what is left is
// asked for behind them (many rows of many heads).
template <int LP, int BW>
__global__ __launch_bounds__(JP_WAVES * 64) void attention_join_project_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const bf16* __restrict__ w,
    float* __restrict__ out, int M, int n_q, int hd, int nsplit, int N, int parts, int tpw, JoinShape js) {
    __shared__ __align__(16) bf16 xs[16 * JP_XS];                       // joined rows, bfloat16
    // [(row, head)][split]: 4,096 in all (the entry point checks); behind them the shares of the joined rows
    // where a row's splits are dealt out over several threads: [share][(row, head, piece)][4], at most 256 units
    __shared__ __align__(16) float wts[16 * 16 * JP_MAX_SPLITS / 4 + JP_WAVES * 64 * 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, q4 = lane >> 4;
    constexpr int SPL = LP == 4 ? 1 : 4;                                // splits a lane holds statistics of
    constexpr int PASS = JP_WAVES * 64 / LP;                            // (row, head) pairs of a pass
    constexpr int SA = LP == 4 ? 1 : 2, UA = BW == 8 ? 2 : 4;
    const int part = blockIdx.x % parts, cblock = blockIdx.x / parts;
    const int K = n_q * hd;
    const int hpk = 1 << js.lg_hpk;
    const int head0 = part * hpk;
    const int heads = n_q - head0 < hpk ? n_q - head0 : hpk;            // heads of this part that exist
    const int nkb = heads * hd / 32;                                    // their dims in 32-wide blocks (whole ones)
    const int kb0 = head0 * hd / 32;                                    // first k block
    const int tiles = N / 16;

    const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<bf16*>(w), 0, static_cast<unsigned>(static_cast<size_t>(N) * K * 2), 0x00020000);
    constexpr unsigned kNowhere = 0xFFFFFFF0u;
    bf16x8 fw[2][JP_KB];
    auto load_w = [&](bf16x8 (&f)[JP_KB], int tile) {
        const unsigned base = (static_cast<unsigned>(tile) * static_cast<unsigned>(K / 32) + kb0) * 1024u + lane * 16u;
#pragma unroll
        for (int kb = 0; kb < JP_KB; ++kb) {
            const unsigned in = 0u - static_cast<unsigned>(tile < tiles && kb < nkb);
            const unsigned off = ((base + kb * 1024u) & in) | (kNowhere & ~in);
            f[kb] = __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, off, 0, JP_READ_ONCE));
        }
    };
    const int tile0 = (cblock * JP_WAVES + wave) * tpw;

    // Loads come back in the order they were asked for, and the weights come from far: so the
    // splits' statistics and the first partial outputs are asked for first, then the weights, and
    // all three trips to memory run at the same time. (Loads of places that do not exist are loads
    // of a place that does, with weight 0: every path then has the same loads in flight.)
    //
    // The splits' statistics: LP lanes per (row, head), lane j of them holding splits j, j + 16, j + 32,
    // j + 48 (LP 16) or split j (LP 4); pair p = row hpk + head of the part.
    const int pairs = M << js.lg_hpk;
    const int sl = lane & (LP - 1);
    struct Stats {
        float2 ml[SPL];
    };
    auto ask_stats = [&](int p0, Stats& st) {
        const int p = p0 + wave * (64 / LP) + lane / LP;
        const int m = p >> js.lg_hpk, hh = p & (hpk - 1);
        const bool p_ok = m < M && hh < heads;
        const unsigned base = static_cast<unsigned>((p_ok ? m : 0) * n_q + head0 + (p_ok ? hh : 0)) * nsplit;
#pragma unroll
        for (int u = 0; u < SPL; ++u) {
            const int i = sl + 16 * u;
            st.ml[u] = *reinterpret_cast<const float2*>(part_ml + (base + (i < nsplit ? i : 0)) * 2);
        }
    };
    // the sums in the order of the join kernel's 64-lane reduction (lanes 32 apart first, then 16, 8, ..)
    auto take_stats = [&](int p0, const Stats& st) {
        const int p = p0 + wave * (64 / LP) + lane / LP;
        const int m = p >> js.lg_hpk, hh = p & (hpk - 1);
        const bool p_ok = m < M && hh < heads;
        float mi[SPL], li[SPL];
#pragma unroll
        for (int u = 0; u < SPL; ++u) {
            const bool ok = p_ok && sl + 16 * u < nsplit;
            mi[u] = ok ? st.ml[u].x : -INFINITY;
            li[u] = ok ? st.ml[u].y : 0.f;
        }
        float mx = SPL == 4 ? fmaxf(fmaxf(mi[0], mi[SPL / 2]), fmaxf(mi[SPL / 4], mi[SPL - 1])) : mi[0];
#pragma unroll
        for (int off = LP / 2; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        float f[SPL];
#pragma unroll
        for (int u = 0; u < SPL; ++u) f[u] = (mi[u] <= kNoMax) ? 0.f : exp2f(mi[u] - mx);
        // (each product rounded by itself, as where a lane holds one split)
        float total = SPL == 4 ? (__fmul_rn(f[0], li[0]) + __fmul_rn(f[SPL / 2], li[SPL / 2])) +
                                     (__fmul_rn(f[SPL / 4], li[SPL / 4]) + __fmul_rn(f[SPL - 1], li[SPL - 1]))
                               : __fmul_rn(f[0], li[0]);
#pragma unroll
        for (int off = LP / 2; off > 0; off >>= 1) total += __shfl_xor(total, off, 64);
        if (p_ok) {
#pragma unroll
            for (int u = 0; u < SPL; ++u)
                if (sl + 16 * u < nsplit) wts[p * nsplit + sl + 16 * u] = f[u] / total;
        }
    };
    // The joined rows: a unit is four neighbouring dims (piece dc of its head) of a (row, head) and one
    // of 2^lg_g shares of its splits (several shares where the rows are few and the splits many, so
    // that every thread has loads to ask for); unit number = (((row 2^lg_g + share) hpk + head) d4p + dc.
    // A unit's splits are taken BW at a time: batch b of unit tid + 256 it.
    const int d4 = hd / 4, d4p = 1 << js.lg_d4p;
    const int groups = 1 << js.lg_g;
    const int spg = (nsplit + groups - 1) >> js.lg_g;                   // splits of a share
    struct Unit {
        bool ok;
        int pair, share, dc, i_end;
        unsigned src;                                                    // of split 0, in floats
    };
    auto unit_of = [&](int it) {
        const int u = tid + JP_WAVES * 64 * it;
        Unit x;
        x.dc = u & (d4p - 1);
        const int hh = (u >> js.lg_d4p) & (hpk - 1);
        x.share = (u >> (js.lg_d4p + js.lg_hpk)) & (groups - 1);
        const int m = u >> (js.lg_d4p + js.lg_hpk + js.lg_g);
        x.ok = m < M && hh < heads && x.dc < d4;
        x.pair = x.ok ? (m << js.lg_hpk) + hh : 0;
        x.src = (static_cast<unsigned>((x.ok ? m : 0) * n_q + head0 + (x.ok ? hh : 0)) * nsplit) * hd + (x.ok ? x.dc : 0) * 4;
        x.i_end = (x.share + 1) * spg < nsplit ? (x.share + 1) * spg : nsplit;
        return x;
    };
    struct Batch {
        float4 v[BW];
    };
    auto ask_batch = [&](const Unit& x, int b, Batch& bt) {
#pragma unroll
        for (int j = 0; j < BW; ++j) {
            const int i = x.share * spg + BW * b + j;
            bt.v[j] = *reinterpret_cast<const float4*>(part_o + x.src + static_cast<unsigned>(i < x.i_end ? i : 0) * hd);
        }
    };
    float4 acc = float4{0.f, 0.f, 0.f, 0.f};
    float* shares = wts + 16 * 16 * JP_MAX_SPLITS / 4;
    auto store_row = [&](int pair, int dc, const float4& v) {
        bf16x4 bv;
        bv[0] = static_cast<__bf16>(v.x); bv[1] = static_cast<__bf16>(v.y);
        bv[2] = static_cast<__bf16>(v.z); bv[3] = static_cast<__bf16>(v.w);
        *reinterpret_cast<bf16x4*>(xs + (pair >> js.lg_hpk) * JP_XS + (pair & (hpk - 1)) * hd + dc * 4) = bv;
    };
    auto take_batch = [&](const Unit& x, int b, const Batch& bt) {
        if (!x.ok) return;
        if (b == 0) acc = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < BW; ++j) {
            const int i = x.share * spg + BW * b + j;
            const float wt = i < x.i_end ? wts[x.pair * nsplit + i] : 0.f;
            acc.x += wt * bt.v[j].x; acc.y += wt * bt.v[j].y; acc.z += wt * bt.v[j].z; acc.w += wt * bt.v[j].w;
        }
        if (b != js.nb - 1) return;
        if (groups > 1)
            *reinterpret_cast<float4*>(shares + (((x.share << js.lg_hpk) * M + x.pair) << js.lg_d4p | x.dc) * 4) = acc;
        else
            store_row(x.pair, x.dc, acc);
    };

    Stats st[SA];
    Batch bt[UA];
    Unit un[UA];
#pragma unroll
    for (int a = 0; a < SA; ++a) ask_stats(a * PASS, st[a]);
#pragma unroll
    for (int a = 0; a < UA; ++a) {
        un[a] = unit_of(js.first_it[a]);
        ask_batch(un[a], js.first_b[a], bt[a]);
    }
    __builtin_amdgcn_sched_barrier(0);
    load_w(fw[0], tile0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int a = 0; a < SA; ++a) take_stats(a * PASS, st[a]);
    for (int p0 = SA * PASS; p0 < pairs; p0 += PASS) {
        Stats later;
        ask_stats(p0, later);
        take_stats(p0, later);
    }
    lds_barrier();                                                      // (LDS only: the weights stay in flight)
#pragma unroll
    for (int a = 0; a < UA; ++a)
        if (a < js.n_seq) take_batch(un[a], js.first_b[a], bt[a]);
    {
        int it = js.first_it[UA - 1], b = js.first_b[UA - 1];
        for (int sq = UA; sq < js.n_seq; ++sq) {
            if (++b == js.nb) {
                b = 0;
                ++it;
            }
            const Unit x = unit_of(it);
            Batch later;
            ask_batch(x, b, later);
            take_batch(x, b, later);
        }
    }
    if (groups > 1) {
        // the shares of a unit, added in the order of the splits
        lds_barrier();
        const int n_out = (M << js.lg_hpk) << js.lg_d4p;
        for (int o = tid; o < n_out; o += JP_WAVES * 64) {
            float4 sum = *reinterpret_cast<const float4*>(shares + static_cast<size_t>(o) * 4);
            for (int g = 1; g < groups; ++g) {
                const float4 sh = *reinterpret_cast<const float4*>(shares + (static_cast<size_t>(g) * n_out + o) * 4);
                sum.x += sh.x; sum.y += sh.y; sum.z += sh.z; sum.w += sh.w;
            }
            const int pair = o >> js.lg_d4p, dc = o & (d4p - 1);
            if ((pair & (hpk - 1)) < heads && dc < d4) store_row(pair, dc, sum);
        }
    }
    lds_barrier();

    // ---- the products: rows m >= M of the tile are whatever LDS holds, and are never added ----
    const bf16* xlane = xs + r * JP_XS + q4 * 8;
    auto multiply = [&](const bf16x8 (&f)[JP_KB], int tile) {
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < JP_KB; ++kb) {
            if (kb < nkb) {
                const bf16x8 fx = *reinterpret_cast<const bf16x8*>(xlane + kb * 32);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f[kb], fx, acc, 0, 0, 0);
            }
        }
        // lane l holds row m = l % 16, columns 16 tile + 4 (l / 16) + e
        if (tile < tiles && r < M) {
            float* op = out + static_cast<size_t>(r) * N + tile * 16 + q4 * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) atomicAdd(op + e, acc[e]);
        }
    };
    // (two sets of weights in turn, written out: a set chosen by a running index would live in memory)
    for (int j = 0; j < tpw; j += 2) {
        if (j + 1 < tpw) load_w(fw[1], tile0 + j + 1);
        multiply(fw[0], tile0 + j);
        if (j + 1 < tpw) {
            if (j + 2 < tpw) load_w(fw[0], tile0 + j + 2);
            multiply(fw[1], tile0 + j + 1);
        }
    }
}

}  // namespace llme

using namespace llme;

// How many heads a workgroup joins: the largest power of two whose dims fit 256 and are whole 32-wide
// blocks of k; 0 if there is none.
static int heads_per_part_log2(int hd) {
    int best = -1;
    for (int lg = 0; (hd << lg) <= JP_MAX_KP; ++lg)
        if ((hd << lg) % 32 == 0) best = lg;
    return best;
}
static int ceil_log2(int v) {
    int lg = 0;
    while ((1 << lg) < v) ++lg;
    return lg;
}

// 1 if llme_attention_join_project takes these sizes.
extern "C" int llme_attention_join_project_supported(int M, int n_q, int hd, int nsplit, int N) {
    if (M <= 0 || M > 16 || n_q <= 0 || hd <= 0 || hd % 4 != 0 || nsplit < 1 || nsplit > JP_MAX_SPLITS) return 0;
    if (N <= 0 || N % 16 != 0 || (static_cast<long long>(n_q) * hd) % 32 != 0) return 0;
    if (static_cast<long long>(N) * n_q * hd * 2 >= (1ll << 32)) return 0;       // a 32-bit offset into the matrix
    if (static_cast<long long>(M) * n_q * nsplit * hd >= (1ll << 30)) return 0;  // and into the parts
    const int lg_hpk = heads_per_part_log2(hd);
    if (lg_hpk < 0) return 0;
    return (M << lg_hpk) * nsplit <= 16 * 16 * JP_MAX_SPLITS / 4 ? 1 : 0;       // the splits' weights fit their LDS
}

// 1 where the one kernel is faster than the join kernel and the projection apart (0 where it is not,
// or where the sizes are not taken). Measured in decode steps at a context of 2,048 to 16,384 (ms a step,
// apart / together): 1B sizes, 1 row 0.755 / 0.716, 8 rows 0.942 / 0.919, 16 rows 1.050 / 1.036; 3B sizes
// (the projection 19 MB, three tiles per wavefront), 1 row 1.83 / 1.75, 8 rows 2.49 / 2.47, 16 rows 2.92 /
// 2.98; 8B sizes (34 MB, four tiles), 1 row 3.20 / 3.10, 4 rows 3.37 / 3.30, 8 rows 4.00 / 4.00, 16 rows
// 4.84 / 4.99: with many rows every workgroup repeats a longer join, and a wavefront with several
// tiles streams its weights one tile ahead only.
extern "C" int llme_attention_join_project_pays(int M, int n_q, int hd, int nsplit, int N) {
    if (!llme_attention_join_project_supported(M, n_q, hd, nsplit, N) || nsplit < 2) return 0;
    const int parts = (n_q + (1 << heads_per_part_log2(hd)) - 1) >> heads_per_part_log2(hd);
    const long long units = static_cast<long long>(N / 16) * parts;          // (tile, stretch of k) pairs
    return (M <= 8 || units <= static_cast<long long>(compute_units()) * JP_WAVES) ? 1 : 0;
}

// part_o [M, n_q, nsplit, hd], part_ml [M, n_q, nsplit, 2] float32: what the decode kernel leaves for
// requests 0 .. M - 1 that bring one token each (row m of the batch is request m); w: the blocked
// output projection [N, n_q hd] bfloat16; out [M, N] float32, added to.
extern "C" int llme_attention_join_project(const float* part_o, const float* part_ml, const void* w, float* out, int M,
                                           int n_q, int hd, int nsplit, int N, hipStream_t stream) {
    if (!part_o || !part_ml || !w || !out) return kErrBadArgument;
    if (!llme_attention_join_project_supported(M, n_q, hd, nsplit, N)) return kErrUnsupported;
    if (reinterpret_cast<uintptr_t>(part_o) % 16 != 0 || reinterpret_cast<uintptr_t>(part_ml) % 8 != 0 ||
        reinterpret_cast<uintptr_t>(w) % 16 != 0)
        return kErrUnsupported;
    JoinShape js;
    js.lg_hpk = heads_per_part_log2(hd);
    js.lg_d4p = ceil_log2(hd / 4);
    const int hpk = 1 << js.lg_hpk;
    const int parts = (n_q + hpk - 1) / hpk;
    const int tiles = N / 16;
    // about one workgroup per compute unit: tiles per wavefront so that parts x column blocks come to that
    const int cus = compute_units();
    int tpw = static_cast<int>((static_cast<long long>(tiles) * parts + static_cast<long long>(cus) * JP_WAVES - 1) /
                               (static_cast<long long>(cus) * JP_WAVES));
    if (tpw < 1) tpw = 1;
    const int cblocks = (tiles + JP_WAVES * tpw - 1) / (JP_WAVES * tpw);
    // few rows with many splits: a (row, head)'s splits are dealt out over 2 or 4 threads
    const int units1 = (M << js.lg_hpk) << js.lg_d4p;
    js.lg_g = 0;
    while (js.lg_g < 2 && (units1 << (js.lg_g + 1)) <= JP_WAVES * 64 && nsplit >= (8 << js.lg_g)) ++js.lg_g;
    const int spg = (nsplit + (1 << js.lg_g) - 1) >> js.lg_g;
    const int bw = spg <= 2 ? 2 : spg <= 4 ? 4 : 8;
    js.nb = (spg + bw - 1) / bw;
    js.n_seq = (((units1 << js.lg_g) + JP_WAVES * 64 - 1) / (JP_WAVES * 64)) * js.nb;
    for (int a = 0; a < 4; ++a) {
        js.first_it[a] = a / js.nb;
        js.first_b[a] = a % js.nb;
    }
#define LLME_JOIN_PROJECT(LP, BW)                                                                                      \
    hipLaunchKernelGGL((attention_join_project_kernel<LP, BW>), dim3(parts * cblocks), dim3(JP_WAVES * 64), 0, stream, \
                       part_o, part_ml, static_cast<const bf16*>(w), out, M, n_q, hd, nsplit, N, parts, tpw, js)
    if (nsplit <= 4) {
        if (bw == 2) LLME_JOIN_PROJECT(4, 2);
        else LLME_JOIN_PROJECT(4, 4);
    } else {
        if (bw == 8) LLME_JOIN_PROJECT(16, 8);
        else if (bw == 4) LLME_JOIN_PROJECT(16, 4);
        else LLME_JOIN_PROJECT(16, 2);
    }
#undef LLME_JOIN_PROJECT
    return launch_status();
}

LLME_LOAD_ENTRY(attention_join_project)
