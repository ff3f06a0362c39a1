// Into how many splits a step of single decoded tokens cuts its keys, decided on the host from the
// requests' lengths. The reference walks one sequence's keys in one loop (src/kernels.cpp:413-474) and
// has nothing of the kind; this belongs to how the decode attention kernel is launched here.
//
// The kernel has a workgroup per (split, request, tile), a tile being a kv head with up to 16 of its
// query heads, the tile counted fastest. The chip deals workgroups to its compute units in turn, so
// piece q = request + requests x split (of every tile) lands on place q mod P, P = units / tiles, and
// pieces that share a place share its path to memory: a place's time goes with the keys it is given.
// The step's time is then the larger of (all keys' bytes at the rate the chip streams them when they
// are shared out evenly) and (the busiest place's keys at a place's own rate, plus a little per piece).
// More splits even the places out, but cost a join kernel, the rotation kernel where the single split
// would have had the decode kernel that rotates, and a little each.
//
// Fitted to decode steps at the 1B sizes (8 tiles, heads of 64, 256 units), 17 to 72 requests at
// contexts of 2,048 and 8,192, all of one length: the kernel times it gives are within 10 % of the
// measured ones, and it picks the measured best or one within 2 % of it. With requests of different
// lengths and more workgroups than units, the busiest place of the uncut step is often one long
// request alone (the scheduler puts long and short together): it finishes on a chip that is draining,
// faster per key than a place that shares the chip to the end (lone_ns; measured 8.3 against 9.5), and
// cutting such a step lost 6 to 14 % where the estimate without this promised 10 to 19 %.
#include <algorithm>
#include <cstdint>
#include <vector>

#include "host_api.h"

extern "C" {

// lens [S]: the keys each request sees in this step, in the step's order. plan_len: the length the
// splits are laid out for (at least the longest; a recorded step is replayed while its requests grow).
// tiles: workgroups per request and split; units: compute units. first: the number of splits that stands
// unless another promises more (1: the keys whole); most: splits at most (>= first).
// tbs: TB/s of the even stream; key_ns: ns a place needs per key of a head of 64 (scaled by the head
// size), lone_ns: the same for a place's only piece of an uncut step that has more workgroups than units;
// piece_us: per piece on a place; apart_us: what any cut costs; each_us: what every split costs;
// gain: a cut must promise this fraction. Returns the number of splits (>= 1), or an error code.
int llme_decode_cut(const int* lens, int S, int tiles, int units, int head_dim, long plan_len, int first, int most,
                    double tbs, double key_ns, double lone_ns, double piece_us, double apart_us, double each_us,
                    double gain) {
    if (!lens || S <= 0 || tiles <= 0 || units <= 0 || head_dim <= 0 || plan_len <= 0 || !(tbs > 0.0) || !(key_ns > 0.0) ||
        !(lone_ns > 0.0) || first < 1 || first > 64)
        return LLME_HOST_BAD_ARGUMENT;
    long longest = 0;
    double total = 0.0;
    for (int s = 0; s < S; ++s) {
        if (lens[s] < 0) return LLME_HOST_BAD_ARGUMENT;
        longest = std::max<long>(longest, lens[s]);
        total += lens[s];
    }
    if (plan_len < longest) plan_len = longest;
    const int places = std::max(1, units / tiles);
    const double even_us = total * tiles * head_dim * 4.0 / (tbs * 1e6);
    const double per_key_us = key_ns * head_dim / 64.0 * 1e-3, lone_key_us = lone_ns * head_dim / 64.0 * 1e-3;
    const bool crowded = static_cast<long>(S) * tiles > units;
    std::vector<double> keys(static_cast<size_t>(places));
    std::vector<int> pieces(static_cast<size_t>(places));
    auto estimate = [&](int n) {
        const long split_len = ((plan_len + n - 1) / n + 31) / 32 * 32;
        std::fill(keys.begin(), keys.end(), 0.0);
        std::fill(pieces.begin(), pieces.end(), 0);
        for (int split = 0; split < n; ++split)
            for (int s = 0; s < S; ++s) {
                const long left = lens[s] - split * split_len;
                if (left <= 0) continue;
                const size_t place = static_cast<size_t>((s + static_cast<long>(S) * split) % places);
                keys[place] += static_cast<double>(std::min(left, split_len));
                ++pieces[place];
            }
        double busiest = 0.0;
        for (size_t p = 0; p < keys.size(); ++p) {
            const bool lone = n == 1 && crowded && pieces[p] == 1;
            busiest = std::max(busiest, keys[p] * (lone ? lone_key_us : per_key_us) + pieces[p] * piece_us);
        }
        return std::max(even_us, busiest) + (n > 1 ? apart_us + each_us * n : 0.0);
    };
    int best = first;
    double best_us = estimate(first) * (1.0 - gain);
    for (int n = first + 1; n <= most && n <= 64; ++n) {
        if (static_cast<long>(S) * tiles * n > 10L * units) break;        // (measured up to 9 workgroups a unit)
        if (plan_len / n < 256) break;                                    // (a split of fewer keys is all start-up)
        const double us = estimate(n);
        if (us < best_us) {
            best = n;
            best_us = us;
        }
    }
    return best;
}

}  // extern "C"
