// A driver for the host runtime alone (csrc/host/*.cpp), meant to be built with the address and
// undefined-behaviour sanitizers and run on the CPU: random orders of requests through the cache
// manager, and random workloads through the scheduler with a stand-in for the model (random
// tokens), with every buffer that the runtime writes into sized exactly, so that a write one
// element too far is seen. It checks what the Python tests check (no page lost, held twice or
// freed twice; every request finishes; all pages come back) and prints "ok".
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

extern "C" {
void* llme_cm_create(int n_groups, const int* is_window, const int* window, const int* num_pages, int page_size,
                     int max_requests);
void llme_cm_destroy(void* h);
int llme_cm_admit(void* h, int64_t key);
int llme_cm_is_live(void* h, int64_t key);
long llme_cm_length(void* h, int64_t key);
int llme_cm_free_slots(void* h);
int llme_cm_reserve_batch(void* h, int n, const int64_t* keys, const long* n_new);
int llme_cm_commit(void* h, int64_t key, long n_new);
int llme_cm_release(void* h, int64_t key);
int llme_cm_table_len(void* h, int64_t key, int group);
int llme_cm_free_pages(void* h, int group);
int llme_cm_num_pages(void* h, int group);
int llme_cm_check(void* h);
int llme_cm_decode_begin(void* h, int S, const int64_t* keys, int* lengths, long max_length);
int llme_cm_commit_batch(void* h, int S, const int64_t* keys, long n_new);
int llme_cm_fill_decode(void* h, int S, const int64_t* keys, int width, int* lengths, int* slots, int* tables,
                        int* done, int64_t* serials);
int llme_cm_lengths(void* h, int S, const int64_t* keys, long* out);
long llme_cm_fill_step(void* h, int S, const int64_t* keys, const int* new_lens, int width, int* positions,
                       int* seq_idx, int* q_start, int* ctx_len, int* slots, int* tables);
void* llme_sched_create(void* cache_manager, int max_concurrent, long budget);
void llme_sched_destroy(void* h);
int llme_sched_set_decode_round(void* h, int requests);
int llme_sched_set_row_round(void* h, long rows, long over);
int llme_decode_cut(const int* lens, int S, int tiles, int units, int head_dim, long plan_len, int first, int most,
                    double tbs, double key_ns, double lone_ns, double piece_us, double apart_us, double each_us,
                    double gain);
long llme_sched_enqueue(void* h, const int* prompt, long n, long max_new_tokens);
int llme_sched_idle(void* h);
int llme_sched_plan(void* h, int* n_admitted, int* admitted_slots, int64_t* entry_seq, int* entry_count, int* entry_want,
                    long* entry_gen, int* tokens, long tokens_cap);
int llme_sched_complete(void* h, const int* sampled, int n, const int* eos, int n_eos);
void llme_sched_abort(void* h);
int llme_sched_fail(void* h);
int llme_sched_num_results(void* h);
int llme_sched_result_info(void* h, int i, int64_t* seq_id, long* prompt_len, long* n_tokens, int* reason);
int llme_sched_result_tokens(void* h, int i, int* out);
int llme_plain_llama_forward(const int32_t* sizes, const double* rope, float eps, const float* embed,
                             const float* final_norm, const float* head, const float* const* layer_weights,
                             const int32_t* tokens, const int32_t* positions, int T, float* logits);
}

#define REQUIRE(cond)                                                              \
    do {                                                                           \
        if (!(cond)) {                                                             \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);                  \
            std::exit(1);                                                          \
        }                                                                          \
    } while (0)

static std::mt19937 rng(12345);      // (main reseeds it from its second argument)
static int pick(int lo, int hi) { return std::uniform_int_distribution<int>(lo, hi)(rng); }

// ---- the cache manager under random orders of requests ----
static void fuzz_cache_manager(int rounds) {
    for (int round = 0; round < rounds; ++round) {
        const int page = 1 << pick(0, 5), slots = pick(1, 9), window = pick(1, 70);
        const int is_window[2] = {0, 1}, win[2] = {0, window}, pages[2] = {pick(4, 60), pick(4, 60)};
        const int G = pick(1, 2);
        void* cm = llme_cm_create(G, is_window, win, pages, page, slots);
        REQUIRE(cm != nullptr);
        std::map<int64_t, long> length;                       // what this driver believes
        std::vector<int> done;
        std::vector<int64_t> serials;
        int64_t next_key = 1;
        for (int op = 0; op < 600; ++op) {
            const int what = pick(0, 9);
            if (what <= 1) {                                  // admit
                const int64_t key = pick(0, 3) ? next_key++ : (length.empty() ? next_key++ : length.begin()->first);
                const int rc = llme_cm_admit(cm, key);
                if (length.count(key)) REQUIRE(rc < 0);       // already live: refused
                else if (static_cast<int>(length.size()) == slots) REQUIRE(rc < 0);
                else {
                    REQUIRE(rc >= 0 && rc < slots);
                    length[key] = 0;
                }
            } else if (what <= 5 && !length.empty()) {        // a step: some live requests bring tokens
                std::vector<int64_t> keys;
                std::vector<long> n_new;
                std::vector<int> new_lens;
                for (auto& kv : length)
                    if (pick(0, 2)) {
                        keys.push_back(kv.first);
                        n_new.push_back(pick(0, 3) ? 1 : pick(1, 3 * page + 5));
                        new_lens.push_back(static_cast<int>(n_new.back()));
                    }
                if (keys.empty()) continue;
                const int S = static_cast<int>(keys.size());
                const int rc = llme_cm_reserve_batch(cm, S, keys.data(), n_new.data());
                REQUIRE(rc == 0 || rc == 1);
                REQUIRE(llme_cm_check(cm) == 0);
                if (rc == 0) continue;                        // pools short: nothing changed
                // what the step function asks of the manager, into buffers of exactly the needed size
                std::vector<long> lens(S);
                REQUIRE(llme_cm_lengths(cm, S, keys.data(), lens.data()) == 0);
                long T = 0;
                int width = 1;
                for (int i = 0; i < S; ++i) {
                    REQUIRE(lens[i] == length[keys[i]]);
                    T += n_new[i];
                    width = std::max(width, static_cast<int>((lens[i] + n_new[i] + page - 1) / page));
                }
                std::vector<int> positions(T), seq_idx(T), q_start(S + 1), ctx_len(S), slot(S), tables(static_cast<size_t>(G) * S * width);
                const long top = llme_cm_fill_step(cm, S, keys.data(), new_lens.data(), width, positions.data(), seq_idx.data(),
                                                   q_start.data(), ctx_len.data(), slot.data(), tables.data());
                REQUIRE(top >= 0 && q_start[S] == T);
                for (int i = 0; i < S; ++i) {
                    REQUIRE(llme_cm_commit(cm, keys[i], n_new[i]) == 0);
                    length[keys[i]] += n_new[i];
                    // the full group's table covers every token; all its entries are pages of the pool
                    const int nb = llme_cm_table_len(cm, keys[i], 0);
                    REQUIRE(nb == (length[keys[i]] + page - 1) / page);
                    for (int b = 0; b < std::min(nb, width); ++b) {
                        const int pg = tables[static_cast<size_t>(i) * width + b];
                        REQUIRE(pg >= 0 && pg < pages[0]);
                    }
                }
            } else if (what <= 7 && !length.empty()) {        // a recorded decode step of all live requests
                std::vector<int64_t> keys;
                for (auto& kv : length) keys.push_back(kv.first);
                const int S = static_cast<int>(keys.size());
                std::vector<int> lens(S);
                const int rc = llme_cm_decode_begin(cm, S, keys.data(), lens.data(), pick(0, 1) ? 0 : 400);
                REQUIRE(rc == 0 || rc == 1 || rc == 2);
                if (rc != 1) continue;
                int width = 1;
                for (int i = 0; i < S; ++i) width = std::max(width, (lens[i] + 1 + page - 1) / page);
                width += pick(0, 3);
                std::vector<int> l2(S), sl(S), tables(static_cast<size_t>(G) * S * width, -7);
                done.assign(static_cast<size_t>(G) * S, 0);
                serials.assign(S, 0);
                REQUIRE(llme_cm_fill_decode(cm, S, keys.data(), width, l2.data(), sl.data(), tables.data(), done.data(),
                                            serials.data()) == 0);
                REQUIRE(llme_cm_commit_batch(cm, S, keys.data(), 1) == 0);
                for (int i = 0; i < S; ++i) {
                    REQUIRE(l2[i] == length[keys[i]]);
                    length[keys[i]] += 1;
                }
            } else if (!length.empty()) {                     // release
                auto it = length.begin();
                std::advance(it, pick(0, static_cast<int>(length.size()) - 1));
                REQUIRE(llme_cm_release(cm, it->first) == 0);
                REQUIRE(llme_cm_release(cm, it->first) < 0);  // twice: refused
                length.erase(it);
            }
            REQUIRE(llme_cm_check(cm) == 0);
        }
        for (auto& kv : length) REQUIRE(llme_cm_release(cm, kv.first) == 0);
        for (int g = 0; g < G; ++g) REQUIRE(llme_cm_free_pages(cm, g) == llme_cm_num_pages(cm, g));
        REQUIRE(llme_cm_free_slots(cm) == slots && llme_cm_check(cm) == 0);
        llme_cm_destroy(cm);
    }
}

// ---- the scheduler with a stand-in for the model ----
static void fuzz_scheduler(int rounds) {
    for (int round = 0; round < rounds; ++round) {
        const int page = 1 << pick(1, 4), max_concurrent = pick(1, 6), budget = pick(1, 40);
        const int is_window[1] = {0}, win[1] = {0}, pages[1] = {pick(3, 40)};
        void* cm = llme_cm_create(1, is_window, win, pages, page, max_concurrent);
        void* sc = llme_sched_create(cm, max_concurrent, budget);
        REQUIRE(cm && sc);
        REQUIRE(llme_sched_set_decode_round(sc, -1) < 0 && llme_sched_set_decode_round(sc, pick(0, 4)) == 0);
        REQUIRE(llme_sched_set_row_round(sc, 4, 4) < 0 && llme_sched_set_row_round(sc, pick(0, 1) * pick(2, 12), 1) == 0);
        const int n_requests = pick(1, 14);
        std::vector<std::vector<int>> prompts;
        std::vector<long> max_new;
        for (int i = 0; i < n_requests; ++i) {
            std::vector<int> p(pick(1, 60));
            for (int& t : p) t = pick(0, 99);
            prompts.push_back(p);
            max_new.push_back(pick(0, 25));
            REQUIRE(llme_sched_enqueue(sc, p.data(), static_cast<long>(p.size()), max_new.back()) == i);
        }
        const int eos[2] = {7, 13};
        const long cap = budget + max_concurrent;             // the most tokens a step can carry
        int guard = 0;
        while (!llme_sched_idle(sc)) {
            REQUIRE(++guard < 5000);
            int n_admitted = 0;
            std::vector<int> admitted(max_concurrent), count(max_concurrent), want(max_concurrent), tokens(cap);
            std::vector<int64_t> seq(max_concurrent);
            std::vector<long> gen(max_concurrent);
            const int E = llme_sched_plan(sc, &n_admitted, admitted.data(), seq.data(), count.data(), want.data(), gen.data(),
                                          tokens.data(), cap);
            REQUIRE(E >= 0 && E <= max_concurrent && n_admitted <= max_concurrent);
            const int fate = pick(0, 19);
            if (E > 0 && fate == 0) {                         // the model run failed before it changed anything
                llme_sched_abort(sc);
                continue;
            }
            std::vector<long> n_new(E);
            long used = 0;
            int wanted = 0;
            for (int i = 0; i < E; ++i) {
                n_new[i] = count[i];
                used += count[i];
                wanted += want[i] ? 1 : 0;
            }
            REQUIRE(used <= cap);
            if (E > 0) {
                REQUIRE(llme_cm_reserve_batch(cm, E, seq.data(), n_new.data()) == 1);   // plan() has counted the pages
                for (int i = 0; i < E; ++i) REQUIRE(llme_cm_commit(cm, seq[i], n_new[i]) == 0);
            }
            if (E > 0 && fate == 1) {                         // the batch ran, the tokens never arrived
                REQUIRE(llme_sched_fail(sc) >= 0);
                REQUIRE(llme_cm_check(cm) == 0);
                continue;
            }
            std::vector<int> sampled(std::max(wanted, 1));
            for (int i = 0; i < wanted; ++i) sampled[i] = pick(0, 99);
            REQUIRE(llme_sched_complete(sc, sampled.data(), wanted, eos, 2) >= 0);
            REQUIRE(llme_cm_check(cm) == 0);
        }
        REQUIRE(llme_sched_num_results(sc) == n_requests);
        for (int i = 0; i < n_requests; ++i) {
            int64_t id;
            long plen, ntok;
            int reason;
            REQUIRE(llme_sched_result_info(sc, i, &id, &plen, &ntok, &reason) == 0);
            REQUIRE(id == i && plen == static_cast<long>(prompts[i].size()) && ntok >= plen && ntok <= plen + max_new[i]);
            REQUIRE(reason >= 1 && reason <= 4);
            std::vector<int> out(std::max<long>(ntok, 1));
            REQUIRE(llme_sched_result_tokens(sc, i, out.data()) == 0);
            for (long t = 0; t < plen; ++t) REQUIRE(out[t] == prompts[i][t]);
            for (long t = plen; t < ntok; ++t) REQUIRE(out[t] != 7 && out[t] != 13);   // an EOS id is never appended
        }
        REQUIRE(llme_cm_free_pages(cm, 0) == pages[0] && llme_cm_free_slots(cm) == max_concurrent);
        llme_sched_destroy(sc);
        llme_cm_destroy(cm);
    }
}

// ---- the plain backend of the whole model: buffers of exactly the needed size ----
static void run_plain_model() {
    const int L = 2, H = 24, F = 40, n_q = 3, n_kv = 1, hd = 8, V = 37, T = 19;
    std::uniform_real_distribution<float> u(-0.3f, 0.3f);
    auto tensor = [&](size_t n) {
        std::vector<float> t(n);
        for (float& x : t) x = u(rng);
        return t;
    };
    std::vector<std::vector<float>> keep;
    std::vector<const float*> layers;
    for (int l = 0; l < L; ++l) {
        const size_t sizes[9] = {size_t(H), size_t(n_q * hd) * H, size_t(n_kv * hd) * H, size_t(n_kv * hd) * H,
                                 size_t(H) * n_q * hd, size_t(H), size_t(F) * H, size_t(F) * H, size_t(H) * F};
        for (size_t n : sizes) {
            keep.push_back(tensor(n));
            layers.push_back(keep.back().data());
        }
    }
    const std::vector<float> embed = tensor(size_t(V) * H), norm = tensor(H), head = tensor(size_t(V) * H);
    std::vector<int32_t> tokens(T), positions(T);
    for (int t = 0; t < T; ++t) {
        tokens[t] = pick(0, V - 1);
        positions[t] = 5 + t;
    }
    const int32_t sizes[8] = {L, H, F, n_q, n_kv, hd, V, 6};
    const double rope[6] = {10000.0, 1.0, 8.0, 1.0, 4.0, 16.0};
    std::vector<float> logits(size_t(T) * V, 123.f);
    REQUIRE(llme_plain_llama_forward(sizes, rope, 1e-5f, embed.data(), norm.data(), head.data(), layers.data(), tokens.data(),
                                     positions.data(), T, logits.data()) == 0);
    for (float x : logits) REQUIRE(x == x && x != 123.f);
    tokens[3] = V;                                            // an id out of range is refused
    REQUIRE(llme_plain_llama_forward(sizes, rope, 1e-5f, embed.data(), norm.data(), head.data(), layers.data(), tokens.data(),
                                     positions.data(), T, logits.data()) < 0);
}

// ---- the decode plan: any sizes, a number of splits within its bounds ----
static void fuzz_decode_plan(int rounds) {
    for (int round = 0; round < rounds; ++round) {
        const int S = pick(1, 300), tiles = pick(1, 40), units = pick(1, 400), most = pick(1, 70);
        std::vector<int> lens(static_cast<size_t>(S));
        for (int& n : lens) n = pick(0, pick(0, 1) ? 200000 : 700);
        const long plan_len = pick(0, 1) ? pick(1, 300000) : 1;
        const int first = pick(1, 6);
        const int n = llme_decode_cut(lens.data(), S, tiles, units, 16 * pick(1, 8), plan_len, first, most, 6.0, 9.5, 8.3,
                                      0.5, pick(0, 20), 1.0, 0.05);
        REQUIRE(n >= first && (n == first || n <= most) && n <= 64);
        REQUIRE(n == first || static_cast<long>(S) * tiles * n <= 10L * units);
    }
}

int main(int argc, char** argv) {
    const int rounds = argc > 1 ? std::atoi(argv[1]) : 40;
    if (argc > 2) rng.seed(static_cast<unsigned>(std::atoi(argv[2])));
    fuzz_cache_manager(rounds);
    fuzz_scheduler(rounds * 5);
    run_plain_model();
    fuzz_decode_plan(rounds * 20);
    std::printf("ok\n");
    return 0;
}
