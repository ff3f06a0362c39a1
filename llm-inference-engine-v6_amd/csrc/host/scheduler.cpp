// Continuous batching above the step function: who is admitted, which tokens a step carries, who
// finishes and why.
//
// State machine, knobs and finish reasons are the reference's ContinuousBatchScheduler
// (src/scheduler.cpp:136-319): requests wait in a FIFO, are admitted while fewer than
// max_concurrent are live (no page check at admission), prefill under one token budget per step
// shared in admission order, then decode one token per step; a sequence ends with "stop" (an EOS
// id was sampled; it is not appended), "length" (max_new_tokens reached, or 0 asked) or
// "capacity" (the page pool cannot hold its next tokens; what it generated so far is kept;
// nothing is preempted or recomputed). Results come back in enqueue order.
//
// What differs from the reference: a step is ONE mixed batch. Prompt portions and the single
// tokens of decoding requests go through the model together, and because pages are reserved
// before the batch runs, running out of pages is decided here, on the host, in the reference's
// order (prompt portions take pages first, then decoding requests). A request whose prompt ends
// in step k decodes first in step k + 1 (the reference does both in step k); token streams are
// the same. Pages of a finished request go back at the end of the step in which it finished,
// which is when the reference's next step would find them.
//
// This file decides; it runs nothing. A step is plan() (admission, the batch), then the caller
// runs the batch through the model and samples, then complete() (the sampled tokens arrive,
// prompts move on by the portions that ran, sequences move on or finish, pages go back). If the
// model run fails, the caller calls abort() instead of complete(): the planned portions have not
// run, the prompts stay where they were, and the next plan() offers them again. (What plan()
// decided apart from the batch stands: admissions, and requests ended for want of pages.) If the
// batch ran, so that the cache holds its tokens, and only what came after failed (the choice of the
// next tokens, the copy to the host), the caller calls fail(): no sequence of the batch can go on
// from a token that is not known, so each of them ends with "error" and keeps what it had.
// The cache manager is the one the step function reserves and commits in; sequence ids are its
// request keys.
#include "host_api.h"

#include <algorithm>
#include <cstdint>
#include <deque>
#include <memory>
#include <utility>
#include <vector>

extern "C" {
int llme_cm_admit(void* h, int64_t key);
int llme_cm_num_groups(void* h);
int llme_cm_pages_needed(void* h, int64_t key, long n_new, int* out);
int llme_cm_can_reserve(void* h, int64_t key, long n_new, const int* pending);
int llme_cm_release(void* h, int64_t key);
}

namespace llme_host {

enum State : int { kWaiting = 0, kPrefilling = 1, kRunning = 2, kFinished = 3 };
enum Reason : int { kNone = 0, kStop = 1, kLength = 2, kCapacity = 3, kError = 4 };

struct Seq {
    int64_t id = 0;
    std::vector<int> tokens;                // prompt, then what was generated
    long prompt_len = 0;
    long max_new = 0;
    State state = kWaiting;
    long cursor = 0;                        // prompt tokens that have gone through the model
    Reason reason = kNone;
    long generated() const { return static_cast<long>(tokens.size()) - prompt_len; }
};

class Scheduler {
public:
    Scheduler(void* cm, int max_concurrent, long budget) : cm_(cm), max_concurrent_(max_concurrent), budget_(budget) {}

    void set_budget(long b) { budget_ = b; }
    void set_decode_round(int requests) { decode_round_ = requests; }
    void set_row_round(long rows, long over) {
        row_round_ = rows;
        row_over_ = over;
    }
    long budget() const { return budget_; }
    int max_concurrent() const { return max_concurrent_; }

    int64_t enqueue(const int* prompt, long n, long max_new) {
        auto s = std::make_unique<Seq>();
        s->id = next_id_++;
        s->tokens.assign(prompt, prompt + n);
        s->prompt_len = n;
        s->max_new = max_new;
        const int64_t id = s->id;
        waiting_.push_back(std::move(s));
        return id;
    }

    bool idle() const { return waiting_.empty() && prefilling_.empty() && running_.empty(); }
    void counts(int* out) const {
        out[0] = static_cast<int>(waiting_.size());
        out[1] = static_cast<int>(prefilling_.size());
        out[2] = static_cast<int>(running_.size());
    }

    // Admission, then the step's batch. Returns the number of entries, or an error code.
    int plan(int* n_admitted, int* admitted_slots, int64_t* entry_seq, int* entry_count, int* entry_want,
             long* entry_gen, int* tokens, long tokens_cap) {
        if (planned_) return LLME_HOST_BAD_ARGUMENT;  // the last step was neither completed nor aborted
        owners_.clear();
        prompt_ends_.clear();
        portions_.clear();
        batch_.clear();
        *n_admitted = 0;
        // admission: no page check, as in the reference
        while (!waiting_.empty() && static_cast<int>(prefilling_.size() + running_.size()) < max_concurrent_) {
            const int slot = llme_cm_admit(cm_, waiting_.front()->id);
            if (slot < 0) return slot;
            std::unique_ptr<Seq> s = std::move(waiting_.front());
            waiting_.pop_front();
            s->state = kPrefilling;
            admitted_slots[(*n_admitted)++] = slot;
            prefilling_.push_back(std::move(s));
        }
        const int G = llme_cm_num_groups(cm_);
        std::vector<int> pending(static_cast<size_t>(G), 0), need(static_cast<size_t>(G), 0);
        auto take_pages = [&](Seq& s, long n) {
            if (llme_cm_can_reserve(cm_, s.id, n, pending.data()) != 1) return false;
            llme_cm_pages_needed(cm_, s.id, n, need.data());
            for (int g = 0; g < G; ++g) pending[static_cast<size_t>(g)] += need[static_cast<size_t>(g)];
            return true;
        };
        int E = 0;
        long used = 0;
        auto add_entry = [&](Seq& s, long first, long n, bool want, long gen) {
            if (used + n > tokens_cap) return false;
            entry_seq[E] = s.id;
            entry_count[E] = static_cast<int>(n);
            entry_want[E] = want ? 1 : 0;
            entry_gen[E] = gen;
            std::copy(s.tokens.begin() + first, s.tokens.begin() + first + n, tokens + used);
            used += n;
            ++E;
            batch_.push_back(&s);
            if (want) owners_.push_back(&s);
            return true;
        };
        // prompt portions under the step's token budget, in admission order
        long budget = budget_;
        long decoding = 0;
        for (auto& sp : running_) decoding += sp->state == kRunning ? 1 : 0;
        for (auto& sp : prefilling_) {
            Seq& s = *sp;
            if (budget <= 0) break;
            long n = std::min(budget, s.prompt_len - s.cursor);
            if (n <= 0 || s.state == kFinished) continue;
            // The portion that uses the budget up, in the middle of its prompt: where the step's rows (prompt
            // tokens and one per decoding request) would come to a few more than a multiple of row_round_,
            // the portion leaves those few for the next step. (The engine's matrix products fill whole rounds
            // of workgroups at such multiples and run a few rows more in launches of their own, which read
            // every weight again: a step of 1,024 + 8 rows took 3.84 ms at the 1B sizes, one of 1,024 3.30.)
            if (row_round_ > 0 && n == budget && n < s.prompt_len - s.cursor) {
                const long rows = (budget_ - budget) + n + decoding, over = rows % row_round_;
                if (rows > row_round_ && over > 0 && over <= row_over_ && over < n) {
                    n -= over;
                    budget = n;                       // (what is given back is nobody else's either)
                }
            }
            if (!take_pages(s, n)) {
                finish(s, kCapacity);
                continue;
            }
            const bool ends = s.cursor + n == s.prompt_len;
            if (!add_entry(s, s.cursor, n, ends && s.max_new > 0, 0)) return LLME_HOST_BAD_ARGUMENT;
            if (ends) prompt_ends_.push_back(&s);
            portions_.push_back({&s, n});             // (the prompt moves on in complete(), once the portion has run)
            budget -= n;
        }
        // one token for every decoding request: pages are taken in the order in which the prompts ended;
        // the entries then stand in the order of the requests' lengths, the longest first (which stays the
        // same from step to step while nobody joins or leaves: every request grows by one). The decode
        // kernels deal a step's requests out to the compute units in turn, so that where there are more
        // requests than units a unit gets one of the longest together with one of the shortest (measured at
        // the 1B sizes, lengths uniform in 256 .. 6,144: 44 requests 2.54 -> 2.16 ms a step, 72 requests
        // 3.04 -> 2.79; up to 32 requests the order makes no difference).
        decoding_.clear();
        for (auto& sp : running_) {
            Seq& s = *sp;
            if (s.state != kRunning) continue;
            if (!take_pages(s, 1)) {
                finish(s, kCapacity);
                continue;
            }
            decoding_.push_back(&s);
        }
        std::stable_sort(decoding_.begin(), decoding_.end(),
                         [](const Seq* a, const Seq* b) { return a->tokens.size() > b->tokens.size(); });
        // Where the engine has said after how many requests its decode kernel has given every compute unit one
        // (decode_round_), the requests are cut into such rounds and every other round, counted from the last,
        // is reversed: the unit that got the shortest request of one round gets the longest of the next, and
        // the last round, which may be short and so lands on the first units, meets the short end of the round
        // before it (measured as above: 44 requests 2.03 -> 1.87 ms a step, 64: 2.30 -> 2.09, 96: 3.04 -> 2.89).
        const size_t n_dec = decoding_.size(), per_round = static_cast<size_t>(decode_round_);
        if (per_round > 0 && n_dec > per_round) {
            const size_t rounds = (n_dec + per_round - 1) / per_round;
            for (size_t back = 1; back < rounds; back += 2) {
                const size_t r = rounds - 1 - back;      // (a full round: only the last can be short)
                std::reverse(decoding_.begin() + static_cast<long>(r * per_round),
                             decoding_.begin() + static_cast<long>((r + 1) * per_round));
            }
        }
        for (Seq* s : decoding_)
            if (!add_entry(*s, static_cast<long>(s->tokens.size()) - 1, 1, true, s->generated())) return LLME_HOST_BAD_ARGUMENT;
        planned_ = true;
        return E;
    }

    // The sampled tokens of the wanted rows, in the order of the entries that wanted one.
    int complete(const int* sampled, int n, const int* eos, int n_eos) {
        if (!planned_ || n != static_cast<int>(owners_.size())) return LLME_HOST_BAD_ARGUMENT;
        planned_ = false;
        for (const auto& portion : portions_) portion.first->cursor += portion.second;
        portions_.clear();
        for (int i = 0; i < n; ++i) {
            Seq& s = *owners_[static_cast<size_t>(i)];
            // a sampled token arrives for a sequence (src/scheduler.cpp:208-227, 271-282)
            if (std::find(eos, eos + n_eos, sampled[i]) != eos + n_eos) {
                finish(s, kStop);
                continue;
            }
            s.tokens.push_back(sampled[i]);
            if (s.generated() >= s.max_new) finish(s, kLength);
        }
        for (Seq* sp : prompt_ends_) {
            Seq& s = *sp;
            if (s.state == kFinished) continue;
            if (s.max_new == 0) {
                finish(s, kLength);             // nothing is sampled (src/scheduler.cpp:203-207)
                continue;
            }
            s.state = kRunning;
            auto it = std::find_if(prefilling_.begin(), prefilling_.end(),
                                   [&](const std::unique_ptr<Seq>& p) { return p.get() == sp; });
            running_.push_back(std::move(*it));
            prefilling_.erase(it);
        }
        owners_.clear();
        prompt_ends_.clear();
        batch_.clear();
        return retire();
    }

    // The planned step ran, but its tokens never arrived: every sequence of the batch ends with
    // "error", with the tokens it had, and its pages go back. Returns how many ended.
    int fail() {
        if (!planned_) return LLME_HOST_BAD_ARGUMENT;
        planned_ = false;
        for (Seq* s : batch_) finish(*s, kError);
        owners_.clear();
        prompt_ends_.clear();
        portions_.clear();
        batch_.clear();
        return retire();
    }

    // The planned step did not run: forget the batch, keep every prompt where it was.
    void abort() {
        planned_ = false;
        owners_.clear();
        prompt_ends_.clear();
        portions_.clear();
        batch_.clear();
    }

    int num_results() const { return static_cast<int>(results_.size()); }
    const Seq* result(int i) const {
        return i >= 0 && i < num_results() ? results_[static_cast<size_t>(i)].get() : nullptr;
    }
    void clear_results() { results_.clear(); }

private:
    static void finish(Seq& s, Reason r) {
        s.state = kFinished;
        s.reason = r;
    }
    // Finished sequences leave the lists, give their pages back and become results (in enqueue order).
    int retire() {
        int finished = 0;
        for (auto* list : {&prefilling_, &running_}) {
            std::vector<std::unique_ptr<Seq>> keep;
            for (auto& sp : *list) {
                if (sp->state == kFinished) {
                    llme_cm_release(cm_, sp->id);
                    results_.push_back(std::move(sp));
                    ++finished;
                } else {
                    keep.push_back(std::move(sp));
                }
            }
            list->swap(keep);
        }
        if (finished)
            std::sort(results_.begin(), results_.end(),
                      [](const std::unique_ptr<Seq>& a, const std::unique_ptr<Seq>& b) { return a->id < b->id; });
        return finished;
    }
    void* cm_;
    int max_concurrent_;
    long budget_;
    int decode_round_ = 0;                             // see set_decode_round
    long row_round_ = 0, row_over_ = 0;                // see set_row_round and plan()
    int64_t next_id_ = 0;
    bool planned_ = false;
    std::deque<std::unique_ptr<Seq>> waiting_;
    std::vector<std::unique_ptr<Seq>> prefilling_, running_, results_;
    std::vector<Seq*> owners_, prompt_ends_, batch_;   // between plan() and complete(): who gets a token, whose prompt ends, who takes part
    std::vector<Seq*> decoding_;                       // plan()'s own: the step's decoding requests while they are put in order
    std::vector<std::pair<Seq*, long>> portions_;  // prompt tokens that the planned step carries
};

}  // namespace llme_host

using llme_host::Scheduler;

extern "C" {

void* llme_sched_create(void* cache_manager, int max_concurrent, long budget) {
    if (!cache_manager || max_concurrent <= 0 || budget <= 0) return nullptr;
    return new Scheduler(cache_manager, max_concurrent, budget);
}
void llme_sched_destroy(void* h) { delete static_cast<Scheduler*>(h); }
// requests > 0: the order of a step's decoding requests is made for a kernel that deals them out to that many
// places in turn (see plan()); 0: longest first.
int llme_sched_set_decode_round(void* h, int requests) {
    if (requests < 0) return LLME_HOST_BAD_ARGUMENT;
    static_cast<Scheduler*>(h)->set_decode_round(requests);
    return 0;
}
// rows > 0: a step's last prompt portion gives up to `over` tokens back where the step's rows would be that many
// more than a multiple of `rows` (see plan()); 0: never.
int llme_sched_set_row_round(void* h, long rows, long over) {
    if (rows < 0 || over < 0 || (rows > 0 && over >= rows)) return LLME_HOST_BAD_ARGUMENT;
    static_cast<Scheduler*>(h)->set_row_round(rows, over);
    return 0;
}
int llme_sched_set_budget(void* h, long budget) {
    if (budget <= 0) return LLME_HOST_BAD_ARGUMENT;
    static_cast<Scheduler*>(h)->set_budget(budget);
    return 0;
}
long llme_sched_enqueue(void* h, const int* prompt, long n, long max_new_tokens) {
    if (n <= 0 || max_new_tokens < 0) return LLME_HOST_BAD_ARGUMENT;
    return static_cast<long>(static_cast<Scheduler*>(h)->enqueue(prompt, n, max_new_tokens));
}
int llme_sched_idle(void* h) { return static_cast<Scheduler*>(h)->idle() ? 1 : 0; }
void llme_sched_counts(void* h, int* out) { static_cast<Scheduler*>(h)->counts(out); }
int llme_sched_plan(void* h, int* n_admitted, int* admitted_slots, int64_t* entry_seq, int* entry_count, int* entry_want,
                    long* entry_gen, int* tokens, long tokens_cap) {
    return static_cast<Scheduler*>(h)->plan(n_admitted, admitted_slots, entry_seq, entry_count, entry_want, entry_gen,
                                            tokens, tokens_cap);
}
int llme_sched_complete(void* h, const int* sampled, int n, const int* eos, int n_eos) {
    return static_cast<Scheduler*>(h)->complete(sampled, n, eos, n_eos);
}
void llme_sched_abort(void* h) { static_cast<Scheduler*>(h)->abort(); }
int llme_sched_fail(void* h) { return static_cast<Scheduler*>(h)->fail(); }
int llme_sched_num_results(void* h) { return static_cast<Scheduler*>(h)->num_results(); }
// reason: 1 "stop", 2 "length", 3 "capacity", 4 "error"
int llme_sched_result_info(void* h, int i, int64_t* seq_id, long* prompt_len, long* n_tokens, int* reason) {
    const auto* s = static_cast<Scheduler*>(h)->result(i);
    if (!s) return LLME_HOST_BAD_ARGUMENT;
    *seq_id = s->id;
    *prompt_len = s->prompt_len;
    *n_tokens = static_cast<long>(s->tokens.size());
    *reason = static_cast<int>(s->reason);
    return 0;
}
int llme_sched_result_tokens(void* h, int i, int* out) {
    const auto* s = static_cast<Scheduler*>(h)->result(i);
    if (!s) return LLME_HOST_BAD_ARGUMENT;
    std::copy(s->tokens.begin(), s->tokens.end(), out);
    return 0;
}
void llme_sched_clear_results(void* h) { static_cast<Scheduler*>(h)->clear_results(); }

}  // extern "C"
