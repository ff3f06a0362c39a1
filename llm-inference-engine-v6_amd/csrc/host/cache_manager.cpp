// The cache manager's bookkeeping on the host: page pools, block tables and state slots.
//
// Reference: BlockManager hands out block ids from a FIFO free list and a PagedKVCache grows a
// per-sequence block table as positions cross block boundaries, giving everything back at
// release_all (src/paged_kv.cpp:8-47, 88-101, 135-139). Here the same bookkeeping is done before
// a step instead of inside the forward pass: pages for all tokens of a step are reserved first,
// so a step never fails for capacity half-way.
//
// Layers with the same needs form a group with a page pool and block tables of its own: a
// "full" group keeps every token of a request; a "window" group gives pages back once every
// position in them lies behind the window of the next token. Beside the pages, every live
// request holds a slot: a row in each fixed-size state tensor.
//
// Plain C++ with a C interface (handles and integer codes), no GPU calls: the Python classes in
// llmengine/cache/manager.py are its face. Requests are named by 64-bit keys that the caller
// chooses. A call that fails changes nothing.
#include "host_api.h"

#include <algorithm>
#include <cstdint>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

namespace llme_host {

// A fixed set of page ids; FIFO reuse like the reference's free list (src/paged_kv.cpp:30-42).
class PagePool {
public:
    explicit PagePool(int num_pages) : num_pages_(num_pages), held_(static_cast<size_t>(num_pages), 0) {
        for (int i = 0; i < num_pages; ++i) free_.push_back(i);
    }
    int num_pages() const { return num_pages_; }
    int free_pages() const { return static_cast<int>(free_.size()); }
    int allocate() {
        if (free_.empty()) return -1;
        const int page = free_.front();
        free_.pop_front();
        held_[static_cast<size_t>(page)] = 1;
        return page;
    }
    bool is_held(int page) const { return page >= 0 && page < num_pages_ && held_[static_cast<size_t>(page)]; }
    bool free(int page) {                       // false: the page is not held
        if (!is_held(page)) return false;
        held_[static_cast<size_t>(page)] = 0;
        free_.push_back(page);
        return true;
    }
    int held_count() const { return num_pages_ - free_pages(); }
    const std::vector<char>& held() const { return held_; }

private:
    int num_pages_;
    std::deque<int> free_;
    std::vector<char> held_;
};

struct Group {
    bool window = false;
    int window_len = 0;
    PagePool pool;
    Group(bool w, int wl, int pages) : window(w), window_len(wl), pool(pages) {}
};

struct Request {
    int64_t serial = 0;                             // counts admissions: tells a request from an earlier one of the same key
    int slot = 0;
    long length = 0;                                // tokens committed
    long reserved = 0;                              // tokens with pages reserved (>= length)
    std::vector<std::vector<int>> tables;           // per group: page per logical block, -1 = given back
};

class CacheManager {
public:
    CacheManager(int page_size, int max_requests) : page_size_(page_size), max_requests_(max_requests) {
        for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);
    }
    void add_group(bool window, int window_len, int pages) { groups_.emplace_back(window, window_len, pages); }
    int num_groups() const { return static_cast<int>(groups_.size()); }
    Group* group(int g) { return g >= 0 && g < num_groups() ? &groups_[static_cast<size_t>(g)] : nullptr; }
    Request* find(int64_t key) {
        auto it = requests_.find(key);
        return it == requests_.end() ? nullptr : &it->second;
    }
    int free_slots() const { return static_cast<int>(free_slots_.size()); }
    int live() const { return static_cast<int>(requests_.size()); }

    int admit(int64_t key) {
        if (requests_.count(key)) return LLME_HOST_ALREADY_LIVE;
        if (free_slots_.empty()) return LLME_HOST_NO_SLOT;
        Request r;
        r.serial = ++admissions_;
        r.slot = free_slots_.back();
        free_slots_.pop_back();
        r.tables.assign(groups_.size(), {});
        const int slot = r.slot;
        requests_.emplace(key, std::move(r));
        order_.push_back(key);
        return slot;
    }

    // First logical block that a token at `position` reads in this group.
    long first_needed_block(const Group& g, long position) const {
        if (!g.window) return 0;
        const long lo = position - g.window_len + 1;
        return (lo > 0 ? lo : 0) / page_size_;
    }

    // Logical blocks that must get a page before n_new tokens are appended.
    void missing(const Request& r, int gi, long n_new, std::vector<long>& out) const {
        const Group& g = groups_[static_cast<size_t>(gi)];
        const std::vector<int>& table = r.tables[static_cast<size_t>(gi)];
        out.clear();
        const long first = first_needed_block(g, r.length);
        const long last = (r.length + n_new - 1) / page_size_;
        if (!g.window) {                            // the table has no holes: only its end grows
            for (long b = std::max<long>(first, static_cast<long>(table.size())); b <= last; ++b) out.push_back(b);
            return;
        }
        for (long b = first; b <= last; ++b)
            if (b >= static_cast<long>(table.size()) || table[static_cast<size_t>(b)] < 0) out.push_back(b);
    }

    int pages_needed(int64_t key, long n_new, int* out) {
        Request* r = find(key);
        if (!r) return LLME_HOST_NOT_LIVE;
        std::vector<long> blocks;
        for (int g = 0; g < num_groups(); ++g) {
            missing(*r, g, n_new, blocks);
            out[g] = static_cast<int>(blocks.size());
        }
        return 0;
    }

    int can_reserve(int64_t key, long n_new, const int* pending) {
        Request* r = find(key);
        if (!r) return LLME_HOST_NOT_LIVE;
        std::vector<long> blocks;
        for (int g = 0; g < num_groups(); ++g) {
            missing(*r, g, n_new, blocks);
            const long need = static_cast<long>(blocks.size()) + (pending ? pending[g] : 0);
            if (need > groups_[static_cast<size_t>(g)].pool.free_pages()) return 0;
        }
        return 1;
    }

    // All of the requests get their pages for n_new[i] more tokens, or nothing changes.
    int reserve_batch(int n, const int64_t* keys, const long* n_new) {
        struct Plan {
            Request* req;
            int group;
            std::vector<long> blocks;
        };
        std::vector<Plan> plans;
        std::vector<long> need(groups_.size(), 0);
        std::vector<long> blocks;
        for (int i = 0; i < n; ++i) {
            if (n_new[i] <= 0) return LLME_HOST_BAD_ARGUMENT;
            Request* r = find(keys[i]);
            if (!r) return LLME_HOST_NOT_LIVE;
            for (int g = 0; g < num_groups(); ++g) {
                missing(*r, g, n_new[i], blocks);
                if (blocks.empty()) continue;           // the common case of decoding: the page is there
                // the same request twice in a batch would count its blocks twice: refuse it
                for (const Plan& p : plans)
                    if (p.req == r && p.group == g) return LLME_HOST_BAD_ARGUMENT;
                need[static_cast<size_t>(g)] += static_cast<long>(blocks.size());
                plans.push_back(Plan{r, g, blocks});
            }
        }
        for (int g = 0; g < num_groups(); ++g)
            if (need[static_cast<size_t>(g)] > groups_[static_cast<size_t>(g)].pool.free_pages()) return 0;
        for (Plan& p : plans) {
            std::vector<int>& table = p.req->tables[static_cast<size_t>(p.group)];
            PagePool& pool = groups_[static_cast<size_t>(p.group)].pool;
            for (long b : p.blocks) {
                if (static_cast<long>(table.size()) <= b) table.resize(static_cast<size_t>(b) + 1, -1);
                table[static_cast<size_t>(b)] = pool.allocate();
            }
        }
        for (int i = 0; i < n; ++i) {
            Request* r = find(keys[i]);
            r->reserved = std::max(r->reserved, r->length + n_new[i]);
        }
        return 1;
    }

    // The step wrote n_new tokens: the request is that much longer, and window groups give back
    // the pages no later token will read.
    int commit(int64_t key, long n_new) {
        Request* r = find(key);
        if (!r) return LLME_HOST_NOT_LIVE;
        if (n_new < 0 || r->length + n_new > r->reserved) return LLME_HOST_NOT_RESERVED;
        r->length += n_new;
        for (int gi = 0; gi < num_groups(); ++gi) {
            Group& g = groups_[static_cast<size_t>(gi)];
            if (!g.window) continue;
            std::vector<int>& table = r->tables[static_cast<size_t>(gi)];
            const long keep_from = first_needed_block(g, r->length);       // the next token's first block
            const long end = std::min<long>(keep_from, static_cast<long>(table.size()));
            for (long b = 0; b < end; ++b)
                if (table[static_cast<size_t>(b)] >= 0) {
                    g.pool.free(table[static_cast<size_t>(b)]);
                    table[static_cast<size_t>(b)] = -1;
                }
        }
        return 0;
    }

    int release(int64_t key) {
        Request* r = find(key);
        if (!r) return LLME_HOST_NOT_LIVE;
        for (int gi = 0; gi < num_groups(); ++gi)
            for (int page : r->tables[static_cast<size_t>(gi)])
                if (page >= 0) groups_[static_cast<size_t>(gi)].pool.free(page);
        free_slots_.push_back(r->slot);
        requests_.erase(key);
        order_.erase(std::find(order_.begin(), order_.end(), key));
        return 0;
    }

    const std::vector<int64_t>& order() const { return order_; }

    // No page is lost or held twice, no slot is held twice. 0, or a code that says what is wrong.
    int check() const {
        for (size_t gi = 0; gi < groups_.size(); ++gi) {
            const PagePool& pool = groups_[gi].pool;
            std::vector<char> seen(static_cast<size_t>(pool.num_pages()), 0);
            long owned = 0;
            for (const auto& kv : requests_)
                for (int page : kv.second.tables[gi]) {
                    if (page < 0) continue;
                    if (page >= pool.num_pages()) return LLME_HOST_CHECK_PAGE_MISMATCH;
                    if (seen[static_cast<size_t>(page)]) return LLME_HOST_CHECK_PAGE_TWICE;
                    seen[static_cast<size_t>(page)] = 1;
                    ++owned;
                }
            if (seen != pool.held()) return LLME_HOST_CHECK_PAGE_MISMATCH;
            if (owned + pool.free_pages() != pool.num_pages()) return LLME_HOST_CHECK_PAGE_LOST;
        }
        std::vector<char> slot_seen(static_cast<size_t>(max_requests_), 0);
        for (const auto& kv : requests_) {
            const int s = kv.second.slot;
            if (s < 0 || s >= max_requests_ || slot_seen[static_cast<size_t>(s)]) return LLME_HOST_CHECK_SLOT_TWICE;
            slot_seen[static_cast<size_t>(s)] = 1;
        }
        for (int s : free_slots_) {
            if (s < 0 || s >= max_requests_ || slot_seen[static_cast<size_t>(s)]) return LLME_HOST_CHECK_SLOT_TWICE;
            slot_seen[static_cast<size_t>(s)] = 1;
        }
        if (static_cast<int>(requests_.size() + free_slots_.size()) != max_requests_) return LLME_HOST_CHECK_SLOT_LOST;
        return 0;
    }

    int page_size() const { return page_size_; }

private:
    int page_size_, max_requests_;
    int64_t admissions_ = 0;
    std::vector<Group> groups_;
    std::vector<int> free_slots_;
    std::unordered_map<int64_t, Request> requests_;
    std::vector<int64_t> order_;                    // live requests in the order of their admission
};

}  // namespace llme_host

using llme_host::CacheManager;
using llme_host::PagePool;

extern "C" {

// ---- a pool on its own ----
void* llme_pool_create(int num_pages) { return num_pages > 0 ? new PagePool(num_pages) : nullptr; }
void llme_pool_destroy(void* p) { delete static_cast<PagePool*>(p); }
int llme_pool_allocate(void* p) { return static_cast<PagePool*>(p)->allocate(); }
int llme_pool_free(void* p, int page) { return static_cast<PagePool*>(p)->free(page) ? 0 : LLME_HOST_NOT_HELD; }
int llme_pool_free_pages(void* p) { return static_cast<PagePool*>(p)->free_pages(); }
int llme_pool_is_held(void* p, int page) { return static_cast<PagePool*>(p)->is_held(page) ? 1 : 0; }

// ---- the manager ----
void* llme_cm_create(int n_groups, const int* is_window, const int* window, const int* num_pages, int page_size,
                     int max_requests) {
    if (n_groups < 0 || page_size <= 0 || max_requests <= 0) return nullptr;
    for (int g = 0; g < n_groups; ++g)
        if (num_pages[g] <= 0 || (is_window[g] && window[g] <= 0)) return nullptr;
    CacheManager* m = new CacheManager(page_size, max_requests);
    for (int g = 0; g < n_groups; ++g) m->add_group(is_window[g] != 0, window[g], num_pages[g]);
    return m;
}
void llme_cm_destroy(void* h) { delete static_cast<CacheManager*>(h); }
int llme_cm_num_groups(void* h) { return static_cast<CacheManager*>(h)->num_groups(); }
int llme_cm_admit(void* h, int64_t key) { return static_cast<CacheManager*>(h)->admit(key); }
int llme_cm_is_live(void* h, int64_t key) { return static_cast<CacheManager*>(h)->find(key) ? 1 : 0; }
int llme_cm_slot(void* h, int64_t key) {
    auto* r = static_cast<CacheManager*>(h)->find(key);
    return r ? r->slot : LLME_HOST_NOT_LIVE;
}
long llme_cm_length(void* h, int64_t key) {
    auto* r = static_cast<CacheManager*>(h)->find(key);
    return r ? r->length : static_cast<long>(LLME_HOST_NOT_LIVE);
}
int llme_cm_free_slots(void* h) { return static_cast<CacheManager*>(h)->free_slots(); }
int llme_cm_live(void* h, int64_t* out, int cap) {
    const auto& order = static_cast<CacheManager*>(h)->order();
    const int n = static_cast<int>(order.size());
    for (int i = 0; i < n && i < cap; ++i) out[i] = order[static_cast<size_t>(i)];
    return n;
}
int llme_cm_pages_needed(void* h, int64_t key, long n_new, int* out) {
    return static_cast<CacheManager*>(h)->pages_needed(key, n_new, out);
}
int llme_cm_can_reserve(void* h, int64_t key, long n_new, const int* pending) {
    return static_cast<CacheManager*>(h)->can_reserve(key, n_new, pending);
}
int llme_cm_reserve_batch(void* h, int n, const int64_t* keys, const long* n_new) {
    return static_cast<CacheManager*>(h)->reserve_batch(n, keys, n_new);
}
int llme_cm_commit(void* h, int64_t key, long n_new) { return static_cast<CacheManager*>(h)->commit(key, n_new); }
int llme_cm_release(void* h, int64_t key) { return static_cast<CacheManager*>(h)->release(key); }
int llme_cm_table_len(void* h, int64_t key, int group) {
    auto* m = static_cast<CacheManager*>(h);
    auto* r = m->find(key);
    if (!r) return LLME_HOST_NOT_LIVE;
    if (!m->group(group)) return LLME_HOST_BAD_ARGUMENT;
    return static_cast<int>(r->tables[static_cast<size_t>(group)].size());
}
// Entries [lo, hi) of a request's block table, to out[0 .. hi - lo); entries past the table's end
// read as -1. Returns the table's length.
int llme_cm_table_copy(void* h, int64_t key, int group, int lo, int hi, int* out) {
    auto* m = static_cast<CacheManager*>(h);
    auto* r = m->find(key);
    if (!r) return LLME_HOST_NOT_LIVE;
    if (!m->group(group) || lo < 0 || hi < lo) return LLME_HOST_BAD_ARGUMENT;
    const std::vector<int>& t = r->tables[static_cast<size_t>(group)];
    for (int b = lo; b < hi; ++b) out[b - lo] = b < static_cast<int>(t.size()) ? t[static_cast<size_t>(b)] : -1;
    return static_cast<int>(t.size());
}
int llme_cm_free_pages(void* h, int group) {
    auto* g = static_cast<CacheManager*>(h)->group(group);
    return g ? g->pool.free_pages() : LLME_HOST_BAD_ARGUMENT;
}
int llme_cm_num_pages(void* h, int group) {
    auto* g = static_cast<CacheManager*>(h)->group(group);
    return g ? g->pool.num_pages() : LLME_HOST_BAD_ARGUMENT;
}
int llme_cm_check(void* h) { return static_cast<CacheManager*>(h)->check(); }

// A step of one new token per request, in one call: the requests' lengths, and a page for each
// new token where it starts a page (all or none). max_length > 0: no request may become longer
// than that; if one would, nothing is reserved and the call returns 2 (the lengths are filled in).
// Returns 1, 0 (pools short, nothing changed), 2 or an error code.
int llme_cm_decode_begin(void* h, int S, const int64_t* keys, int* lengths, long max_length) {
    auto* m = static_cast<CacheManager*>(h);
    std::vector<long> ones(static_cast<size_t>(S), 1);
    bool too_long = false;
    for (int i = 0; i < S; ++i) {
        auto* r = m->find(keys[i]);
        if (!r) return LLME_HOST_NOT_LIVE;
        lengths[i] = static_cast<int>(r->length);
        if (max_length > 0 && r->length + 1 > max_length) too_long = true;
    }
    if (too_long) return 2;
    return m->reserve_batch(S, keys, ones.data());
}
// commit for several requests: n_new tokens each
int llme_cm_commit_batch(void* h, int S, const int64_t* keys, long n_new) {
    auto* m = static_cast<CacheManager*>(h);
    for (int i = 0; i < S; ++i) {
        const int rc = m->commit(keys[i], n_new);
        if (rc != 0) return rc;
    }
    return 0;
}

// What a recorded decode step needs before every replay, in one call: for each of the S requests
// its length (the new token's position) and slot, and into the block tables of every group
// (rows of `width` entries, group after group) the entries [done, blocks) that are not there
// yet; window groups are written whole (their early entries turn into -1 over time). The caller
// keeps serials[i] and done[g * S + i] between calls (both start at 0): a request in place i
// that is not the one of the last call (another key, or the same key admitted anew) has its
// rows written from their start. Returns 0 or an error code.
int llme_cm_fill_decode(void* h, int S, const int64_t* keys, int width, int* lengths, int* slots, int* tables,
                        int* done, int64_t* serials) {
    auto* m = static_cast<CacheManager*>(h);
    const int G = m->num_groups();
    for (int i = 0; i < S; ++i) {
        auto* r = m->find(keys[i]);
        if (!r) return LLME_HOST_NOT_LIVE;
        lengths[i] = static_cast<int>(r->length);
        slots[i] = r->slot;
        const bool same = serials[i] == r->serial;
        serials[i] = r->serial;
        for (int g = 0; g < G; ++g) {
            const std::vector<int>& t = r->tables[static_cast<size_t>(g)];
            const int nb = static_cast<int>(std::min<size_t>(t.size(), static_cast<size_t>(width)));
            int* row = tables + (static_cast<size_t>(g) * S + i) * width;
            int& d = done[g * S + i];
            const int lo = (m->group(g)->window || !same) ? 0 : std::min(d, nb);
            for (int b = lo; b < nb; ++b) row[b] = t[static_cast<size_t>(b)];
            d = nb;
        }
    }
    return 0;
}

// Tokens cached for each of S live requests. Returns 0 or an error code.
int llme_cm_lengths(void* h, int S, const int64_t* keys, long* out) {
    auto* m = static_cast<CacheManager*>(h);
    for (int i = 0; i < S; ++i) {
        auto* r = m->find(keys[i]);
        if (!r) return LLME_HOST_NOT_LIVE;
        out[i] = r->length;
    }
    return 0;
}

// The integer arrays of a step of any kind, for S requests that bring new_lens[i] tokens each: the
// tokens' positions and request indices (T = sum of new_lens values each), the first row of every
// request (S + 1), the tokens cached before the step (S), the slots (S), and for every group the rows
// of the block table, `width` entries each (entries behind a request's last page are 0; pages of a
// window group that were given back stay -1: no token of the step reads them). The arrays are
// written in the caller's one buffer at the given places. Returns the highest position of the
// step, or an error code (negative).
long llme_cm_fill_step(void* h, int S, const int64_t* keys, const int* new_lens, int width, int* positions,
                       int* seq_idx, int* q_start, int* ctx_len, int* slots, int* tables) {
    auto* m = static_cast<CacheManager*>(h);
    const int G = m->num_groups();
    long row = 0, top = -1;
    for (int i = 0; i < S; ++i) {
        auto* r = m->find(keys[i]);
        if (!r) return LLME_HOST_NOT_LIVE;
        const int n = new_lens[i];
        if (n <= 0) return LLME_HOST_BAD_ARGUMENT;
        const long c = r->length;
        q_start[i] = static_cast<int>(row);
        ctx_len[i] = static_cast<int>(c);
        slots[i] = r->slot;
        for (int t = 0; t < n; ++t) {
            positions[row + t] = static_cast<int>(c + t);
            seq_idx[row + t] = i;
        }
        row += n;
        top = std::max(top, c + n - 1);
        for (int g = 0; g < G; ++g) {
            const std::vector<int>& t = r->tables[static_cast<size_t>(g)];
            const int nb = static_cast<int>(std::min<size_t>(t.size(), static_cast<size_t>(width)));
            int* out = tables + (static_cast<size_t>(g) * S + i) * width;
            for (int b = 0; b < nb; ++b) out[b] = t[static_cast<size_t>(b)];
            for (int b = nb; b < width; ++b) out[b] = 0;
        }
    }
    q_start[S] = static_cast<int>(row);
    return top;
}

}  // extern "C"
