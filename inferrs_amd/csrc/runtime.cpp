// The host runtime: cache manager, step assembly and scheduler, in plain C++ behind a C interface.
//
// Cache manager.  Addressing and pool discipline follow the reference's BlockPool and BlockTable
// (inferrs-models/src/kv_cache.rs:80-140, :154-222): a page holds page_size token slots,
// slot = table[pos / page_size] * page_size + pos % page_size; free pages form a FIFO (taken from
// the front, given back to the back), so the physical layout of a replayed trace is
// deterministic.  Beyond the reference: reservation is all-or-nothing over all groups of layers,
// groups with a window give pages back once the window has passed them, and every request owns a
// slot in the arrays of fixed-size per-request state.
//
// Scheduler.  The reference's loop (inferrs/src/engine.rs:1380-1912) admits from a FIFO while fewer
// than max_batch_size requests are active, runs whole prompts, then one forward per request per
// round, and fails a request that finds no free block ("paged attention: out of KV blocks",
// engine.rs:2093-2095).  Here one step serves all running requests: decodes first, then portions
// of prompts (oldest first) under the token budget, then admissions in arrival order; when pages
// run out the most recently admitted request is preempted and recomputed later.
#include "runtime.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <memory>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

// ---- pools ----------------------------------------------------------------------------------
struct PagePool {
    int num_pages = 0;
    std::deque<int> free_;
    std::vector<int> refs;

    explicit PagePool(int n) : num_pages(n), refs(n, 0) {
        for (int i = 0; i < n; ++i) free_.push_back(i);
    }
    int num_free() const { return (int)free_.size(); }
    // n pages from the front of the free list, or false (and nothing taken)
    bool allocate(int n, std::vector<int>& out) {
        if ((int)free_.size() < n) return false;
        for (int i = 0; i < n; ++i) {
            const int p = free_.front();
            free_.pop_front();
            refs[p] = 1;
            out.push_back(p);
        }
        return true;
    }
    int release(int p) {
        if (p < 0 || p >= num_pages) return fail(IAR_ERROR, "page %d does not belong to this pool of %d", p, num_pages);
        if (refs[p] <= 0) return fail(IAR_ERROR, "page %d freed twice", p);
        if (--refs[p] == 0) free_.push_back(p);
        return 0;
    }
};

struct SlotPool {
    std::vector<char> held;
    explicit SlotPool(int n) : held(n, 0) {}
    int num_free() const { return (int)std::count(held.begin(), held.end(), 0); }
    int allocate() {                                  // lowest free id first
        for (size_t i = 0; i < held.size(); ++i)
            if (!held[i]) { held[i] = 1; return (int)i; }
        return -1;
    }
    int release(int s) {
        if (s < 0 || s >= (int)held.size() || !held[s]) return fail(IAR_ERROR, "state slot %d freed twice or never held", s);
        held[s] = 0;
        return 0;
    }
};

struct Sequence {
    int64_t key = 0;
    int length = 0;       // tokens whose keys are cached
    int reserved = 0;     // tokens reserved beyond length
    int state_slot = -1;
    std::vector<std::vector<int>> tables;             // group -> logical page -> physical page
};

struct Group {
    int window;           // < 0: all keys
    PagePool pool;
    Group(int w, int pages) : window(w), pool(pages) {}
};

struct Cache {
    int page_size, max_seqs;
    std::vector<Group> groups;
    SlotPool slots;
    std::unordered_map<int64_t, Sequence> seqs;

    Cache(int ps, int ms) : page_size(ps), max_seqs(ms), slots(ms) {}

    Sequence* find(int64_t key) {
        auto it = seqs.find(key);
        return it == seqs.end() ? nullptr : &it->second;
    }
    int pages_for(int length) const { return (length + page_size - 1) / page_size; }
    void pages_needed(const Sequence& s, int n_new, std::vector<int>& out) const {
        const int total = pages_for(s.length + s.reserved + n_new);
        out.resize(groups.size());
        for (size_t g = 0; g < groups.size(); ++g) out[g] = std::max(0, total - (int)s.tables[g].size());
    }
    int reserve(Sequence& s, int n_new) {
        std::vector<int> need;
        pages_needed(s, n_new, need);
        for (size_t g = 0; g < groups.size(); ++g)
            if (need[g] > groups[g].pool.num_free()) return IAR_NO_PAGES;
        for (size_t g = 0; g < groups.size(); ++g) groups[g].pool.allocate(need[g], s.tables[g]);
        s.reserved += n_new;
        return 0;
    }
    bool can_reserve(int n, const int64_t* keys, const int* n_new) {
        std::vector<int> want(groups.size(), 0), need;
        for (int i = 0; i < n; ++i) {
            Sequence* s = find(keys[i]);
            if (!s) return false;
            pages_needed(*s, n_new[i], need);
            for (size_t g = 0; g < groups.size(); ++g) want[g] += need[g];
        }
        for (size_t g = 0; g < groups.size(); ++g)
            if (want[g] > groups[g].pool.num_free()) return false;
        return true;
    }
    int commit(Sequence& s, int n_new) {
        if (n_new > s.reserved) return fail(IAR_ERROR, "commit of %d tokens but %d reserved", n_new, s.reserved);
        s.length += n_new;
        s.reserved -= n_new;
        for (size_t g = 0; g < groups.size(); ++g) {
            const int w = groups[g].window;
            if (w < 0) continue;
            // the next query sits at position length and reads keys > length - w
            const int first_needed = std::max(0, s.length - w + 1);
            std::vector<int>& table = s.tables[g];
            const int upto = std::min(first_needed / page_size, (int)table.size());
            for (int i = 0; i < upto; ++i)
                if (table[i] != IAR_RELEASED) {
                    if (groups[g].pool.release(table[i])) return IAR_ERROR;
                    table[i] = IAR_RELEASED;
                }
        }
        return 0;
    }
    int free_sequence(int64_t key) {
        auto it = seqs.find(key);
        if (it == seqs.end()) return fail(IAR_ERROR, "request is not live");
        Sequence& s = it->second;
        for (size_t g = 0; g < groups.size(); ++g)
            for (int p : s.tables[g])
                if (p != IAR_RELEASED && groups[g].pool.release(p)) return IAR_ERROR;
        if (slots.release(s.state_slot)) return IAR_ERROR;
        seqs.erase(it);
        return 0;
    }
    int add_sequence(int64_t key) {
        if (seqs.count(key)) return fail(IAR_ERROR, "request is already live");
        const int slot = slots.allocate();
        if (slot < 0) return fail(IAR_ERROR, "all %d request slots are in use", max_seqs);
        Sequence s;
        s.key = key;
        s.state_slot = slot;
        s.tables.resize(groups.size());
        seqs.emplace(key, std::move(s));
        return slot;
    }
    int min_total_pages() const {
        int m = 1 << 30;
        for (const Group& g : groups) m = std::min(m, g.pool.num_pages);
        return m;
    }
};

// ---- scheduler ------------------------------------------------------------------------------
enum { WAITING = 0, RUNNING = 1, FINISHED = 2 };

struct Req {
    int64_t key = 0;
    std::vector<int> tokens;      // prompt, then output
    int n_prompt = 0;
    int computed = 0;             // tokens whose keys and values are in the cache
    int status = WAITING;
    int max_tokens = 0;
    bool bypass_stop = false;
    std::vector<int> extra_stop;
    int preemptions = 0;
    std::string error;
    int total() const { return (int)tokens.size(); }
    int n_output() const { return (int)tokens.size() - n_prompt; }
};

struct PlanEntry { Req* req; int start, count; bool samples; };

struct Sched {
    Cache* cache;
    int max_batch_size, max_tokens_per_step, prefill_chunk, max_seq_len;
    int row_multiple = 0;                 // > 1: a portion that does not end its prompt is cut so that the step's tokens are a multiple of this
    std::unordered_set<int> stop_ids;
    std::unordered_map<int64_t, std::unique_ptr<Req>> reqs;
    std::deque<Req*> waiting;
    std::vector<Req*> running;    // in order of admission
    std::vector<PlanEntry> plan;
    std::vector<int64_t> preempted, failed;
    bool broken = false;          // the last plan met a misuse; the message is in the error channel
    std::unordered_set<int64_t> left_out;   // decodes that found no budget in the last plan: served first in the next

    bool is_running(const Req* r) const { return std::find(running.begin(), running.end(), r) != running.end(); }
    bool fits_alone(int n_tokens) const {
        return cache->groups.empty() || cache->pages_for(n_tokens) <= cache->min_total_pages();
    }
    Req* preempt_latest(const Req* exclude) {
        for (int i = (int)running.size() - 1; i >= 0; --i) {
            Req* v = running[i];
            if (v == exclude) continue;
            running.erase(running.begin() + i);
            cache->free_sequence(v->key);
            v->computed = 0;
            v->status = WAITING;
            v->preemptions += 1;
            waiting.push_front(v);
            return v;
        }
        return nullptr;
    }
    void fail_request(Req* r, const std::string& message, bool live) {
        if (live) {
            auto it = std::find(running.begin(), running.end(), r);
            if (it != running.end()) running.erase(it);
            if (cache->find(r->key)) cache->free_sequence(r->key);
        }
        r->status = FINISHED;
        r->error = message;
        failed.push_back(r->key);
    }
    void drop_entries_of(const Req* v, int& budget) {
        for (size_t i = 0; i < plan.size();)
            if (plan[i].req == v) { budget += plan[i].count; plan.erase(plan.begin() + i); }
            else ++i;
    }
    // The tokens of a request that this step takes, given what it has left to feed and what the step's budget still
    // allows.  The large products tile a step's rows (256 at a time in the vendor's GEMM: a step of 520 rows costs as
    // much as one of 768), so a portion that is cut anyway is cut where the step's tokens so far make a whole
    // multiple of `row_multiple`; a portion that ends its prompt is what it is.
    int portion(int left, int budget) const {
        int n = std::min(std::min(left, prefill_chunk), budget);
        if (row_multiple > 1 && n < left) {
            const int rows = max_tokens_per_step - budget + n;
            const int over = rows % row_multiple;
            if (over != 0 && rows - over >= row_multiple && n - over >= 1) n -= over;
        }
        return n;
    }
    void make_plan(bool fresh) {
        if (fresh) { plan.clear(); preempted.clear(); failed.clear(); broken = false; }
        plan.clear();
        int budget = max_tokens_per_step;
        const size_t failed_before = failed.size(), preempted_before = preempted.size();
        char buf[256];

        // 1. decodes: running requests with exactly one token left to feed
        std::vector<Req*> decoding;
        for (Req* r : running)
            if (r->total() - r->computed == 1 && r->n_output() > 0) decoding.push_back(r);
        // (a budget smaller than the number of decoding requests must not starve the late ones: whoever was
        // left out last time goes first, in admission order, then the others)
        std::stable_partition(decoding.begin(), decoding.end(), [&](Req* r) { return left_out.count(r->key) != 0; });
        left_out.clear();
        for (Req* r : decoding) {
            if (!is_running(r)) continue;                 // preempted while serving an earlier one
            if (budget < 1) { left_out.insert(r->key); continue; }
            bool ok = true;
            while (cache->reserve(*cache->find(r->key), 1) != 0) {
                Req* victim = preempt_latest(r);
                if (!victim) {
                    // it holds every page there is and needs one more: it cannot go on
                    snprintf(buf, sizeof(buf), "paged attention: out of KV blocks at position %d", r->computed);
                    fail_request(r, buf, true);
                    ok = false;
                    break;
                }
                preempted.push_back(victim->key);
                drop_entries_of(victim, budget);
            }
            if (ok) {
                plan.push_back({r, r->total() - 1, 1, true});
                budget -= 1;
            }
        }
        // 2. portions of prompts of running requests, oldest first
        std::vector<Req*> snapshot = running;
        for (Req* r : snapshot) {
            if (budget < 1) break;
            bool planned = false;
            for (const PlanEntry& e : plan) planned |= e.req == r;
            const int left = r->total() - r->computed;
            if (planned || left < 1) continue;
            if (left == 1 && r->n_output() > 0) continue;          // a decode that found no budget
            const int n = portion(left, budget);
            if (cache->reserve(*cache->find(r->key), n) != 0) continue;   // waits for pages
            plan.push_back({r, r->computed, n, r->computed + n == r->total()});
            budget -= n;
        }
        // 3. admissions, in arrival order
        while (!waiting.empty() && budget >= 1 && (int)running.size() < max_batch_size) {
            Req* r = waiting.front();
            if (!fits_alone(r->total() + 1)) {
                waiting.pop_front();
                snprintf(buf, sizeof(buf), "paged attention: out of KV blocks: the request needs %d pages, the pool has %d",
                         cache->pages_for(r->total() + 1), cache->min_total_pages());
                fail_request(r, buf, false);
                continue;
            }
            const int n = portion(r->total() - r->computed, budget);
            if (cache->add_sequence(r->key) < 0) {        // the key is in use outside this scheduler, or no slot is left
                broken = true;
                break;
            }
            // admitted only when all it has so far, and one token more, would fit now: a request that
            // is let in on its first portion alone tends to be preempted later
            const int all = r->total() + 1;
            if (!cache->can_reserve(1, &r->key, &all) || cache->reserve(*cache->find(r->key), n) != 0) {
                cache->free_sequence(r->key);
                break;                                    // no pages now: it stays first in line
            }
            waiting.pop_front();
            r->status = RUNNING;
            running.push_back(r);
            plan.push_back({r, r->computed, n, r->computed + n == r->total()});
            budget -= n;
        }
        if (broken) return;
        if (plan.empty() && !running.empty() && failed.size() == failed_before && preempted.size() == preempted_before) {
            // every running request waits for pages that nobody will free: preempt the latest so that
            // the oldest can go on
            Req* victim = preempt_latest(running.front());
            if (victim) {
                preempted.push_back(victim->key);
                make_plan(false);
                return;
            }
            Req* r = running.front();
            snprintf(buf, sizeof(buf), "paged attention: out of KV blocks at position %d", r->computed);
            fail_request(r, buf, true);
        }
    }
    // -1: goes on; 0: stop; 1: length  (check_stop of the reference, inferrs/src/engine.rs:866-887)
    int stop_reason(const Req* r, int token) const {
        if (!r->bypass_stop && (stop_ids.count(token) ||
                                std::find(r->extra_stop.begin(), r->extra_stop.end(), token) != r->extra_stop.end()))
            return 0;
        if (r->n_output() >= r->max_tokens) return 1;
        if (r->total() >= max_seq_len) return 1;
        return -1;
    }
    // one entry ran: returns the finish reason or -1
    int advance(Req* r, int count, bool samples, int token) {
        Sequence* s = cache->find(r->key);
        if (!s || cache->commit(*s, count)) return -2;
        r->computed += count;
        if (!samples) return -1;
        r->tokens.push_back(token);
        const int reason = stop_reason(r, token);
        if (reason >= 0) {
            r->status = FINISHED;
            auto it = std::find(running.begin(), running.end(), r);
            if (it != running.end()) running.erase(it);
            cache->free_sequence(r->key);
        }
        return reason;
    }
};

Cache* C(void* p) { return (Cache*)p; }
Sched* S(void* p) { return (Sched*)p; }

}  // namespace

extern "C" {

const char* iar_last_error(void) { return g_error; }
int iar_abi_version(void) { return IAR_ABI_VERSION; }

// ---- cache manager --------------------------------------------------------------------------
void* iar_cache_create(int page_size, int max_seqs, int n_groups, const int* windows, const int* num_pages) {
    if (page_size < 1) { fail(IAR_ERROR, "page_size must be >= 1, got %d", page_size); return nullptr; }
    if (max_seqs < 1) { fail(IAR_ERROR, "max_seqs must be >= 1, got %d", max_seqs); return nullptr; }
    for (int g = 0; g < n_groups; ++g)
        if (num_pages[g] < 0) { fail(IAR_ERROR, "num_pages must be >= 0, got %d", num_pages[g]); return nullptr; }
    Cache* c = new Cache(page_size, max_seqs);
    for (int g = 0; g < n_groups; ++g) c->groups.emplace_back(windows[g], num_pages[g]);
    return c;
}
void iar_cache_destroy(void* cache) { delete C(cache); }
int iar_cache_add_sequence(void* cache, int64_t key) { return C(cache)->add_sequence(key); }
int iar_cache_free_sequence(void* cache, int64_t key) { return C(cache)->free_sequence(key); }
int iar_cache_has_sequence(void* cache, int64_t key) { return C(cache)->find(key) ? 1 : 0; }
int iar_cache_num_sequences(void* cache) { return (int)C(cache)->seqs.size(); }

#define SEQ_OR_FAIL(s, cache, key)                                          \
    Sequence* s = C(cache)->find(key);                                      \
    if (!s) return fail(IAR_ERROR, "request is not live")

int iar_cache_length(void* cache, int64_t key) { SEQ_OR_FAIL(s, cache, key); return s->length; }
int iar_cache_reserved(void* cache, int64_t key) { SEQ_OR_FAIL(s, cache, key); return s->reserved; }
int iar_cache_state_slot(void* cache, int64_t key) { SEQ_OR_FAIL(s, cache, key); return s->state_slot; }
int iar_cache_reserve(void* cache, int64_t key, int n_new) {
    if (n_new < 0) return fail(IAR_ERROR, "cannot reserve %d tokens", n_new);
    SEQ_OR_FAIL(s, cache, key);
    return C(cache)->reserve(*s, n_new);
}
int iar_cache_can_reserve(void* cache, int n, const int64_t* keys, const int* n_new) {
    return C(cache)->can_reserve(n, keys, n_new) ? 1 : 0;
}
int iar_cache_commit(void* cache, int64_t key, int n_new) { SEQ_OR_FAIL(s, cache, key); return C(cache)->commit(*s, n_new); }
int iar_cache_count_live(void* cache, int n, const int64_t* keys) {
    int live = 0;
    for (int i = 0; i < n; ++i) live += C(cache)->find(keys[i]) != nullptr;
    return live;
}
int iar_cache_max_length(void* cache, int n, const int64_t* keys) {
    int longest = 0;
    for (int i = 0; i < n; ++i) {
        SEQ_OR_FAIL(s, cache, keys[i]);
        longest = std::max(longest, s->length);
    }
    return longest;
}
int iar_cache_ensure_reserved(void* cache, int n, const int64_t* keys, const int* n_tokens) {
    Cache* c = C(cache);
    std::vector<int> more(n);
    for (int i = 0; i < n; ++i) {
        SEQ_OR_FAIL(s, cache, keys[i]);
        more[i] = std::max(0, n_tokens[i] - s->reserved);
    }
    if (!c->can_reserve(n, keys, more.data())) return IAR_NO_PAGES;
    for (int i = 0; i < n; ++i)
        if (more[i] && c->reserve(*c->find(keys[i]), more[i])) return fail(IAR_ERROR, "pages vanished between the check and the reservation");
    return 0;
}
int iar_cache_commit_many(void* cache, int n, const int64_t* keys, const int* n_new) {
    for (int i = 0; i < n; ++i) {
        SEQ_OR_FAIL(s, cache, keys[i]);
        if (C(cache)->commit(*s, n_new[i])) return IAR_ERROR;
    }
    return 0;
}
int iar_cache_table_size(void* cache, int64_t key, int group) {
    SEQ_OR_FAIL(s, cache, key);
    if (group < 0 || group >= (int)s->tables.size()) return fail(IAR_ERROR, "no group %d", group);
    return (int)s->tables[group].size();
}
int iar_cache_table(void* cache, int64_t key, int group, int* out, int capacity) {
    SEQ_OR_FAIL(s, cache, key);
    if (group < 0 || group >= (int)s->tables.size()) return fail(IAR_ERROR, "no group %d", group);
    const int n = std::min(capacity, (int)s->tables[group].size());
    std::copy(s->tables[group].begin(), s->tables[group].begin() + n, out);
    return n;
}
int iar_cache_set_table(void* cache, int64_t key, int group, const int* pages, int n) {
    SEQ_OR_FAIL(s, cache, key);
    if (group < 0 || group >= (int)s->tables.size()) return fail(IAR_ERROR, "no group %d", group);
    s->tables[group].assign(pages, pages + n);
    return 0;
}
int iar_cache_slot_ids(void* cache, int64_t key, int group, int start, int n, int* out) {
    SEQ_OR_FAIL(s, cache, key);
    if (group < 0 || group >= (int)s->tables.size()) return fail(IAR_ERROR, "no group %d", group);
    const int ps = C(cache)->page_size;
    const std::vector<int>& table = s->tables[group];
    for (int i = 0; i < n; ++i) {
        const int pos = start + i;
        if (pos / ps >= (int)table.size()) return fail(IAR_ERROR, "position %d lies beyond the request's pages", pos);
        const int page = table[pos / ps];
        if (page == IAR_RELEASED) return fail(IAR_ERROR, "position %d lies in a released page", pos);
        out[i] = page * ps + pos % ps;
    }
    return 0;
}
int iar_cache_num_free(void* cache, int group) { return C(cache)->groups[group].pool.num_free(); }
int iar_cache_num_pages(void* cache, int group) { return C(cache)->groups[group].pool.num_pages; }
int iar_cache_free_slots(void* cache) { return C(cache)->slots.num_free(); }
int iar_cache_pool_allocate(void* cache, int group, int n, int* out) {
    if (n < 0) return fail(IAR_ERROR, "cannot allocate %d pages", n);
    std::vector<int> got;
    if (!C(cache)->groups[group].pool.allocate(n, got)) return IAR_NO_PAGES;
    std::copy(got.begin(), got.end(), out);
    return n;
}
int iar_cache_pool_free(void* cache, int group, const int* pages, int n) {
    for (int i = 0; i < n; ++i)
        if (C(cache)->groups[group].pool.release(pages[i])) return IAR_ERROR;
    return 0;
}
int iar_cache_slot_allocate(void* cache) {
    const int s = C(cache)->slots.allocate();
    return s < 0 ? IAR_NO_PAGES : s;
}
int iar_cache_slot_free(void* cache, int slot) { return C(cache)->slots.release(slot); }
int iar_cache_check_invariants(void* cache) {
    Cache* c = C(cache);
    for (size_t g = 0; g < c->groups.size(); ++g) {
        const PagePool& pool = c->groups[g].pool;
        std::vector<int> seen(pool.num_pages, 0);
        int held = 0;
        for (const auto& kv : c->seqs)
            for (int p : kv.second.tables[g]) {
                if (p == IAR_RELEASED) continue;
                if (p < 0 || p >= pool.num_pages) return fail(IAR_ERROR, "group %d: a table holds page %d of %d", (int)g, p, pool.num_pages);
                if (seen[p]++) return fail(IAR_ERROR, "group %d: page %d is held twice", (int)g, p);
                if (pool.refs[p] != 1) return fail(IAR_ERROR, "group %d: page %d is in a table but the pool counts %d holders", (int)g, p, pool.refs[p]);
                ++held;
            }
        std::vector<int> on_list(pool.num_pages, 0);
        for (int p : pool.free_) {
            if (on_list[p]++) return fail(IAR_ERROR, "group %d: page %d is on the free list twice", (int)g, p);
            if (seen[p]) return fail(IAR_ERROR, "group %d: page %d is free and held", (int)g, p);
        }
        int pool_held = 0;
        for (int r : pool.refs) pool_held += r > 0;
        if (pool_held != held) return fail(IAR_ERROR, "group %d: tables hold %d pages, the pool says %d", (int)g, held, pool_held);
        if ((int)pool.free_.size() + held != pool.num_pages)
            return fail(IAR_ERROR, "group %d: %d free + %d held != %d", (int)g, (int)pool.free_.size(), held, pool.num_pages);
    }
    std::vector<int> slot_seen(c->max_seqs, 0);
    for (const auto& kv : c->seqs)
        if (slot_seen[kv.second.state_slot]++) return fail(IAR_ERROR, "state slot %d is held twice", kv.second.state_slot);
    return 0;
}

// ---- step assembly --------------------------------------------------------------------------
long long iar_step_words(void* cache, int n_entries, const int64_t* keys, const int* q_lens, int n_want,
                         int pad_pages, int advance) {
    Cache* c = C(cache);
    long long n = 0;
    int max_pages = 1;
    for (int i = 0; i < n_entries; ++i) {
        Sequence* s = c->find(keys[i]);
        if (!s) return fail(IAR_ERROR, "request is not live");
        n += q_lens[i];
        max_pages = std::max(max_pages, c->pages_for(s->length + advance + q_lens[i]));
    }
    if (pad_pages > 0) max_pages = std::max(max_pages, pad_pages);
    return 3 * n + (n_entries + 1) + n_entries + n_want + (long long)c->groups.size() * (n + (long long)n_entries * max_pages);
}

int iar_build_step(void* cache, int n_entries, const int64_t* keys, const int* q_lens, const int* tokens,
                   const int* want_counts, const int* want, int pad_pages, int advance, int32_t* out,
                   long long capacity, int* meta, int* order_out) {
    Cache* c = C(cache);
    const int ps = c->page_size;
    const int n_groups = (int)c->groups.size();
    if (n_entries < 1) return fail(IAR_ERROR, "a step needs at least one entry");
    // single-token requests first, in their order; the others after them
    std::vector<int> order;
    order.reserve(n_entries);
    for (int pass = 0; pass < 2; ++pass)
        for (int i = 0; i < n_entries; ++i)
            if ((q_lens[i] == 1) == (pass == 0)) order.push_back(i);
    std::vector<int> rank(n_entries), tok_off(n_entries + 1, 0), want_off(n_entries + 1, 0);
    for (int i = 0; i < n_entries; ++i) {
        rank[order[i]] = i;
        tok_off[i + 1] = tok_off[i] + q_lens[i];
        want_off[i + 1] = want_off[i] + want_counts[i];
    }
    std::vector<Sequence*> seqs(n_entries);
    std::vector<int> starts(n_entries), cu(n_entries + 1, 0);
    int n = 0, max_pages = 1, max_q = 0, max_kv = 0, n_single = 0, kv_single = 0, kv_multi = 0;
    for (int j = 0; j < n_entries; ++j) {
        const int i = order[j];
        if (q_lens[i] < 1) return fail(IAR_ERROR, "a step entry needs at least one token");
        seqs[j] = c->find(keys[i]);
        if (!seqs[j]) return fail(IAR_ERROR, "request is not live");
        starts[j] = seqs[j]->length + advance;
        cu[j + 1] = cu[j] + q_lens[i];
        n += q_lens[i];
        const int end = starts[j] + q_lens[i];
        max_pages = std::max(max_pages, c->pages_for(end));
        max_q = std::max(max_q, q_lens[i]);
        max_kv = std::max(max_kv, end);
        if (q_lens[i] == 1) { ++n_single; kv_single = std::max(kv_single, end); }
        else kv_multi = std::max(kv_multi, end);
    }
    if (pad_pages > 0) {
        if (pad_pages < max_pages) return fail(IAR_ERROR, "block tables of %d pages are too narrow for %d", pad_pages, max_pages);
        max_pages = pad_pages;
        max_kv = std::max(max_kv, pad_pages * ps);
        if (n_single) kv_single = std::max(kv_single, pad_pages * ps);
        if (n_single < n_entries) kv_multi = std::max(kv_multi, pad_pages * ps);
    }
    const int n_want = want_off[n_entries];
    const long long total = 3LL * n + (n_entries + 1) + n_entries + n_want + (long long)n_groups * (n + (long long)n_entries * max_pages);
    if (total > capacity) return fail(IAR_ERROR, "the step needs %lld words, the buffer has %lld", total, capacity);
    int32_t* token_ids = out;
    int32_t* positions = token_ids + n;
    int32_t* token_seq = positions + n;
    int32_t* cu_out = token_seq + n;
    int32_t* state_slots = cu_out + n_entries + 1;
    int32_t* want_rows = state_slots + n_entries;
    int32_t* rest = want_rows + n_want;
    for (int j = 0; j < n_entries; ++j) {
        const int i = order[j];
        for (int t = 0; t < q_lens[i]; ++t) {
            token_ids[cu[j] + t] = tokens[tok_off[i] + t];
            positions[cu[j] + t] = starts[j] + t;
            token_seq[cu[j] + t] = j;
        }
        cu_out[j] = cu[j];
        state_slots[j] = seqs[j]->state_slot;
        order_out[j] = i;
    }
    cu_out[n_entries] = n;
    for (int i = 0, w = 0; i < n_entries; ++i)
        for (int k = 0; k < want_counts[i]; ++k, ++w) {
            const int at = want[want_off[i] + k];
            if (at < 0 || at >= q_lens[i]) return fail(IAR_ERROR, "a wanted place %d lies outside its entry's %d tokens", at, q_lens[i]);
            want_rows[w] = cu[rank[i]] + at;
        }
    for (int g = 0; g < n_groups; ++g) {
        int32_t* slots = rest;
        int32_t* table = slots + n;
        rest = table + (long long)n_entries * max_pages;
        std::memset(table, 0, sizeof(int32_t) * (size_t)n_entries * max_pages);
        for (int j = 0; j < n_entries; ++j) {
            const int i = order[j];
            const std::vector<int>& t = seqs[j]->tables[g];
            const int need = c->pages_for(starts[j] + q_lens[i]);
            if ((int)t.size() < need)
                return fail(IAR_ERROR, "a request holds %d pages, too few for %d tokens", (int)t.size(), starts[j] + q_lens[i]);
            for (int q = 0; q < q_lens[i]; ++q) {
                const int pos = starts[j] + q;
                const int page = t[pos / ps];
                if (page == IAR_RELEASED) return fail(IAR_ERROR, "a new token falls into a page that was already released");
                slots[cu[j] + q] = page * ps + pos % ps;
            }
            const int copy = std::min((int)t.size(), max_pages);
            for (int q = 0; q < copy; ++q) table[(long long)j * max_pages + q] = t[q] < 0 ? 0 : t[q];   // (a released entry names page 0: kernels that round a window's start down may load from it, and use nothing of it)
        }
    }
    meta[0] = (int)total; meta[1] = n; meta[2] = n_entries; meta[3] = n_want; meta[4] = max_pages; meta[5] = max_q;
    meta[6] = max_kv; meta[7] = n_single; meta[8] = kv_single; meta[9] = kv_multi; meta[10] = n_groups;
    return 0;
}

// ---- scheduler ------------------------------------------------------------------------------
void* iar_sched_create(void* cache, int max_batch_size, int max_tokens_per_step, int prefill_chunk,
                       int max_seq_len, const int* stop_ids, int n_stop) {
    if (max_batch_size < 1 || max_tokens_per_step < 1) { fail(IAR_ERROR, "max_batch_size and max_tokens_per_step must be >= 1"); return nullptr; }
    if (max_batch_size > C(cache)->max_seqs) {
        fail(IAR_ERROR, "max_batch_size %d exceeds the cache's %d request slots", max_batch_size, C(cache)->max_seqs);
        return nullptr;
    }
    if (prefill_chunk < 1) { fail(IAR_ERROR, "prefill_chunk must be >= 1"); return nullptr; }
    Sched* s = new Sched();
    s->cache = C(cache);
    s->max_batch_size = max_batch_size;
    s->max_tokens_per_step = max_tokens_per_step;
    s->prefill_chunk = prefill_chunk;
    s->max_seq_len = max_seq_len;
    for (int i = 0; i < n_stop; ++i) s->stop_ids.insert(stop_ids[i]);
    return s;
}
void iar_sched_destroy(void* sched) { delete S(sched); }
int iar_sched_set_row_multiple(void* sched, int row_multiple) {
    if (row_multiple < 0) return fail(IAR_ERROR, "row_multiple must be >= 0");
    S(sched)->row_multiple = row_multiple;
    return 0;
}

int iar_sched_add(void* sched, int64_t key, const int* prompt, int n_prompt, int max_tokens, int bypass_stop,
                  const int* extra_stop, int n_extra) {
    Sched* s = S(sched);
    if (n_prompt < 1) return fail(IAR_ERROR, "the prompt is empty");
    if (n_prompt >= s->max_seq_len) return fail(IAR_ERROR, "the prompt has %d tokens, the limit is %d", n_prompt, s->max_seq_len - 1);
    if (s->reqs.count(key)) return fail(IAR_ERROR, "a request of this key exists");
    std::unique_ptr<Req> r(new Req());
    r->key = key;
    r->tokens.assign(prompt, prompt + n_prompt);
    r->n_prompt = n_prompt;
    r->max_tokens = max_tokens;
    r->bypass_stop = bypass_stop != 0;
    r->extra_stop.assign(extra_stop, extra_stop + n_extra);
    s->waiting.push_back(r.get());
    s->reqs.emplace(key, std::move(r));
    return 0;
}
int iar_sched_adopt(void* sched, int64_t key, const int* tokens, int n_tokens, int n_prompt, int max_tokens,
                    int bypass_stop, const int* extra_stop, int n_extra) {
    Sched* s = S(sched);
    if (n_prompt < 1 || n_prompt > n_tokens) return fail(IAR_ERROR, "a request has at least one prompt token and no more than all its tokens");
    if (n_tokens >= s->max_seq_len) return fail(IAR_ERROR, "the request has %d tokens, the limit is %d", n_tokens, s->max_seq_len - 1);
    if (s->reqs.count(key)) return fail(IAR_ERROR, "a request of this key exists");
    Sequence* seq = s->cache->find(key);
    if (!seq) return fail(IAR_ERROR, "request is not live: only a request with a cache entry can be adopted");
    if (seq->length >= n_tokens) return fail(IAR_ERROR, "the cache holds %d tokens of the request's %d: at least one must be left to feed", seq->length, n_tokens);
    if ((int)s->running.size() >= s->max_batch_size) return fail(IAR_ERROR, "%d requests are running already", s->max_batch_size);
    std::unique_ptr<Req> r(new Req());
    r->key = key;
    r->tokens.assign(tokens, tokens + n_tokens);
    r->n_prompt = n_prompt;
    r->computed = seq->length;
    r->status = RUNNING;
    r->max_tokens = max_tokens;
    r->bypass_stop = bypass_stop != 0;
    r->extra_stop.assign(extra_stop, extra_stop + n_extra);
    s->running.push_back(r.get());
    s->reqs.emplace(key, std::move(r));
    return seq->length;
}
int iar_sched_num_waiting(void* sched) { return (int)S(sched)->waiting.size(); }
int iar_sched_num_running(void* sched) { return (int)S(sched)->running.size(); }
int iar_sched_waiting(void* sched, int64_t* out, int capacity) {
    int n = 0;
    for (Req* r : S(sched)->waiting) if (n < capacity) out[n++] = r->key;
    return n;
}
int iar_sched_running(void* sched, int64_t* out, int capacity) {
    int n = 0;
    for (Req* r : S(sched)->running) if (n < capacity) out[n++] = r->key;
    return n;
}
int iar_sched_plan(void* sched) {
    S(sched)->make_plan(true);
    if (S(sched)->broken) {
        // what was reserved for this plan's entries stays reserved: the caller has to end these requests
        std::string why = g_error;
        return fail(IAR_ERROR, "a waiting request cannot get a cache entry: %s", why.c_str());
    }
    return (int)S(sched)->plan.size();
}
int iar_sched_plan_entries(void* sched, int64_t* keys, int* starts, int* counts, int* samples) {
    const std::vector<PlanEntry>& p = S(sched)->plan;
    for (size_t i = 0; i < p.size(); ++i) {
        keys[i] = p[i].req->key; starts[i] = p[i].start; counts[i] = p[i].count; samples[i] = p[i].samples;
    }
    return (int)p.size();
}
int iar_sched_plan_tokens(void* sched, int entry, int* out, int capacity) {
    const std::vector<PlanEntry>& p = S(sched)->plan;
    if (entry < 0 || entry >= (int)p.size()) return fail(IAR_ERROR, "no entry %d in the plan", entry);
    const PlanEntry& e = p[entry];
    if (e.count > capacity) return fail(IAR_ERROR, "entry %d has %d tokens, the buffer %d", entry, e.count, capacity);
    std::copy(e.req->tokens.begin() + e.start, e.req->tokens.begin() + e.start + e.count, out);
    return e.count;
}
int iar_sched_plan_preempted(void* sched, int64_t* out, int capacity) {
    const std::vector<int64_t>& v = S(sched)->preempted;
    const int n = std::min(capacity, (int)v.size());
    std::copy(v.begin(), v.begin() + n, out);
    return (int)v.size();
}
int iar_sched_plan_failed(void* sched, int64_t* out, int capacity) {
    const std::vector<int64_t>& v = S(sched)->failed;
    const int n = std::min(capacity, (int)v.size());
    std::copy(v.begin(), v.begin() + n, out);
    return (int)v.size();
}
const char* iar_sched_failure(void* sched, int64_t key) {
    auto it = S(sched)->reqs.find(key);
    return it == S(sched)->reqs.end() ? "" : it->second->error.c_str();
}
int iar_sched_commit(void* sched, const int* sampled, int n_sampled, int64_t* finished, int* reasons, int capacity) {
    Sched* s = S(sched);
    int n_fin = 0, used = 0;
    std::vector<PlanEntry> plan = s->plan;             // advance() may touch `running`, not the plan; copy for safety
    for (const PlanEntry& e : plan) {
        int token = 0;
        if (e.samples) {
            if (used >= n_sampled) return fail(IAR_ERROR, "the plan samples more tokens than the %d given", n_sampled);
            token = sampled[used++];
        }
        const int reason = s->advance(e.req, e.count, e.samples, token);
        if (reason == -2) return IAR_ERROR;
        if (reason >= 0 && n_fin < capacity) { finished[n_fin] = e.req->key; reasons[n_fin] = reason; ++n_fin; }
    }
    s->plan.clear();
    return n_fin;
}
int iar_sched_commit_decode(void* sched, int n, const int64_t* keys, const int* tokens, int64_t* finished,
                            int* reasons, int capacity) {
    Sched* s = S(sched);
    int n_fin = 0;
    for (int i = 0; i < n; ++i) {
        auto it = s->reqs.find(keys[i]);
        if (it == s->reqs.end()) return fail(IAR_ERROR, "no such request");
        Req* r = it->second.get();
        if (r->status != RUNNING) continue;             // finished earlier in this run of steps
        const int reason = s->advance(r, 1, true, tokens[i]);
        if (reason == -2) return IAR_ERROR;
        if (reason >= 0 && n_fin < capacity) { finished[n_fin] = r->key; reasons[n_fin] = reason; ++n_fin; }
    }
    return n_fin;
}
int iar_sched_request_state(void* sched, int64_t key, int* out5) {
    auto it = S(sched)->reqs.find(key);
    if (it == S(sched)->reqs.end()) return fail(IAR_ERROR, "no such request");
    const Req& r = *it->second;
    out5[0] = r.computed; out5[1] = r.n_output(); out5[2] = r.status; out5[3] = r.preemptions; out5[4] = r.n_prompt;
    return 0;
}
int iar_sched_request_output(void* sched, int64_t key, int* out, int capacity) {
    auto it = S(sched)->reqs.find(key);
    if (it == S(sched)->reqs.end()) return fail(IAR_ERROR, "no such request");
    const Req& r = *it->second;
    const int n = std::min(capacity, r.n_output());
    std::copy(r.tokens.begin() + r.n_prompt, r.tokens.begin() + r.n_prompt + n, out);
    return r.n_output();
}
int iar_sched_finish(void* sched, int64_t key) {
    Sched* s = S(sched);
    auto it = s->reqs.find(key);
    if (it == s->reqs.end()) return fail(IAR_ERROR, "no such request");
    Req* r = it->second.get();
    if (r->status == FINISHED) return 0;
    auto w = std::find(s->waiting.begin(), s->waiting.end(), r);
    if (w != s->waiting.end()) s->waiting.erase(w);
    auto run = std::find(s->running.begin(), s->running.end(), r);
    if (run != s->running.end()) s->running.erase(run);
    if (s->cache->find(key) && s->cache->free_sequence(key)) return IAR_ERROR;
    int budget = 0;
    s->drop_entries_of(r, budget);
    r->status = FINISHED;
    return 0;
}
int iar_sched_forget(void* sched, int64_t key) {
    Sched* s = S(sched);
    auto it = s->reqs.find(key);
    if (it == s->reqs.end()) return 0;
    if (it->second->status != FINISHED) return fail(IAR_ERROR, "the request is not finished");
    s->reqs.erase(it);
    return 0;
}

}  // extern "C"
