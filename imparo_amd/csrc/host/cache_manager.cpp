// The host runtime: page pools, the cache manager and the packing of a step.
//
// Allocation takes the lowest free page, so which pages a request gets is a
// function of which pages are free and never of history; a page freed twice is
// an error. The reference's block allocator keeps the same two rules
// (/root/reference/crates/imparo-kv/src/alloc.rs:1-11,51-75). Page addressing
// follows its table form: position p lives in page table[p / page_size], slot
// p % page_size (/root/reference/crates/imparo-cuda/native/kv_paging.cuh:25-30).
#include "host_api.h"

#include <algorithm>
#include <cstring>
#include <functional>
#include <queue>
#include <unordered_map>
#include <vector>

struct ImparoPool {
    int n_pages = 0;
    int n_free = 0;
    int high_water = 0;
    std::vector<char> is_free;
    // min-heap of ranks; rank == page unless placement is scrambled
    std::priority_queue<int, std::vector<int>, std::greater<int>> heap;
    std::vector<int> place, rank;   // rank -> page, page -> rank (empty: identity)

    explicit ImparoPool(int n) : n_pages(n), n_free(n), is_free((size_t)n, 1) {
        for (int i = 0; i < n; ++i) heap.push(i);
    }
    int alloc() {
        if (n_free == 0) return IMPARO_E_OUT_OF_PAGES;
        int page = heap.top();
        heap.pop();
        if (!place.empty()) page = place[(size_t)page];
        is_free[(size_t)page] = 0;
        --n_free;
        high_water = std::max(high_water, page + 1);
        return page;
    }
    int free_page(int page) {
        if (page < 0 || page >= n_pages) return IMPARO_E_RANGE;
        if (is_free[(size_t)page]) return IMPARO_E_DOUBLE_FREE;
        is_free[(size_t)page] = 1;
        ++n_free;
        heap.push(rank.empty() ? page : rank[(size_t)page]);
        return 0;
    }
    int scramble(uint64_t seed) {
        if (n_free != n_pages) return IMPARO_E_BUSY;
        place.resize((size_t)n_pages);
        rank.resize((size_t)n_pages);
        for (int i = 0; i < n_pages; ++i) place[(size_t)i] = i;
        uint64_t s = seed * 0x9E3779B97F4A7C15ull + 0xD1342543DE82EF95ull;
        for (int i = n_pages - 1; i > 0; --i) {       // Fisher-Yates with a splitmix stream
            s += 0x9E3779B97F4A7C15ull;
            uint64_t z = s;
            z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
            z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
            z ^= z >> 31;
            std::swap(place[(size_t)i], place[(size_t)(z % (uint64_t)(i + 1))]);
        }
        for (int r = 0; r < n_pages; ++r) rank[(size_t)place[(size_t)r]] = r;
        return 0;
    }
};

struct Request {
    int slot = -1;
    int length = 0;
    std::vector<std::vector<int32_t>> tables;            // per group; -1 = behind the window, given back
    std::vector<std::pair<int, int32_t>> pending;        // (group, page) taken since the last commit
};

struct ImparoCache {
    int page_size;
    std::vector<int> windows;                            // 0 = every position
    std::vector<ImparoPool> pools;
    ImparoPool slots;
    std::unordered_map<int64_t, Request> live;

    ImparoCache(int n_groups, const int32_t* w, int ps, const int32_t* n_pages, int n_slots)
        : page_size(ps), slots(n_slots) {
        for (int g = 0; g < n_groups; ++g) {
            windows.push_back(w ? w[g] : 0);
            pools.emplace_back(n_pages[g]);          // every group has a pool of its own size
        }
    }
    int first_needed_page(int g, int next_position) const {
        if (windows[(size_t)g] <= 0) return 0;
        return std::max(0, next_position + 1 - windows[(size_t)g]) / page_size;
    }
    void undo(Request& r) {
        for (auto it = r.pending.rbegin(); it != r.pending.rend(); ++it) {
            r.tables[(size_t)it->first].pop_back();
            if (it->second >= 0) pools[(size_t)it->first].free_page(it->second);
        }
        r.pending.clear();
    }
};

#ifndef IMPARO_SOURCE_HASH
#define IMPARO_SOURCE_HASH "unknown"
#endif

extern "C" {

// the hash of the sources this library was built from (given by the build)
const char* imparo_host_source_hash() { return IMPARO_SOURCE_HASH; }

ImparoPool* imparo_pool_new(int n_pages) { return n_pages < 0 ? nullptr : new ImparoPool(n_pages); }
void imparo_pool_delete(ImparoPool* p) { delete p; }
int imparo_pool_alloc(ImparoPool* p) { return p->alloc(); }
int imparo_pool_free(ImparoPool* p, int page) { return p->free_page(page); }
int imparo_pool_n_free(const ImparoPool* p) { return p->n_free; }
int imparo_pool_n_pages(const ImparoPool* p) { return p->n_pages; }
int imparo_pool_high_water(const ImparoPool* p) { return p->high_water; }
int imparo_pool_is_free(const ImparoPool* p, int page) {
    return (page < 0 || page >= p->n_pages) ? IMPARO_E_RANGE : (int)p->is_free[(size_t)page];
}
int imparo_pool_scramble(ImparoPool* p, uint64_t seed) { return p->scramble(seed); }

ImparoCache* imparo_cache_new(int n_groups, const int32_t* windows, int page_size, const int32_t* n_pages,
                              int n_slots) {
    if (n_groups < 0 || page_size <= 0 || (page_size & (page_size - 1)) || n_slots < 0) return nullptr;
    if (n_groups > 0 && !n_pages) return nullptr;
    for (int g = 0; g < n_groups; ++g)
        if (n_pages[g] < 0) return nullptr;
    return new ImparoCache(n_groups, windows, page_size, n_pages, n_slots);
}
void imparo_cache_delete(ImparoCache* c) { delete c; }
ImparoPool* imparo_cache_group_pool(ImparoCache* c, int group) {
    return (group < 0 || group >= (int)c->pools.size()) ? nullptr : &c->pools[(size_t)group];
}
ImparoPool* imparo_cache_slot_pool(ImparoCache* c) { return &c->slots; }

int imparo_cache_admit(ImparoCache* c, int64_t req) {
    if (c->live.count(req)) return IMPARO_E_ALREADY_LIVE;
    const int slot = c->slots.alloc();
    if (slot < 0) return IMPARO_E_OUT_OF_PAGES;
    Request& r = c->live[req];
    r.slot = slot;
    r.tables.resize(c->pools.size());
    return slot;
}

int imparo_cache_release(ImparoCache* c, int64_t req) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    for (size_t g = 0; g < c->pools.size(); ++g)
        for (int32_t page : it->second.tables[g])
            if (page >= 0) c->pools[g].free_page(page);
    c->slots.free_page(it->second.slot);
    c->live.erase(it);
    return 0;
}

int imparo_cache_reserve(ImparoCache* c, int64_t req, int new_length) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    Request& r = it->second;
    if (new_length < r.length) return IMPARO_E_SHRINK;
    const size_t mark = r.pending.size();
    const int total = (new_length + c->page_size - 1) / c->page_size;
    for (size_t g = 0; g < c->pools.size(); ++g) {
        std::vector<int32_t>& table = r.tables[g];
        const int first = c->first_needed_page((int)g, r.length);
        while ((int)table.size() < total) {
            int32_t page = -1;                                  // wholly behind the window: never needed
            if ((int)table.size() >= first) {
                page = c->pools[g].alloc();
                if (page < 0) {                                 // undo what this call took, nothing else
                    while (r.pending.size() > mark) {
                        auto p = r.pending.back();
                        r.pending.pop_back();
                        r.tables[(size_t)p.first].pop_back();
                        if (p.second >= 0) c->pools[(size_t)p.first].free_page(p.second);
                    }
                    return IMPARO_E_OUT_OF_PAGES;
                }
            }
            table.push_back(page);
            r.pending.emplace_back((int)g, page);
        }
    }
    return 0;
}

int imparo_cache_rollback(ImparoCache* c, int64_t req) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    c->undo(it->second);
    return 0;
}

int imparo_cache_commit(ImparoCache* c, int64_t req, int new_length) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    Request& r = it->second;
    r.length = new_length;
    r.pending.clear();
    for (size_t g = 0; g < c->pools.size(); ++g) {
        if (c->windows[g] <= 0) continue;
        std::vector<int32_t>& table = r.tables[g];
        const int upto = std::min(c->first_needed_page((int)g, new_length), (int)table.size());
        for (int i = 0; i < upto; ++i)
            if (table[(size_t)i] >= 0) {
                c->pools[g].free_page(table[(size_t)i]);
                table[(size_t)i] = -1;
            }
    }
    return 0;
}

int imparo_cache_is_live(const ImparoCache* c, int64_t req) { return (int)c->live.count(req); }
int imparo_cache_length(const ImparoCache* c, int64_t req) {
    auto it = c->live.find(req);
    return it == c->live.end() ? IMPARO_E_NOT_LIVE : it->second.length;
}
int imparo_cache_slot(const ImparoCache* c, int64_t req) {
    auto it = c->live.find(req);
    return it == c->live.end() ? IMPARO_E_NOT_LIVE : it->second.slot;
}
int imparo_cache_table_len(const ImparoCache* c, int group, int64_t req) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    if (group < 0 || group >= (int)c->pools.size()) return IMPARO_E_RANGE;
    return (int)it->second.tables[(size_t)group].size();
}
int imparo_cache_table_copy(const ImparoCache* c, int group, int64_t req, int32_t* out, int capacity) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    if (group < 0 || group >= (int)c->pools.size()) return IMPARO_E_RANGE;
    const std::vector<int32_t>& t = it->second.tables[(size_t)group];
    if ((int)t.size() > capacity) return IMPARO_E_CAPACITY;
    if (!t.empty()) std::memcpy(out, t.data(), t.size() * sizeof(int32_t));
    return (int)t.size();
}
int imparo_cache_pages_needed(const ImparoCache* c, int64_t req, int new_length, int32_t* per_group) {
    auto it = c->live.find(req);
    if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
    const int total = (new_length + c->page_size - 1) / c->page_size;
    int worst = 0;
    for (size_t g = 0; g < c->pools.size(); ++g) {
        const int need = std::max(0, total - (int)it->second.tables[g].size());
        if (per_group) per_group[g] = need;
        worst = std::max(worst, need);
    }
    return worst;
}
int imparo_cache_first_needed_page(const ImparoCache* c, int group, int next_position) {
    if (group < 0 || group >= (int)c->pools.size()) return IMPARO_E_RANGE;
    return c->first_needed_page(group, next_position);
}
int imparo_cache_n_live(const ImparoCache* c) { return (int)c->live.size(); }
int imparo_cache_page_size(const ImparoCache* c) { return c->page_size; }
int imparo_cache_n_groups(const ImparoCache* c) { return (int)c->pools.size(); }
int imparo_cache_live_requests(const ImparoCache* c, int64_t* out, int capacity) {
    if ((int)c->live.size() > capacity) return IMPARO_E_CAPACITY;
    int i = 0;
    for (const auto& kv : c->live) out[i++] = kv.first;
    return i;
}

int imparo_cache_check(const ImparoCache* c) {
    for (size_t g = 0; g < c->pools.size(); ++g) {
        const ImparoPool& pool = c->pools[g];
        std::vector<char> held((size_t)pool.n_pages, 0);
        int n_held = 0;
        for (const auto& kv : c->live)
            for (int32_t page : kv.second.tables[g]) {
                if (page < 0) continue;
                if (page >= pool.n_pages || held[(size_t)page] || pool.is_free[(size_t)page]) return IMPARO_E_SHARED_PAGE;
                held[(size_t)page] = 1;
                ++n_held;
            }
        if (n_held + pool.n_free != pool.n_pages) return IMPARO_E_LOST_PAGE;
    }
    std::vector<char> taken((size_t)c->slots.n_pages, 0);
    for (const auto& kv : c->live) {
        const int s = kv.second.slot;
        if (s < 0 || s >= c->slots.n_pages || taken[(size_t)s] || c->slots.is_free[(size_t)s]) return IMPARO_E_SLOTS;
        taken[(size_t)s] = 1;
    }
    if ((int)c->live.size() + c->slots.n_free != c->slots.n_pages) return IMPARO_E_SLOTS;
    return 0;
}

int imparo_cache_begin_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens,
                            const int32_t* tokens, const int32_t* n_want, const int32_t* want, int vocab,
                            int max_position, int32_t* new_slots, int32_t* info) {
    int bad_row = -1, widest = 1, code = 0, no_slot = 0;
    // ---- what can be refused without touching anything
    {
        std::unordered_map<int64_t, int> seen;
        int64_t t = 0, w = 0;
        for (int r = 0; r < n_rows && !code; ++r) {
            const int n = n_tokens[r];
            auto it = c->live.find(reqs[r]);
            const int length = it == c->live.end() ? 0 : it->second.length;
            if (!seen.emplace(reqs[r], r).second) code = IMPARO_E_TWICE;
            else if (n <= 0) code = IMPARO_E_EMPTY;
            else if ((int64_t)length + n > max_position) code = IMPARO_E_POSITIONS;
            for (int i = 0; i < n && !code; ++i)
                if (tokens[t + i] < 0 || tokens[t + i] >= vocab) code = IMPARO_E_TOKEN;
            for (int i = 0; i < n_want[r] && !code; ++i)
                if (want[w + i] < 0 || want[w + i] >= n) code = IMPARO_E_WANT;
            if (code) bad_row = r;
            t += std::max(n, 0);
            w += n_want[r];
        }
    }
    // ---- slots and pages, all or nothing
    int done = 0;
    for (; done < n_rows && !code; ++done) {
        new_slots[done] = -1;
        if (!c->live.count(reqs[done])) {
            const int slot = imparo_cache_admit(c, reqs[done]);
            if (slot < 0) {
                code = IMPARO_E_OUT_OF_PAGES;
                bad_row = done;
                no_slot = 1;
                break;
            }
            new_slots[done] = slot;
        }
        Request& r = c->live[reqs[done]];
        const int rc = imparo_cache_reserve(c, reqs[done], r.length + n_tokens[done]);
        if (rc < 0) {
            if (new_slots[done] >= 0) imparo_cache_release(c, reqs[done]);
            code = rc;
            bad_row = done;
            break;
        }
        for (const auto& table : r.tables) widest = std::max(widest, (int)table.size());
    }
    if (code) {
        for (int r = done - 1; r >= 0; --r) {     // rows before the failing one
            if (new_slots[r] >= 0) imparo_cache_release(c, reqs[r]);
            else c->undo(c->live[reqs[r]]);
        }
    }
    if (info) {
        info[0] = bad_row;
        info[1] = widest;
        info[2] = no_slot;
    }
    return code;
}

int imparo_cache_abort_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* new_slots) {
    for (int r = n_rows - 1; r >= 0; --r) {
        auto it = c->live.find(reqs[r]);
        if (it == c->live.end()) continue;
        if (new_slots[r] >= 0) imparo_cache_release(c, reqs[r]);
        else c->undo(it->second);
    }
    return 0;
}

int imparo_cache_end_step(ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens) {
    for (int r = 0; r < n_rows; ++r) {
        auto it = c->live.find(reqs[r]);
        if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
        imparo_cache_commit(c, reqs[r], it->second.length + n_tokens[r]);
    }
    return 0;
}

int64_t imparo_cache_pack(const ImparoCache* c, int n_rows, const int64_t* reqs, const int32_t* n_tokens,
                          const int32_t* tokens, const int32_t* n_want, const int32_t* want, int table_width,
                          int32_t* out, int64_t capacity, int32_t* layout) {
    const int R = n_rows, G = (int)c->pools.size();
    int64_t T = 0, W = 0;
    int P = std::max(1, table_width), max_seg = 0, max_ctx = 0, n_single = 0;
    std::vector<const Request*> rows((size_t)R);
    for (int r = 0; r < R; ++r) {
        auto it = c->live.find(reqs[r]);
        if (it == c->live.end()) return IMPARO_E_NOT_LIVE;
        rows[(size_t)r] = &it->second;
        T += n_tokens[r];
        W += n_want[r];
        max_seg = std::max(max_seg, n_tokens[r]);
        max_ctx = std::max(max_ctx, it->second.length + n_tokens[r]);
        if (n_tokens[r] == 1) ++n_single;
        if (table_width <= 0)
            for (int g = 0; g < G; ++g) P = std::max(P, (int)it->second.tables[(size_t)g].size());
    }
    for (int r = 0; r < R && table_width > 0; ++r)
        for (int g = 0; g < G; ++g)
            if ((int)rows[(size_t)r]->tables[(size_t)g].size() > P) return IMPARO_E_RANGE;
    const int64_t total = 3 * T + 4 * (int64_t)R + W + (int64_t)G * R * P;
    if (total > capacity) return IMPARO_E_CAPACITY;
    int32_t* o_tok = out;
    int32_t* o_pos = out + T;
    int32_t* o_row = out + 2 * T;
    int32_t* o_start = out + 3 * T;
    int32_t* o_len = o_start + R;
    int32_t* o_slot = o_len + R;
    int32_t* o_lists = o_slot + R;
    int32_t* o_want = o_lists + R;
    int32_t* o_tab = o_want + W;
    int64_t t = 0, w = 0;
    int i_single = 0, i_multi = n_single;
    for (int r = 0; r < R; ++r) {
        const int n = n_tokens[r];
        const int base = rows[(size_t)r]->length;
        for (int i = 0; i < n; ++i) {
            o_tok[t + i] = tokens[t + i];
            o_pos[t + i] = base + i;
            o_row[t + i] = r;
        }
        o_start[r] = (int32_t)t;
        o_len[r] = n;
        o_slot[r] = rows[(size_t)r]->slot;
        if (n == 1) o_lists[i_single++] = r; else o_lists[i_multi++] = r;
        for (int i = 0; i < n_want[r]; ++i) {
            if (want[w + i] < 0 || want[w + i] >= n) return IMPARO_E_RANGE;
            o_want[w + i] = (int32_t)t + want[w + i];
        }
        t += n;
        w += n_want[r];
    }
    for (int g = 0; g < G; ++g)
        for (int r = 0; r < R; ++r) {
            int32_t* dst = o_tab + ((int64_t)g * R + r) * P;
            const std::vector<int32_t>& tab = rows[(size_t)r]->tables[(size_t)g];
            std::copy(tab.begin(), tab.end(), dst);
            std::fill(dst + tab.size(), dst + P, -1);
        }
    if (layout) {
        const int32_t v[10] = {(int32_t)T, R, (int32_t)W, G, P, n_single, R - n_single, max_seg, max_ctx,
                               (int32_t)total};
        std::memcpy(layout, v, sizeof(v));
    }
    return total;
}

}  // extern "C"
