// The scheduler's decisions. One iteration: every running request gets its next tokens under
// a token budget (one decoded token each first, in arrival order, then portions of prompts),
// newcomers are admitted first come first served while they fit, and if the pages do not
// suffice the youngest running request is pre-empted. The reference's loop has the same
// duties (/root/reference/crates/imparo-server/src/sched.rs:4-19); its admission rule is
// "pages of the newcomer plus one per running request must be obtainable"
// (/root/reference/crates/imparo-server/src/main.rs:2230-2246). Where the reference parks a
// row on a disk tier when pages run out (sched.rs:483-488,701-732) this one gives the
// youngest request's pages back and recomputes it later.
#include "host_api.h"

#include <algorithm>
#include <deque>
#include <unordered_map>
#include <vector>

struct SchedRequest {
    int prompt_len = 0;
    int n_generated = 0;
    int pending_len = 0;      // tokens to (re)compute before decoding goes on
    int fed = 0;              // how many of them the cache holds
    bool has_next = false;    // a sampled token waits to be fed
    int max_tokens = 0;
    int arrival = 0;
};

struct Planned {
    int64_t id;
    int offset, count, wants;
};

struct ImparoSched {
    ImparoCache* cache;
    int max_batch_tokens, max_running, portion;
    int arrivals = 0;
    std::deque<int64_t> waiting;
    std::vector<int64_t> running;
    std::unordered_map<int64_t, SchedRequest> reqs;
    std::vector<Planned> planned;

    int pages_for(int n_tokens) const {
        // page size comes from the cache: ask it how many pages n positions of a fresh request take
        const int ps = page_size;
        return (n_tokens + ps - 1) / ps;
    }
    int page_size = 1;
    int n_groups = 0;

    int free_pages() const {
        int least = 1 << 30;
        for (int g = 0; g < n_groups; ++g)
            least = std::min(least, imparo_pool_n_free(imparo_cache_group_pool(cache, g)));
        return least;
    }
    Planned next_tokens(int64_t id, const SchedRequest& r, int budget) const {
        if (r.fed < r.pending_len) {
            const int n = std::min({portion, budget, r.pending_len - r.fed});
            return Planned{id, r.fed, n, (r.fed + n == r.pending_len && !r.has_next) ? 1 : 0};
        }
        return Planned{id, -1, 1, 1};
    }
    int pages_needed(const Planned& p) const {
        if (imparo_cache_is_live(cache, p.id))
            return imparo_cache_pages_needed(cache, p.id, imparo_cache_length(cache, p.id) + p.count, nullptr);
        return pages_for(p.count);
    }
    void leave(int64_t id) {
        running.erase(std::remove(running.begin(), running.end(), id), running.end());
        if (imparo_cache_is_live(cache, id)) imparo_cache_release(cache, id);
    }
};

extern "C" {

ImparoSched* imparo_sched_new(ImparoCache* cache, int max_batch_tokens, int max_running, int portion) {
    if (!cache || max_batch_tokens <= 0 || max_running <= 0 || portion <= 0) return nullptr;
    ImparoSched* s = new ImparoSched();
    s->cache = cache;
    s->max_batch_tokens = max_batch_tokens;
    s->max_running = max_running;
    s->portion = portion;
    s->page_size = imparo_cache_page_size(cache);
    s->n_groups = imparo_cache_n_groups(cache);
    return s;
}
void imparo_sched_delete(ImparoSched* s) { delete s; }

int imparo_sched_add(ImparoSched* s, int64_t id, int prompt_len, int max_tokens) {
    if (s->reqs.count(id)) return IMPARO_E_ALREADY_LIVE;
    if (prompt_len <= 0) return IMPARO_E_RANGE;
    const int arrival = s->arrivals++;
    if (max_tokens <= 0) return 1;
    SchedRequest r;
    r.prompt_len = r.pending_len = prompt_len;
    r.max_tokens = max_tokens;
    r.arrival = arrival;
    s->reqs[id] = r;
    s->waiting.push_back(id);
    return 0;
}

int imparo_sched_plan(ImparoSched* s, int64_t* ids, int32_t* offsets, int32_t* counts, int32_t* wants, int capacity,
                      int64_t* ev_ids, int32_t* ev_kinds, int ev_capacity, int32_t* n_events) {
    int n_ev = 0;
    auto event = [&](int64_t id, int kind) {
        if (n_ev < ev_capacity) {
            ev_ids[n_ev] = id;
            ev_kinds[n_ev] = kind;
        }
        ++n_ev;
    };
    int budget = s->max_batch_tokens;
    std::vector<Planned>& planned = s->planned;
    planned.clear();
    // 1. running requests: decoders first, then prompts in progress, each in arrival order
    std::vector<int64_t> order = s->running;
    std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) {
        const SchedRequest &ra = s->reqs[a], &rb = s->reqs[b];
        const bool pa = ra.fed < ra.pending_len, pb = rb.fed < rb.pending_len;
        if (pa != pb) return !pa;
        return ra.arrival < rb.arrival;
    });
    for (int64_t id : order) {
        if (budget <= 0) break;
        planned.push_back(s->next_tokens(id, s->reqs[id], budget));
        budget -= planned.back().count;
    }
    int spoken_for = 0;
    for (const Planned& p : planned) spoken_for += s->pages_needed(p);
    // 2. admissions, first come first served; the head of the line blocks the rest
    while (!s->waiting.empty() && budget > 0 && (int)s->running.size() < s->max_running) {
        const int64_t id = s->waiting.front();
        const Planned p = s->next_tokens(id, s->reqs[id], budget);
        const int need = s->pages_for(p.count) + (int)s->running.size();     // one page of headroom per running request
        // every request planned for this step that is not live yet takes a slot when the step runs
        int slots_left = imparo_pool_n_free(imparo_cache_slot_pool(s->cache));
        for (const Planned& q : planned)
            if (!imparo_cache_is_live(s->cache, q.id)) --slots_left;
        if (slots_left <= 0 || (!s->running.empty() && need > s->free_pages() - spoken_for)) {
            event(id, IMPARO_EV_WAIT);
            break;
        }
        s->waiting.pop_front();
        s->running.push_back(id);
        event(id, IMPARO_EV_ADMIT);
        planned.push_back(p);
        spoken_for += s->pages_for(p.count);
        budget -= p.count;
    }
    // 3. do the pages suffice? if not, the youngest running request goes back in line
    while (!planned.empty()) {
        int need = 0;
        for (const Planned& p : planned) need += s->pages_needed(p);
        if (need <= s->free_pages()) break;
        if (s->running.size() == 1) {
            const int64_t id = s->running[0];
            s->leave(id);
            s->reqs.erase(id);
            event(id, IMPARO_EV_FAIL);
            planned.clear();
            break;
        }
        int64_t victim = s->running[0];
        for (int64_t id : s->running)
            if (s->reqs[id].arrival > s->reqs[victim].arrival) victim = id;
        s->leave(victim);
        SchedRequest& r = s->reqs[victim];
        r.pending_len = r.prompt_len + r.n_generated;
        r.fed = 0;
        r.has_next = false;
        s->waiting.push_front(victim);
        event(victim, IMPARO_EV_PREEMPT);
        planned.erase(std::remove_if(planned.begin(), planned.end(), [&](const Planned& p) { return p.id == victim; }),
                      planned.end());
    }
    if ((int)planned.size() > capacity) return IMPARO_E_CAPACITY;
    for (size_t i = 0; i < planned.size(); ++i) {
        ids[i] = planned[i].id;
        offsets[i] = planned[i].offset;
        counts[i] = planned[i].count;
        wants[i] = planned[i].wants;
    }
    if (n_events) *n_events = n_ev;
    return (int)planned.size();
}

void imparo_sched_advance(ImparoSched* s) {
    for (const Planned& p : s->planned) {
        auto it = s->reqs.find(p.id);
        if (it == s->reqs.end()) continue;
        if (p.offset >= 0)
            it->second.fed += p.count;
        else
            it->second.has_next = false;        // the decoded token is in the cache now
    }
    s->planned.clear();
}

int imparo_sched_token(ImparoSched* s, int64_t id, int is_stop) {
    auto it = s->reqs.find(id);
    if (it == s->reqs.end()) return IMPARO_E_NOT_LIVE;
    SchedRequest& r = it->second;
    int outcome = 0;
    if (is_stop) {
        outcome = 1;                             // a stop token ends the reply unsent
    } else {
        ++r.n_generated;
        if (r.n_generated >= r.max_tokens) outcome = 2;   // the last token needs no forward
        else r.has_next = true;
    }
    if (outcome) {
        s->running.erase(std::remove(s->running.begin(), s->running.end(), id), s->running.end());
        s->reqs.erase(it);
    }
    return outcome;
}

int imparo_sched_retract(ImparoSched* s, int64_t id) {
    auto it = s->reqs.find(id);
    if (it == s->reqs.end()) return IMPARO_E_NOT_LIVE;
    s->running.erase(std::remove(s->running.begin(), s->running.end(), id), s->running.end());
    s->waiting.erase(std::remove(s->waiting.begin(), s->waiting.end(), id), s->waiting.end());
    s->planned.erase(std::remove_if(s->planned.begin(), s->planned.end(), [&](const Planned& p) { return p.id == id; }),
                     s->planned.end());
    s->reqs.erase(it);
    return 0;
}

int imparo_sched_drop_waiting_head(ImparoSched* s, int64_t* id) {
    if (s->waiting.empty()) return 0;
    *id = s->waiting.front();
    s->waiting.pop_front();
    s->reqs.erase(*id);
    return 1;
}

int imparo_sched_n_waiting(const ImparoSched* s) { return (int)s->waiting.size(); }
int imparo_sched_n_running(const ImparoSched* s) { return (int)s->running.size(); }
int imparo_sched_waiting(const ImparoSched* s, int64_t* out, int capacity) {
    if ((int)s->waiting.size() > capacity) return IMPARO_E_CAPACITY;
    std::copy(s->waiting.begin(), s->waiting.end(), out);
    return (int)s->waiting.size();
}
int imparo_sched_running(const ImparoSched* s, int64_t* out, int capacity) {
    if ((int)s->running.size() > capacity) return IMPARO_E_CAPACITY;
    std::copy(s->running.begin(), s->running.end(), out);
    return (int)s->running.size();
}

}  // extern "C"
