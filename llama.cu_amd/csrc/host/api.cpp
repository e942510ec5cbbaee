// The C interface of the host library (cache manager and scheduler), as Python's
// ctypes calls it.  Handles are opaque pointers; every function returns a status
// (0 = ok) or a count.
#include <cstring>
#include <string>

#include "cache.h"
#include "sched.h"

using namespace lcu;

#define API extern "C" __attribute__((visibility("default")))

API void *lcu_cache_create(int n_groups, const int *num_pages, const int *page_size, const int *window, const int *slack,
                           int n_slots, int can_truncate) {
    std::vector<GroupDesc> g;
    for (int i = 0; i < n_groups; ++i) {
        if (num_pages[i] < 0 || page_size[i] <= 0 || window[i] < 0 || slack[i] < 0) return nullptr;
        g.push_back({num_pages[i], page_size[i], window[i], slack[i]});
    }
    if (n_slots < 0) return nullptr;
    return new CacheManager(g, n_slots, can_truncate != 0);
}
API void lcu_cache_destroy(void *h) { delete (CacheManager *)h; }
API int lcu_cache_add(void *h, long long id) { return ((CacheManager *)h)->add(id); }
API int lcu_cache_reserve(void *h, long long id, int new_len) { return ((CacheManager *)h)->reserve(id, new_len); }
API int lcu_cache_commit(void *h, long long id) { return ((CacheManager *)h)->commit(id); }
API int lcu_cache_truncate(void *h, long long id, int new_len) { return ((CacheManager *)h)->truncate(id, new_len); }
API int lcu_cache_truncate_or_reset(void *h, long long id, int new_len) { return ((CacheManager *)h)->truncate_or_reset(id, new_len); }
API int lcu_cache_release(void *h, long long id) { return ((CacheManager *)h)->release(id); }
API int lcu_cache_has(void *h, long long id) { return ((CacheManager *)h)->has(id) ? 1 : 0; }
API int lcu_cache_len(void *h, long long id) {
    const RequestCache *rc = ((CacheManager *)h)->get(id);
    return rc ? rc->len : -1;
}
API int lcu_cache_reserved(void *h, long long id) {
    const RequestCache *rc = ((CacheManager *)h)->get(id);
    return rc ? rc->reserved : -1;
}
API int lcu_cache_slot(void *h, long long id) {
    const RequestCache *rc = ((CacheManager *)h)->get(id);
    return rc ? rc->slot : -1;
}
API int lcu_cache_free_pages(void *h, int g) { return ((CacheManager *)h)->free_pages(g); }
API int lcu_cache_free_slots(void *h) { return ((CacheManager *)h)->free_slots(); }
API int lcu_cache_live(void *h) { return ((CacheManager *)h)->live_requests(); }
API int lcu_cache_max_reservable(void *h, long long id, int want) { return ((CacheManager *)h)->max_reservable(id, want); }
// The request's table of group g as it is (given-back pages are -1); returns the
// number of logical pages, also when out is too small (then nothing is written).
API int lcu_cache_table(void *h, long long id, int g, int *out, int cap) {
    const RequestCache *rc = ((CacheManager *)h)->get(id);
    if (!rc || g < 0 || g >= (int)rc->tables.size()) return -1;
    const auto &t = rc->tables[g];
    if ((int)t.size() <= cap) std::memcpy(out, t.data(), t.size() * sizeof(int));
    return (int)t.size();
}
API int lcu_cache_fill_batch(void *h, int n_req, const long long *ids, const int *n_new, int *positions,
                             int *req_of_token, int *q_start, int *ctx_len, int *state_slot, int *const *block_tables,
                             const int *max_pages, int *const *slots) {
    return ((CacheManager *)h)->fill_batch(n_req, (const int64_t *)ids, n_new, positions, req_of_token, q_start,
                                           ctx_len, state_slot, block_tables, max_pages, slots);
}
// owners[p] = the request that holds page p of group g, -1 if it is free; returns the number of
// pages of the group (-1 for a bad group, and nothing is written if cap is too small).
API int lcu_cache_page_owners(void *h, int g, long long *owners, int cap) {
    CacheManager *m = (CacheManager *)h;
    if (g < 0 || g >= m->n_groups()) return -1;
    const int n = m->group(g).num_pages;
    if (n <= cap) m->page_owners(g, (int64_t *)owners);
    return n;
}
API int lcu_cache_check(void *h, char *why, int cap) {
    std::string w;
    const int st = ((CacheManager *)h)->check(&w);
    if (why && cap > 0) {
        std::strncpy(why, w.c_str(), cap - 1);
        why[cap - 1] = 0;
    }
    return st;
}

// ---------------------------------------------------------------- scheduler

struct SchedHandle {
    Scheduler sched;
    std::vector<PlanEntry> last_plan;
    SchedHandle(const SchedConfig &c, CacheManager *cm) : sched(c, cm) {}
};

API void *lcu_sched_create(void *cache, int max_num_seqs, int max_batch_tokens, int prefill_chunk, int max_model_len) {
    if (!cache || max_num_seqs <= 0 || max_batch_tokens <= 0 || prefill_chunk <= 0 || max_model_len <= 0) return nullptr;
    return new SchedHandle(SchedConfig{max_num_seqs, max_batch_tokens, prefill_chunk, max_model_len}, (CacheManager *)cache);
}
API void lcu_sched_destroy(void *h) { delete (SchedHandle *)h; }
API int lcu_sched_add(void *h, long long id, const int *tokens, int n, int max_new, int keep) {
    return ((SchedHandle *)h)->sched.add(id, tokens, n, max_new, keep);
}
API int lcu_sched_extend(void *h, long long id, const int *tokens, int n, int max_new) {
    return ((SchedHandle *)h)->sched.extend(id, tokens, n, max_new);
}
API int lcu_sched_abort(void *h, long long id) { return ((SchedHandle *)h)->sched.abort(id); }
API int lcu_sched_drop(void *h, long long id) { return ((SchedHandle *)h)->sched.drop(id); }
// Plans the next step; entries are written as (id, start, count, want_logits) into the
// four arrays.  Returns the number of entries (-1 if cap is too small).
API int lcu_sched_plan(void *h, long long *ids, int *start, int *count, int *want, int cap) {
    SchedHandle *s = (SchedHandle *)h;
    s->last_plan = s->sched.plan();
    if ((int)s->last_plan.size() > cap) return -1;
    for (size_t i = 0; i < s->last_plan.size(); ++i) {
        ids[i] = s->last_plan[i].id;
        start[i] = s->last_plan[i].start;
        count[i] = s->last_plan[i].count;
        want[i] = s->last_plan[i].want_logits;
    }
    return (int)s->last_plan.size();
}
API void lcu_sched_commit(void *h) {
    SchedHandle *s = (SchedHandle *)h;
    s->sched.commit(s->last_plan);
    s->last_plan.clear();
}
API int lcu_sched_append(void *h, long long id, int token, int is_eos) {
    return ((SchedHandle *)h)->sched.append(id, token, is_eos);
}
API int lcu_sched_set_token(void *h, long long id, int index, int token) {
    return ((SchedHandle *)h)->sched.set_token(id, index, token);
}
API int lcu_sched_finish(void *h, long long id, int reason, int n_tokens) {
    return ((SchedHandle *)h)->sched.finish_now(id, reason, n_tokens);
}
API int lcu_sched_n_waiting(void *h) { return ((SchedHandle *)h)->sched.n_waiting(); }
API int lcu_sched_n_running(void *h) { return ((SchedHandle *)h)->sched.n_running(); }
API long long lcu_sched_preemptions(void *h) { return ((SchedHandle *)h)->sched.total_preemptions(); }
API int lcu_sched_take_finished(void *h, long long *ids, int cap) {
    auto v = ((SchedHandle *)h)->sched.take_finished();
    int n = 0;
    for (auto id : v)
        if (n < cap) ids[n++] = id;
    return n;
}
// state of one request: out = {n_tokens, prompt_len, computed, generated, reason, preemptions}
API int lcu_sched_info(void *h, long long id, int *out) {
    const SchedRequest *r = ((SchedHandle *)h)->sched.get(id);
    if (!r) return CACHE_UNKNOWN_REQUEST;
    out[0] = (int)r->tokens.size();
    out[1] = r->prompt_len;
    out[2] = r->computed;
    out[3] = r->generated;
    out[4] = r->reason;
    out[5] = r->preemptions;
    return CACHE_OK;
}
API int lcu_sched_tokens(void *h, long long id, int *out, int cap) {
    const SchedRequest *r = ((SchedHandle *)h)->sched.get(id);
    if (!r) return -1;
    if ((int)r->tokens.size() <= cap) std::memcpy(out, r->tokens.data(), r->tokens.size() * sizeof(int));
    return (int)r->tokens.size();
}
