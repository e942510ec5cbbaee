#include "cache.h"

#include <algorithm>

namespace lcu {

PagePool::PagePool(int n) : held_(n > 0 ? n : 0, 0) {
    free_.reserve(held_.size());
    for (int i = (int)held_.size() - 1; i >= 0; --i) free_.push_back(i);   // page 0 is taken first
}

int PagePool::take() {
    if (free_.empty()) return -1;
    int p = free_.back();
    free_.pop_back();
    held_[p] = 1;
    return p;
}

bool PagePool::give(int page) {
    if (page < 0 || page >= (int)held_.size() || !held_[page]) return false;
    held_[page] = 0;
    free_.push_back(page);
    return true;
}

CacheManager::CacheManager(const std::vector<GroupDesc> &groups, int n_slots, bool can_truncate)
    : groups_(groups), n_slots_(n_slots), can_truncate_(can_truncate) {
    for (const auto &g : groups_) pools_.emplace_back(g.num_pages);
    for (int i = n_slots - 1; i >= 0; --i) free_slots_.push_back(i);
}

const RequestCache *CacheManager::get(int64_t id) const {
    auto it = reqs_.find(id);
    return it == reqs_.end() ? nullptr : &it->second;
}

int CacheManager::add(int64_t id) {
    if (reqs_.count(id)) return CACHE_DUPLICATE_REQUEST;
    if (free_slots_.empty()) return CACHE_NO_SLOT;
    RequestCache rc;
    rc.slot = free_slots_.back();
    free_slots_.pop_back();
    rc.tables.resize(groups_.size());
    reqs_.emplace(id, std::move(rc));
    return CACHE_OK;
}

int CacheManager::pages_needed(int64_t id, int g, int new_len) const {
    const RequestCache *rc = get(id);
    if (!rc) return 0;
    const int have = (int)rc->tables[g].size();
    const int want = pages_for(new_len, groups_[g].page_size);
    return want > have ? want - have : 0;
}

int CacheManager::max_reservable(int64_t id, int want) const {
    const RequestCache *rc = get(id);
    if (!rc) return 0;
    int best = want;
    for (size_t g = 0; g < groups_.size(); ++g) {
        const int ps = groups_[g].page_size;
        const int can = ((int)rc->tables[g].size() + pools_[g].free_count()) * ps;
        best = std::min(best, can);
    }
    return std::max(best, rc->reserved);
}

int CacheManager::reserve(int64_t id, int new_len) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    RequestCache &rc = it->second;
    if (new_len < rc.len) return CACHE_BAD_ARGUMENT;
    for (size_t g = 0; g < groups_.size(); ++g)
        if (pages_needed(id, (int)g, new_len) > pools_[g].free_count()) return CACHE_NO_PAGES;
    for (size_t g = 0; g < groups_.size(); ++g) {
        const int want = pages_for(new_len, groups_[g].page_size);
        while ((int)rc.tables[g].size() < want) rc.tables[g].push_back(pools_[g].take());
    }
    rc.reserved = std::max(rc.reserved, new_len);
    return CACHE_OK;
}

int CacheManager::commit(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    RequestCache &rc = it->second;
    rc.len = rc.reserved;
    // A window has passed a page when the next query (at position len) cannot see any of its
    // tokens: the first key it sees is len - window + 1 (with slack: the query at len - slack).
    for (size_t g = 0; g < groups_.size(); ++g) {
        const int w = groups_[g].window;
        if (w <= 0) continue;
        const int first_key = rc.len - groups_[g].slack - w + 1;
        if (first_key <= 0) continue;
        const int first_page = first_key / groups_[g].page_size;
        auto &tab = rc.tables[g];
        for (int p = 0; p < first_page && p < (int)tab.size(); ++p) {
            if (tab[p] >= 0) {
                if (!pools_[g].give(tab[p])) return CACHE_CORRUPT;
                tab[p] = -1;
            }
        }
    }
    return CACHE_OK;
}

int CacheManager::truncate(int64_t id, int new_len) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    RequestCache &rc = it->second;
    if (new_len < 0 || new_len > rc.len) return CACHE_BAD_ARGUMENT;
    if (new_len < rc.len && !can_truncate_) return CACHE_CANNOT_TRUNCATE;
    // a windowed group must still hold what the query at new_len will see
    for (size_t g = 0; g < groups_.size(); ++g) {
        const int w = groups_[g].window;
        if (w <= 0) continue;
        const int first_key = std::max(0, new_len - w + 1);
        const auto &tab = rc.tables[g];
        for (int p = first_key / groups_[g].page_size; p < pages_for(new_len, groups_[g].page_size); ++p)
            if (p < (int)tab.size() && tab[p] < 0) return CACHE_WINDOW_PASSED;
    }
    for (size_t g = 0; g < groups_.size(); ++g) {
        const int keep = pages_for(new_len, groups_[g].page_size);
        auto &tab = rc.tables[g];
        while ((int)tab.size() > keep) {
            if (tab.back() >= 0 && !pools_[g].give(tab.back())) return CACHE_CORRUPT;
            tab.pop_back();
        }
    }
    rc.len = rc.reserved = new_len;
    return CACHE_OK;
}

int CacheManager::truncate_or_reset(int64_t id, int new_len) {
    const int st = truncate(id, new_len);
    if (st != CACHE_CANNOT_TRUNCATE && st != CACHE_WINDOW_PASSED) return st;
    RequestCache &rc = reqs_.at(id);
    int reserved = new_len;
    for (size_t g = 0; g < groups_.size(); ++g) {
        auto &tab = rc.tables[g];
        const int keep = groups_[g].window > 0 ? 0 : pages_for(new_len, groups_[g].page_size);
        while ((int)tab.size() > keep) {
            if (tab.back() >= 0 && !pools_[g].give(tab.back())) return CACHE_CORRUPT;
            tab.pop_back();
        }
        reserved = std::min(reserved, (int)tab.size() * groups_[g].page_size);
    }
    rc.len = 0;
    rc.reserved = reserved;
    return CACHE_RESET;
}

int CacheManager::release(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    RequestCache &rc = it->second;
    int status = CACHE_OK;
    for (size_t g = 0; g < groups_.size(); ++g)
        for (int p : rc.tables[g])
            if (p >= 0 && !pools_[g].give(p)) status = CACHE_CORRUPT;
    free_slots_.push_back(rc.slot);
    reqs_.erase(it);
    return status;
}

int CacheManager::fill_batch(int n_req, const int64_t *ids, const int *n_new, int *positions, int *req_of_token,
                             int *q_start, int *ctx_len, int *state_slot, int *const *block_tables,
                             const int *max_pages, int *const *slots) const {
    int t = 0;
    for (int r = 0; r < n_req; ++r) {
        const RequestCache *rc = get(ids[r]);
        if (!rc) return CACHE_UNKNOWN_REQUEST;
        if (n_new[r] <= 0 || rc->len + n_new[r] > rc->reserved) return CACHE_BAD_ARGUMENT;
        q_start[r] = t;
        ctx_len[r] = rc->len + n_new[r];
        state_slot[r] = rc->slot;
        for (size_t g = 0; g < groups_.size(); ++g) {
            const auto &tab = rc->tables[g];
            const int ps = groups_[g].page_size;
            if ((int)tab.size() > max_pages[g]) return CACHE_BAD_ARGUMENT;
            int *row = block_tables[g] + (size_t)r * max_pages[g];
            for (int p = 0; p < max_pages[g]; ++p) row[p] = (p < (int)tab.size() && tab[p] >= 0) ? tab[p] : 0;
            for (int i = 0; i < n_new[r]; ++i) {
                const int pos = rc->len + i;
                const int page = tab[pos / ps];
                if (page < 0) return CACHE_CORRUPT;
                slots[g][t + i] = page * ps + pos % ps;
            }
        }
        for (int i = 0; i < n_new[r]; ++i) {
            positions[t + i] = rc->len + i;
            req_of_token[t + i] = r;
        }
        t += n_new[r];
    }
    q_start[n_req] = t;
    return CACHE_OK;
}

void CacheManager::page_owners(int g, int64_t *owners) const {
    for (int p = 0; p < pools_[g].size(); ++p) owners[p] = -1;
    for (const auto &kv : reqs_)
        for (int p : kv.second.tables[g])
            if (p >= 0 && p < pools_[g].size()) owners[p] = kv.first;
}

int CacheManager::check(std::string *why) const {
    auto fail = [&](const std::string &m) {
        if (why) *why = m;
        return (int)CACHE_CORRUPT;
    };
    for (size_t g = 0; g < groups_.size(); ++g) {
        std::vector<int> owners(pools_[g].size(), 0);
        for (const auto &kv : reqs_)
            for (int p : kv.second.tables[g]) {
                if (p < 0) continue;
                if (p >= pools_[g].size()) return fail("a table holds a page outside the pool");
                if (++owners[p] > 1) return fail("a page is held twice");
                if (!pools_[g].is_held(p)) return fail("a table holds a page that the pool thinks free");
            }
        int held = 0;
        for (int p = 0; p < pools_[g].size(); ++p) {
            if (pools_[g].is_held(p)) {
                ++held;
                if (!owners[p]) return fail("a page is lost: held by the pool, in no table");
            }
        }
        if (held + pools_[g].free_count() != pools_[g].size()) return fail("free and held pages do not add up");
    }
    std::vector<int> slot_owner(n_slots_, 0);
    for (const auto &kv : reqs_) {
        const int s = kv.second.slot;
        if (s < 0 || s >= n_slots_) return fail("a request holds a slot outside the pool");
        if (++slot_owner[s] > 1) return fail("a slot is held twice");
    }
    for (int s : free_slots_)
        if (s < 0 || s >= n_slots_ || slot_owner[s]) return fail("a free slot is also held");
    if ((int)free_slots_.size() + (int)reqs_.size() != n_slots_) return fail("free and held slots do not add up");
    return CACHE_OK;
}

}  // namespace lcu
