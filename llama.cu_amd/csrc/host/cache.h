// The cache manager: pages of keys and values with a block table per request, in
// groups with pools of their own, and slots for per-request state of fixed size.
//
// The reference pages its cache through the GPU's virtual memory: every request
// reserves a virtual range for its whole context and physical pages are mapped as it
// grows and unmapped as it shrinks (llama.cu/src/exec/kv_cache.rs:34-50,
// llama.cu/src/memory.rs:36-53); its pool creates pages without bound.  Here the
// table is explicit, the pool is bounded, and running out of pages is an answer
// (`reserve` returns false), not a crash.  No GPU code: this file compiles with any
// C++17 compiler and is tested on the CPU.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace lcu {

struct GroupDesc {
    int num_pages;   // pages in this group's pool
    int page_size;   // tokens per page
    int window;      // 0: all tokens are kept; w > 0: a token sees the last w tokens, itself included
    int slack = 0;   // a window gives a page back only when a request cut back by up to this many tokens
                     // would not see it either (an engine that runs one round ahead of its sampler's
                     // results cuts a request back by the one token it computed beyond its end)
};

class PagePool {
  public:
    explicit PagePool(int n);
    int take();                 // a free page, or -1
    bool give(int page);        // false if the page is not held (double free) or out of range
    int free_count() const { return (int)free_.size(); }
    int size() const { return (int)held_.size(); }
    bool is_held(int page) const { return page >= 0 && page < size() && held_[page]; }

  private:
    std::vector<int> free_;     // used as a stack: the page given back last is taken first
    std::vector<uint8_t> held_;
};

struct RequestCache {
    int len = 0;                            // tokens whose keys and values are written
    int reserved = 0;                       // tokens that have pages (>= len)
    int slot = -1;                          // state slot
    std::vector<std::vector<int>> tables;   // per group: logical page -> physical page, -1 once given back
};

enum CacheStatus {
    CACHE_OK = 0,
    CACHE_NO_PAGES = 1,       // not enough free pages: nothing was changed
    CACHE_NO_SLOT = 2,        // all state slots are taken
    CACHE_RESET = 3,          // truncate_or_reset: the request was not cut back but set to length 0
    CACHE_UNKNOWN_REQUEST = -1,
    CACHE_DUPLICATE_REQUEST = -2,
    CACHE_BAD_ARGUMENT = -3,
    CACHE_WINDOW_PASSED = -4, // truncate below what a window has already given back
    CACHE_CORRUPT = -5,
    CACHE_CANNOT_TRUNCATE = -6,   // the model keeps per-request state that cannot be cut back to a shorter length
};

class CacheManager {
  public:
    // can_truncate: whether everything that the model keeps for a request can be cut back to a
    // shorter length.  Pages can; a state of fixed size that has folded tokens in cannot, and
    // then `truncate` to less than the request holds is refused.
    CacheManager(const std::vector<GroupDesc> &groups, int n_slots, bool can_truncate = true);

    int add(int64_t id);                       // CACHE_OK and a slot taken, or an error
    int reserve(int64_t id, int new_len);      // pages for tokens [len, new_len) in every group, all or nothing
    int commit(int64_t id);                    // the reserved tokens are written; windows slide
    int truncate(int64_t id, int new_len);     // forget the tokens at and after new_len, give tail pages back
    // truncate where everything the request holds can be cut back to new_len.  Where something cannot (a
    // state of fixed size; a window that has given back a page that the shorter request would see), the
    // request has to be computed again from its first token, and only what cannot be cut is given up:
    // the request's length becomes 0, every group without a window keeps its pages up to new_len (the
    // recomputation writes the same keys and values into them and asks the pool for nothing), a group
    // with a window gives its pages back (their place in the table depends on where the window stood),
    // the slot stays (its owner starts the state anew at position 0).  CACHE_OK: cut back; CACHE_RESET:
    // set to 0; anything else: an error, nothing changed.
    int truncate_or_reset(int64_t id, int new_len);
    int release(int64_t id);                   // give everything back
    bool has(int64_t id) const { return reqs_.count(id) != 0; }
    const RequestCache *get(int64_t id) const;

    int n_groups() const { return (int)groups_.size(); }
    const GroupDesc &group(int g) const { return groups_[g]; }
    int free_pages(int g) const { return pools_[g].free_count(); }
    int free_slots() const { return (int)free_slots_.size(); }
    int n_slots() const { return n_slots_; }
    bool can_truncate() const { return can_truncate_; }
    int live_requests() const { return (int)reqs_.size(); }
    // pages that `reserve(id, new_len)` would take from group g
    int pages_needed(int64_t id, int g, int new_len) const;
    // the largest new_len <= want that the free pages allow for this request (>= its len)
    int max_reservable(int64_t id, int want) const;

    // The batch arrays for the requests ids[0..n_req) that feed n_new[i] tokens each (pages
    // reserved before).  positions, req_of_token: [sum n_new]; q_start: [n_req + 1]; ctx_len,
    // state_slot: [n_req]; block_tables[g]: [n_req, max_pages[g]] (an entry that was given
    // back, or lies beyond the request, is 0: no kernel reads it); slots[g]: [sum n_new].
    int fill_batch(int n_req, const int64_t *ids, const int *n_new, int *positions, int *req_of_token,
                   int *q_start, int *ctx_len, int *state_slot, int *const *block_tables, const int *max_pages,
                   int *const *slots) const;

    // owners[p] = the request that holds page p of group g, or -1 for a free page (owners has
    // room for the group's pages).
    void page_owners(int g, int64_t *owners) const;

    // Every page is free or held by exactly one table entry; every slot likewise.
    int check(std::string *why = nullptr) const;

  private:
    static int pages_for(int tokens, int page_size) { return (tokens + page_size - 1) / page_size; }
    std::vector<GroupDesc> groups_;
    std::vector<PagePool> pools_;
    std::vector<int> free_slots_;
    int n_slots_;
    bool can_truncate_;
    std::unordered_map<int64_t, RequestCache> reqs_;
};

}  // namespace lcu
