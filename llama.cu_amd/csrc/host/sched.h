// The scheduler: admits requests, cuts prompts into portions under a token budget,
// decodes one token per running request, finishes and frees.
//
// The reference's scheduler (llama.cu/src/exec/engine_manager.rs:72-130) puts every live
// session into every round with all its pending tokens: no budget, no portions
// (`assert_eq!(out, 1, "TODO: chunked prefill")`, :83), and its page pool cannot run
// out.  Kept from it: batch order is admission order, a request's step budget counts
// every generated token including the first (:118-122), a request whose context is full
// ends (`Overflow`, :85-90).
//
// When pages run out: a request that decodes and cannot get a page makes the request
// admitted last give up its pages (it goes back to the front of the waiting queue and
// is computed again from its tokens); a prompt portion shrinks to the pages that are
// free, or waits; if nothing at all can run, the request admitted last is preempted; a
// request that does not fit into the empty pool ends with reason LENGTH.
#pragma once
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache.h"

namespace lcu {

struct SchedConfig {
    int max_num_seqs;       // running requests at a time (also bounded by state slots)
    int max_batch_tokens;   // tokens per step
    int prefill_chunk;      // most tokens of one prompt per step
    int max_model_len;      // most tokens a request may hold
};

enum FinishReason { NOT_FINISHED = 0, FINISH_EOS = 1, FINISH_MAX_STEPS = 2, FINISH_LENGTH = 3, FINISH_ABORTED = 4 };

struct PlanEntry {
    int64_t id;
    int start;        // index of the first token of this portion in the request's tokens
    int count;        // tokens in this portion
    int want_logits;  // 1: the portion reaches the request's last known token
};

struct SchedRequest {
    int64_t id = 0;
    std::vector<int> tokens;   // prompt, then generated tokens
    int prompt_len = 0;
    int computed = 0;          // tokens whose keys and values are in the cache
    int max_new = 0;
    int generated = 0;
    int keep = 0;              // keep the cache when finished (a later turn goes on from it)
    int reason = NOT_FINISHED;
    int preemptions = 0;
};

class Scheduler {
  public:
    Scheduler(const SchedConfig &cfg, CacheManager *cache) : cfg_(cfg), cache_(cache) {}

    int add(int64_t id, const int *tokens, int n, int max_new, int keep);
    // A kept, finished request goes on with more tokens.
    int extend(int64_t id, const int *tokens, int n, int max_new);
    int abort(int64_t id);
    // Forget a finished request (and its kept cache).
    int drop(int64_t id);

    // Decide the next step.  Requests that ended without running (too long) are in
    // `finished_now` afterwards.
    std::vector<PlanEntry> plan();
    // The step ran: its tokens are in the cache.
    void commit(const std::vector<PlanEntry> &plan);
    // A sampled token for a request whose portion wanted logits; `is_eos` ends it.
    // Returns the finish reason (NOT_FINISHED = 0 if it goes on).
    int append(int64_t id, int token, int is_eos);
    // The value of a token that was appended before it was known (the engine runs ahead of
    // its sampler's results).
    int set_token(int64_t id, int index, int token);
    // End a request from outside (an end-of-sequence token learned late): its tokens are cut to
    // n_tokens (if that is not negative) and a kept cache to what precedes the last of them, as if
    // the request had ended when that token was appended.  A request that ended by count at the
    // same token takes the new reason.  Where the cache cannot be cut back (a window has passed a
    // page that the shorter request would see, or the model keeps a state of fixed size), the
    // request gives up what cannot be cut (CacheManager::truncate_or_reset) and a later turn
    // computes it again from its tokens.
    int finish_now(int64_t id, int reason, int n_tokens);

    const SchedRequest *get(int64_t id) const;
    int n_waiting() const { return (int)waiting_.size(); }
    int n_running() const { return (int)running_.size(); }
    bool idle() const { return waiting_.empty() && running_.empty(); }
    std::vector<int64_t> take_finished();     // ids finished since the last call
    const std::vector<int64_t> &running() const { return running_; }
    int64_t total_preemptions() const { return preemptions_; }

  private:
    bool reserve_or_preempt(SchedRequest &r, int new_len, bool may_preempt, std::vector<PlanEntry> &plan);
    void preempt_last(std::vector<PlanEntry> &plan);
    void finish(SchedRequest &r, int reason);

    SchedConfig cfg_;
    CacheManager *cache_;
    std::unordered_map<int64_t, SchedRequest> reqs_;
    std::deque<int64_t> waiting_;
    std::vector<int64_t> running_;     // in admission order
    std::vector<int64_t> finished_;
    int64_t preemptions_ = 0;
    bool preempted_now_ = false;       // the plan being made has preempted a request
};

}  // namespace lcu
