#include "sched.h"

#include <algorithm>

namespace lcu {

int Scheduler::add(int64_t id, const int *tokens, int n, int max_new, int keep) {
    if (reqs_.count(id)) return CACHE_DUPLICATE_REQUEST;
    if (n <= 0 || max_new < 0) return CACHE_BAD_ARGUMENT;
    SchedRequest r;
    r.id = id;
    r.tokens.assign(tokens, tokens + n);
    r.prompt_len = n;
    r.max_new = max_new;
    r.keep = keep;
    reqs_.emplace(id, std::move(r));
    waiting_.push_back(id);
    return CACHE_OK;
}

int Scheduler::extend(int64_t id, const int *tokens, int n, int max_new) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    SchedRequest &r = it->second;
    if (r.reason == NOT_FINISHED || n <= 0) return CACHE_BAD_ARGUMENT;
    r.tokens.insert(r.tokens.end(), tokens, tokens + n);
    r.prompt_len = (int)r.tokens.size();
    r.max_new = max_new;
    r.generated = 0;
    r.reason = NOT_FINISHED;
    if (!cache_->has(id) || cache_->get(id)->len < r.computed) r.computed = 0;       // the cache was not kept (or was taken away)
    waiting_.push_back(id);
    return CACHE_OK;
}

const SchedRequest *Scheduler::get(int64_t id) const {
    auto it = reqs_.find(id);
    return it == reqs_.end() ? nullptr : &it->second;
}

void Scheduler::finish(SchedRequest &r, int reason) {
    r.reason = reason;
    running_.erase(std::remove(running_.begin(), running_.end(), r.id), running_.end());
    waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), r.id), waiting_.end());
    if (!(r.keep && reason != FINISH_ABORTED) && cache_->has(r.id)) cache_->release(r.id);
    finished_.push_back(r.id);
}

int Scheduler::abort(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    if (it->second.reason == NOT_FINISHED) finish(it->second, FINISH_ABORTED);
    else if (cache_->has(id)) cache_->release(id);
    return CACHE_OK;
}

int Scheduler::drop(int64_t id) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    if (it->second.reason == NOT_FINISHED) return CACHE_BAD_ARGUMENT;
    if (cache_->has(id)) cache_->release(id);
    reqs_.erase(it);
    finished_.erase(std::remove(finished_.begin(), finished_.end(), id), finished_.end());
    return CACHE_OK;
}

std::vector<int64_t> Scheduler::take_finished() {
    std::vector<int64_t> out;
    out.swap(finished_);
    return out;
}

// The running request admitted last gives its pages back and waits again, first in line.
void Scheduler::preempt_last(std::vector<PlanEntry> &plan) {
    const int64_t victim = running_.back();
    running_.pop_back();
    SchedRequest &v = reqs_.at(victim);
    plan.erase(std::remove_if(plan.begin(), plan.end(), [&](const PlanEntry &e) { return e.id == victim; }), plan.end());
    if (cache_->has(victim)) cache_->release(victim);
    v.computed = 0;
    v.preemptions++;
    preemptions_++;
    preempted_now_ = true;
    waiting_.push_front(victim);
}

// Pages for r up to new_len; with may_preempt, later-admitted requests are preempted until
// it fits.  False: r itself is no longer running (preempted or ended), or, without
// may_preempt, the pages are not there.
bool Scheduler::reserve_or_preempt(SchedRequest &r, int new_len, bool may_preempt, std::vector<PlanEntry> &plan) {
    for (;;) {
        const int st = cache_->reserve(r.id, new_len);
        if (st == CACHE_OK) return true;
        if (st != CACHE_NO_PAGES || !may_preempt) return false;
        if (running_.back() == r.id) {
            if (running_.size() == 1) {
                // alone and still too large for the pool
                finish(r, FINISH_LENGTH);
                return false;
            }
            preempt_last(plan);
            return false;
        }
        preempt_last(plan);
    }
}

std::vector<PlanEntry> Scheduler::plan() {
    std::vector<PlanEntry> plan;
    preempted_now_ = false;
    for (;;) {
        plan.clear();
        int budget = cfg_.max_batch_tokens;

        // 1. decoding requests: one token each, in admission order
        for (size_t i = 0; i < running_.size() && budget > 0;) {
            SchedRequest &r = reqs_.at(running_[i]);
            const int pending = (int)r.tokens.size() - r.computed;
            if (pending != 1 || r.computed < r.prompt_len) { ++i; continue; }
            const int64_t id = r.id;
            if (reserve_or_preempt(r, r.computed + 1, true, plan)) {
                plan.push_back({id, r.computed, 1, 1});
                --budget;
                ++i;
            } else if (i < running_.size() && running_[i] == id) {
                ++i;      // cannot happen (a failed request leaves the list); keeps the loop finite
            }
        }
        // 2. prompt portions of running requests
        for (size_t i = 0; i < running_.size() && budget > 0; ++i) {
            SchedRequest &r = reqs_.at(running_[i]);
            const int pending = (int)r.tokens.size() - r.computed;
            if (pending == 1 && r.computed >= r.prompt_len) continue;
            int n = std::min({pending, budget, cfg_.prefill_chunk});
            n = std::min(n, cache_->max_reservable(r.id, r.computed + n) - r.computed);
            if (n <= 0) continue;                      // waits for pages
            if (cache_->reserve(r.id, r.computed + n) != CACHE_OK) continue;
            plan.push_back({r.id, r.computed, n, r.computed + n == (int)r.tokens.size()});
            budget -= n;
        }
        // 3. admission, first come first served; not in a round that had to preempt (the pages
        //    that the victim gave back would go straight to it again)
        while (!preempted_now_ && !waiting_.empty() && budget > 0 && (int)running_.size() < cfg_.max_num_seqs) {
            SchedRequest &r = reqs_.at(waiting_.front());
            if ((int)r.tokens.size() > cfg_.max_model_len) {
                finish(r, FINISH_LENGTH);
                continue;
            }
            if (!cache_->has(r.id)) {
                if (cache_->add(r.id) != CACHE_OK) break;          // no state slot
            }
            const int pending = (int)r.tokens.size() - r.computed;
            int n = std::min({pending, budget, cfg_.prefill_chunk});
            n = std::min(n, cache_->max_reservable(r.id, r.computed + n) - r.computed);
            if (n <= 0 || cache_->reserve(r.id, r.computed + n) != CACHE_OK) {
                if (running_.empty() && plan.empty() && r.computed == 0) {
                    // the pool is as empty as it gets and the first page does not fit
                    if (cache_->max_reservable(r.id, 1) < 1) { finish(r, FINISH_LENGTH); continue; }
                }
                if (r.computed == 0) cache_->release(r.id);        // give the slot back while it waits
                break;
            }
            waiting_.pop_front();
            running_.push_back(r.id);
            plan.push_back({r.id, r.computed, n, r.computed + n == (int)r.tokens.size()});
            budget -= n;
        }
        if (!plan.empty() || running_.empty()) break;
        // Requests are running and none can take a step: all wait for pages that only they
        // hold.  The one admitted last gives way; then plan once more.
        if (running_.size() == 1) {
            finish(reqs_.at(running_.back()), FINISH_LENGTH);
        } else {
            preempt_last(plan);
        }
        // plan again: each such round takes one request out of the running list, so it ends
    }
    return plan;
}

void Scheduler::commit(const std::vector<PlanEntry> &plan) {
    for (const auto &e : plan) {
        auto it = reqs_.find(e.id);
        if (it == reqs_.end() || it->second.reason != NOT_FINISHED) continue;
        it->second.computed = e.start + e.count;
        cache_->commit(e.id);
    }
}

int Scheduler::append(int64_t id, int token, int is_eos) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    SchedRequest &r = it->second;
    if (r.reason != NOT_FINISHED) return r.reason;
    r.tokens.push_back(token);
    r.generated++;
    if (is_eos) finish(r, FINISH_EOS);
    else if (r.generated >= r.max_new) finish(r, FINISH_MAX_STEPS);
    else if ((int)r.tokens.size() >= cfg_.max_model_len) finish(r, FINISH_LENGTH);
    return r.reason;
}

}  // namespace lcu

namespace lcu {

int Scheduler::set_token(int64_t id, int index, int token) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    if (index < 0 || index >= (int)it->second.tokens.size()) return CACHE_BAD_ARGUMENT;
    it->second.tokens[index] = token;
    return CACHE_OK;
}

int Scheduler::finish_now(int64_t id, int reason, int n_tokens) {
    auto it = reqs_.find(id);
    if (it == reqs_.end()) return CACHE_UNKNOWN_REQUEST;
    SchedRequest &r = it->second;
    if (n_tokens > (int)r.tokens.size() || n_tokens == 0) return CACHE_BAD_ARGUMENT;
    if (r.reason == FINISH_ABORTED) return r.reason;
    if (n_tokens > 0) {
        r.generated -= (int)r.tokens.size() - n_tokens;
        r.tokens.resize(n_tokens);
        if (r.computed > n_tokens - 1) {
            r.computed = n_tokens - 1;
            if (cache_->has(id) && cache_->get(id)->len > r.computed) {
                // What was computed beyond the end may not be there to take back: a window has given back a
                // page that the shorter request would still see, or the model keeps a state that has folded
                // the tokens in.  Then the request gives up what cannot be cut (its other pages stay its
                // own) and, if it goes on (a kept request's next turn), is computed again from its tokens.
                const int st = cache_->truncate_or_reset(id, r.computed);
                if (st == CACHE_RESET) {
                    r.computed = 0;
                } else if (st != CACHE_OK) {
                    cache_->release(id);
                    r.computed = 0;
                }
            }
        }
    }
    if (r.reason == NOT_FINISHED) finish(r, reason);
    else r.reason = reason;
    return r.reason;
}

}  // namespace lcu
