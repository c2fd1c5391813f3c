// The scheduler's mechanics: which requests run in the next step, with how many tokens each, who is
// admitted and who gives pages back.  It knows a request as (id, number of prompt tokens, number of
// tokens so far, how many of them are in the cache, slot); the tokens themselves, sampling options
// and finish reasons stay with the Python request.
//
// Compared with the reference (crates/mach-model/src/continuous.rs:753-929, 943-1201): there every
// page of a request is reserved at admission and nothing is taken back from a running request; here
// pages are taken step by step, and when they run out the youngest running request is preempted: its
// pages and slot go back, it returns to the front of the waiting queue and is recomputed.
#pragma once
#include <deque>

#include "cache.hpp"

namespace mshost {

struct SchedulerError : std::invalid_argument {
    using std::invalid_argument::invalid_argument;
};

struct PlanItem {
    long id;
    int start, count;
    bool sample;  // the portion reaches the end of the request's tokens: its last row is sampled
};

struct StepPlan {
    std::vector<PlanItem> items;
    std::vector<long> preempted;
    std::vector<std::pair<long, int>> admitted;  // (id, slot)
};

class SchedulerCore {
public:
    SchedulerCore(CacheCore& cache, int max_batch_tokens, int chunk_size, int max_running, int max_positions)
        : cache_(cache), budget_(max_batch_tokens), chunk_(chunk_size > 0 ? chunk_size : max_batch_tokens),
          max_running_(std::min(max_running > 0 ? max_running : cache.max_requests(), cache.max_requests())),
          max_positions_(max_positions) {
        if (max_batch_tokens < 1) throw SchedulerError("max_batch_tokens must be at least 1");
    }
    int max_batch_tokens() const { return budget_; }
    int chunk_size() const { return chunk_; }
    int max_running() const { return max_running_; }

    // Refusals (continuous.rs:788-800 for the first two): an empty prompt, a prompt beyond the model's
    // positions, and a request that the pool could never hold.
    void add(long id, int prompt_len, int max_new) {
        if (prompt_len < 1) throw SchedulerError("empty prompt");
        if (max_new < 1) throw SchedulerError(cat("max_new ", max_new, " must be at least 1"));
        if (max_positions_ > 0 && prompt_len >= max_positions_)
            throw SchedulerError(cat("prompt of ", prompt_len, " tokens leaves no room within ", max_positions_, " positions"));
        int total = prompt_len + max_new - 1;  // the last generated token is never fed
        if (max_positions_ > 0) total = std::min(total, max_positions_);
        const int ps = cache_.page_size();
        for (int g = 0; g < cache_.num_groups(); ++g) {
            // a window group holds the pages that the keys [L - window + 1, L + n) of a step touch, n being a
            // portion at most; a group of all keys holds every page of the request
            int pages = (total + ps - 1) / ps;
            const int window = cache_.group_window(g);
            if (window > 0) pages = std::min(pages, (window + std::min(chunk_, budget_) - 1 + ps - 1) / ps + 1);
            if (pages > cache_.group_pages(g))
                throw SchedulerError(cat("request of up to ", total, " cached tokens needs ", pages, " pages at a time; group ",
                                         cache_.group_name(g), " has ", cache_.group_pages(g)));
        }
        if (reqs_.count(id)) throw SchedulerError(cat("request ", id, " exists already"));
        reqs_[id] = Req{id, prompt_len, prompt_len, 0, -1};
        waiting_.push_back(id);
    }
    bool has_work() const { return !waiting_.empty() || !running_.empty(); }
    std::vector<long> waiting() const { return {waiting_.begin(), waiting_.end()}; }
    std::vector<long> running() const { return running_; }
    int fed(long id) const { return reqs_.at(id).fed; }
    int slot(long id) const { return reqs_.at(id).slot; }
    bool decoding(long id) const { return reqs_.at(id).decoding(); }

    // The next step: every decoding request's token first, then prompt portions of running requests,
    // then newly admitted requests, under the token budget and the free pages.
    StepPlan schedule() {
        StepPlan plan;
        const int G = cache_.num_groups(), ps = cache_.page_size();
        // There are never more decoding requests than the budget holds: a request starts (and a prompt ends) only in
        // a step that had budget left for it beside every decoding request, so the sum never grows beyond it.  Checked
        // before anything is preempted, so that a refusal leaves the queues and the pages as they were.
        {
            int decoders = 0;
            for (long id : running_) decoders += reqs_.at(id).decoding();
            if (decoders > budget_)
                throw SchedulerError(cat(decoders, " requests decode under a budget of ", budget_, " tokens a step"));
        }
        while (true) {
            plan.items.clear();
            int budget = budget_;
            // 1. decoded tokens, oldest request first; they must all fit, or the youngest goes
            std::vector<int> need(G, 0);
            for (long id : running_) {
                const Req& r = reqs_.at(id);
                if (!r.decoding()) continue;
                auto n = cache_.pages_needed(r.slot, 1);
                for (int g = 0; g < G; ++g) need[g] += n[g];
            }
            bool short_of = false;
            for (int g = 0; g < G; ++g) short_of |= cache_.group_available(g) < need[g];
            if (short_of) {
                preempt_youngest(plan);
                continue;
            }
            for (long id : running_) {
                const Req& r = reqs_.at(id);
                if (!r.decoding()) continue;
                plan.items.push_back({id, r.fed, 1, true});
                --budget;
            }
            // 2. portions of prompts (or of a recomputation) already running, oldest first; an older
            //    request that lacks pages takes them from the youngest
            bool restart = false;
            for (long id : running_) {
                const Req& r = reqs_.at(id);
                if (r.decoding() || budget == 0) continue;
                const int n = std::min({r.n_tokens - r.fed, chunk_, budget});
                if (!cache_.can_extend(r.slot, n, reserved(plan))) {
                    if (id != running_.back()) {
                        preempt_youngest(plan);
                        restart = true;
                        break;
                    }
                    continue;
                }
                plan.items.push_back({id, r.fed, n, r.fed + n == r.n_tokens});
                budget -= n;
            }
            if (restart) continue;
            // 3. admission, first come first served
            while (!waiting_.empty() && budget > 0 && (int)running_.size() < max_running_ && cache_.slots_available() > 0) {
                Req& r = reqs_.at(waiting_.front());
                if (std::find(plan.preempted.begin(), plan.preempted.end(), r.id) != plan.preempted.end())
                    break;  // it lost its pages in this very step
                const int n = std::min({r.n_tokens, chunk_, budget});
                auto res = reserved(plan);
                bool fits = true;
                for (int g = 0; g < G; ++g) fits &= cache_.group_available(g) - res[g] >= (n + ps - 1) / ps;
                if (!fits) break;
                waiting_.pop_front();
                r.slot = cache_.admit();
                r.fed = 0;
                running_.push_back(r.id);
                plan.admitted.emplace_back(r.id, r.slot);
                plan.items.push_back({r.id, 0, n, n == r.n_tokens});
                budget -= n;
            }
            if (!plan.items.empty() || running_.empty()) return plan;
            // running requests exist but none can move: they hold each other's pages
            preempt_youngest(plan);
        }
    }

    // The step ran: every item's tokens are in the cache, and a sampled item has one token more.
    void advance(const std::vector<PlanItem>& items) {
        for (auto& it : items) {
            Req& r = reqs_.at(it.id);
            r.fed += it.count;
            if (it.sample) ++r.n_tokens;
        }
    }
    // The request ended or was cancelled: its pages and slot go back, and it is forgotten.
    bool finish(long id) {
        auto it = reqs_.find(id);
        if (it == reqs_.end()) return false;
        if (it->second.slot >= 0) cache_.release(it->second.slot);
        running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
        waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), id), waiting_.end());
        reqs_.erase(it);
        return true;
    }

private:
    struct Req {
        long id;
        int prompt_len, n_tokens, fed, slot;
        bool decoding() const { return fed == n_tokens - 1 && n_tokens > prompt_len; }
    };
    void preempt_youngest(StepPlan& plan) {
        const long id = running_.back();
        running_.pop_back();
        Req& r = reqs_.at(id);
        cache_.release(r.slot);
        r.slot = -1;
        r.fed = 0;
        waiting_.push_front(id);
        plan.preempted.push_back(id);
        plan.items.erase(std::remove_if(plan.items.begin(), plan.items.end(), [&](const PlanItem& i) { return i.id == id; }),
                         plan.items.end());
    }
    std::vector<int> reserved(const StepPlan& plan) const {
        std::vector<int> res(cache_.num_groups(), 0);
        for (auto& it : plan.items) {
            auto n = cache_.pages_needed(reqs_.at(it.id).slot, it.count);
            for (size_t g = 0; g < res.size(); ++g) res[g] += n[g];
        }
        return res;
    }

    CacheCore& cache_;
    int budget_, chunk_, max_running_, max_positions_;
    std::unordered_map<long, Req> reqs_;
    std::deque<long> waiting_;
    std::vector<long> running_;  // oldest first
};

}  // namespace mshost
