// The scheduler's decisions on the host: admission, prompt portions under a token budget,
// decoding, finishing, and what happens when pages run out.
//
// The reference schedules by threads: each generating thread submits the pass it needs and one
// of them runs the merged batch (src/core/engine.cpp:1842-2041); prompts go in portions of 256
// tokens (:2863-2864), a decoding request brings one token a pass (:4311-4334), and a request
// stops at an end-of-generation token, at max_tokens or on its callback's word (:4351-4393).
// When the cache cannot grow the reference fails the request (src/core/kv_cache.cpp:249-252,
// src/core/engine.cpp:3878-3882). Here one loop owns all requests:
//
//   * every step first gives each decoding request its one token, then hands the rest of the
//     token budget to prompt portions in order of admission (a portion is as small as the budget
//     leaves, down to one token), then admits waiting requests, the higher priority first and
//     first come, first served among equals, while a request slot, budget and pages for the
//     first portion are there (the reference has two classes, foreground and background, and
//     lets foreground requests go first: src/core/engine.cpp:1936-1945; here a priority is any
//     integer, the larger the sooner, and it orders admission only);
//   * when a request cannot get its pages, the most recently admitted running request is
//     preempted: its pages and slot go back, it returns to the waiting queue ahead of every
//     request of its own or a lower priority and is
//     recomputed from its prompt plus what it has generated. A request is never preempted for
//     its own sake by a later one, and a request that could not fit the pool alone is refused
//     on arrival.
//
// A step may be launched before the tokens of the step before have reached the host: a request
// then has a token "pending" (sampled on the device, not yet known here), which counts as one
// of its tokens; a request with a pending token is never preempted (the caller reads the tokens
// first whenever pressure() says pages may run short).
#pragma once

#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace liyab_host {

enum RequestState : int { kWaiting = 0, kRunning = 1, kFinished = 2 };
enum FinishReason : int { kGoesOn = 0, kStop = 1, kLength = 2, kContext = 3, kAlreadyFinished = -1 };

struct Scheduled {
    int id;           // the request
    int slot;         // its state slot
    int first;        // index of the first token run in this step
    int count;        // how many tokens
    int wants_logits; // the portion reaches the request's last token
};

struct SchedulerStats {
    long long steps, batched_tokens, prefill_tokens, decode_tokens, preemptions;
};

class Scheduler {
public:
    Scheduler(CacheManager* manager, int max_num_seqs, int max_batched_tokens, int prefill_chunk);

    // A new request of n_prompt tokens that may generate max_tokens; its id goes to *id. It
    // waits behind every request of its own or a higher priority.
    Status add(int n_prompt, int max_tokens, int priority, int* id, std::string* err);
    bool has_unfinished() const { return !waiting_.empty() || !running_.empty(); }
    // Whether the request's pending token is its last whatever it turns out to be.
    bool draining(int id) const;
    // Whether the running requests' next portions may not all fit the free pages.
    bool pressure() const;
    // Chooses this step's batch; opens and preempts requests accordingly (ids in the order it
    // happened). Pages are only counted here; the step function maps them.
    Status schedule(std::vector<Scheduled>* batch, std::vector<int>* opened, std::vector<int>* preempted, std::string* err);
    // The step has been launched: its tokens are in the cache; requests whose portion reached
    // their last token have a token pending.
    void advance(const Scheduled* batch, int n);
    // A sampled token of the request has reached the host. Returns why the request ends with it
    // (it is finished then), kGoesOn, or kAlreadyFinished when the request ended meanwhile.
    int token(int id, bool is_stop_token);
    // Ends a request for any other reason (callback, cancel); gives back what it holds.
    Status finish(int id, std::string* err);

    // A finished request is forgotten (ids are never given out twice): it reads as finished,
    // holding nothing.
    int state(int id) const { const Request* r = find(id); return r ? r->state : kFinished; }
    int computed(int id) const { const Request* r = find(id); return r ? r->computed : 0; }
    int pending(int id) const { const Request* r = find(id); return r ? r->pending : 0; }
    int n_generated(int id) const { const Request* r = find(id); return r ? r->n_generated : 0; }
    int preemptions(int id) const { const Request* r = find(id); return r ? r->preemptions : 0; }
    int slot(int id) const { const Request* r = find(id); return r ? r->slot : -1; }
    int priority(int id) const { const Request* r = find(id); return r ? r->priority : 0; }
    int n_requests() const { return static_cast<int>(reqs_.size()); }  // the unfinished ones
    const std::vector<int>& running() const { return running_; }
    const std::deque<int>& waiting() const { return waiting_; }
    const SchedulerStats& stats() const { return stats_; }

private:
    struct Request {
        int n_prompt, max_tokens;
        int n_generated = 0, pending = 0, computed = 0;
        int state = kWaiting, slot = -1, preemptions = 0, priority = 0;
        int n_tokens() const { return n_prompt + n_generated + pending; }
        int remaining() const { return n_tokens() - computed; }
    };
    int extra_pages(const Request& r, int count) const {
        // new pages per group for positions [computed, computed + count): the request's pages reach
        // its computed length at least, so this never undercounts
        const int p = m_->page_size();
        return (r.computed + count + p - 1) / p - (r.computed + p - 1) / p;
    }
    Status preempt(int id, std::string* err);
    const Request* find(int id) const {
        auto it = reqs_.find(id);
        return it == reqs_.end() ? nullptr : &it->second;
    }
    Request& req(int id) { return reqs_.at(id); }
    const Request& req(int id) const { return reqs_.at(id); }

    CacheManager* m_;
    int max_num_seqs_, max_batched_tokens_, prefill_chunk_;
    std::unordered_map<int, Request> reqs_;  // waiting and running requests by id; a finished one is erased
    int next_id_ = 0;
    std::deque<int> waiting_;
    std::vector<int> running_;  // in order of admission
    SchedulerStats stats_{};
};

}  // namespace liyab_host
