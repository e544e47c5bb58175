#include "scheduler.h"

#include <algorithm>

namespace liyab_host {

static Status fail(std::string* err, Status s, const std::string& msg) {
    if (err != nullptr) *err = msg;
    return s;
}

Scheduler::Scheduler(CacheManager* manager, int max_num_seqs, int max_batched_tokens, int prefill_chunk)
    : m_(manager), max_num_seqs_(std::min(max_num_seqs, manager->max_requests())), max_batched_tokens_(max_batched_tokens),
      prefill_chunk_(prefill_chunk) {}

Status Scheduler::add(int n_prompt, int max_tokens, int priority, int* id, std::string* err) {
    if (n_prompt <= 0) return fail(err, kInvalidArgument, "the prompt is empty");  // src/core/engine.cpp:3867-3871
    if (max_tokens <= 0) return fail(err, kInvalidArgument, "max_tokens must be positive");
    if (n_prompt >= m_->max_positions() + 1)
        return fail(err, kInvalidArgument, "the prompt has " + std::to_string(n_prompt) + " tokens; the context holds " +
                                               std::to_string(m_->max_positions()));
    // the most positions it can come to hold: every token but the last sampled one is run
    const int most = std::min(n_prompt + max_tokens - 1, m_->max_positions());
    const int need = (most + m_->page_size() - 1) / m_->page_size();
    for (int g = 0; g < m_->n_groups(); ++g)
        if (m_->window(g) <= 0 && need > m_->pool(g).num_pages())
            return fail(err, kOutOfPages, "the request may need " + std::to_string(need) + " pages; the pool has " +
                                              std::to_string(m_->pool(g).num_pages()) + " in all");
    Request r;
    r.n_prompt = n_prompt;
    r.max_tokens = max_tokens;
    r.priority = priority;
    *id = next_id_++;
    reqs_.emplace(*id, r);
    // behind every waiting request of its own or a higher priority
    auto at = waiting_.begin();
    while (at != waiting_.end() && req(*at).priority >= priority) ++at;
    waiting_.insert(at, *id);
    return kOk;
}

bool Scheduler::draining(int id) const {
    if (find(id) == nullptr) return false;
    const Request& r = req(id);
    return r.pending > 0 && (r.n_generated + r.pending >= r.max_tokens || r.n_tokens() > m_->max_positions());
}

bool Scheduler::pressure() const {
    const int G = m_->n_groups(), page = m_->page_size();
    int free = G > 0 ? m_->pool(0).free_pages() : 0;
    for (int g = 1; g < G; ++g) free = std::min(free, m_->pool(g).free_pages());
    // a portion of c tokens takes at most ceil(c / page) + 1 new pages of a group
    long long bound = 0;
    for (int id : running_) {
        const int count = std::min(req(id).remaining(), prefill_chunk_);
        if (count > 0) bound += (count + page - 1) / page + 1;
    }
    if (bound <= free) return false;
    std::vector<int> need(static_cast<size_t>(G), 0), extra(static_cast<size_t>(G));
    for (int id : running_) {
        const Request& r = req(id);
        const int count = std::min(r.remaining(), prefill_chunk_);
        if (count <= 0) continue;
        m_->pages_needed(r.slot, r.computed + count, extra.data());
        for (int g = 0; g < G; ++g) need[g] += extra[g];
    }
    for (int g = 0; g < G; ++g)
        if (need[g] > m_->pool(g).free_pages()) return true;
    return false;
}

Status Scheduler::preempt(int id, std::string* err) {
    Request& r = req(id);
    if (r.pending > 0)
        return fail(err, kInternal, "a request with a pending token cannot be preempted: read the tokens first");
    if (Status s = m_->close(r.slot, err)) return s;
    running_.erase(std::find(running_.begin(), running_.end(), id));
    r.slot = -1;
    r.computed = 0;
    r.state = kWaiting;
    r.preemptions += 1;
    stats_.preemptions += 1;
    // ahead of every waiting request of its own or a lower priority
    auto at = waiting_.begin();
    while (at != waiting_.end() && req(*at).priority > r.priority) ++at;
    waiting_.insert(at, id);
    return kOk;
}

Status Scheduler::schedule(std::vector<Scheduled>* batch, std::vector<int>* opened, std::vector<int>* preempted, std::string* err) {
    batch->clear();
    opened->clear();
    preempted->clear();
    const int G = m_->n_groups();
    int budget = max_batched_tokens_;
    int need = 0;  // pages this step's batch takes so far: the same count in every group
    auto min_free = [&]() {
        int f = G > 0 ? m_->pool(0).free_pages() : (1 << 30);
        for (int g = 1; g < G; ++g) f = std::min(f, m_->pool(g).free_pages());
        return f;
    };
    int free = min_free();  // read again whenever a request is preempted
    auto fits = [&](const Request& r, int count) { return need + extra_pages(r, count) <= free; };
    auto take = [&](int id, int count) {
        Request& r = req(id);
        need += extra_pages(r, count);
        batch->push_back({id, r.slot, r.computed, count, r.computed + count == r.n_tokens() ? 1 : 0});
        budget -= count;
    };

    // running requests: decoding ones first, then prompt portions, each in order of admission
    std::vector<int> order;
    for (int pass = 0; pass < 2; ++pass)
        for (int id : running_) {
            if (draining(id)) continue;
            const int rem = req(id).remaining();
            if ((pass == 0 && rem == 1) || (pass == 1 && rem > 1)) order.push_back(id);
        }
    for (int id : order) {
        Request& r = req(id);
        if (r.state != kRunning || budget <= 0) continue;
        int count = std::min({r.remaining(), prefill_chunk_, budget});
        while (!fits(r, count)) {
            const int victim = running_.back();
            if (victim == id) {
                // nobody later to take pages from: shrink the portion or wait
                while (count > 1 && !fits(r, count)) --count;
                if (!fits(r, count)) count = 0;
                break;
            }
            for (size_t i = 0; i < batch->size();) {
                if ((*batch)[i].id == victim) {
                    need -= extra_pages(req(victim), (*batch)[i].count);
                    budget += (*batch)[i].count;
                    batch->erase(batch->begin() + static_cast<long>(i));
                } else {
                    ++i;
                }
            }
            if (Status s = preempt(victim, err)) return s;
            preempted->push_back(victim);
            free = min_free();
        }
        if (count > 0 && r.state == kRunning) take(id, count);
    }
    // admission: the queue's order (priority, then first come first served)
    while (!waiting_.empty() && static_cast<int>(running_.size()) < max_num_seqs_ && budget > 0) {
        const int id = waiting_.front();
        Request& r = req(id);
        const int count = std::min({r.remaining(), prefill_chunk_, budget});
        const int pages = (count + m_->page_size() - 1) / m_->page_size();
        if (m_->free_slots() == 0 || need + pages > free) break;
        if (Status s = m_->open(&r.slot, err)) return s;
        opened->push_back(id);
        waiting_.pop_front();
        r.state = kRunning;
        running_.push_back(id);
        take(id, count);
    }
    if (batch->empty() && has_unfinished()) {
        bool any_pending = false;
        for (int id : running_) any_pending = any_pending || req(id).pending > 0;
        if (!any_pending)
            return fail(err, kOutOfPages, "no request can make progress: the page pool is too small for any of them");
    }
    stats_.steps += 1;
    for (const Scheduled& s : *batch) {
        stats_.batched_tokens += s.count;
        if (s.count == 1 && s.wants_logits && req(s.id).n_generated > 0) stats_.decode_tokens += 1;
    }
    stats_.prefill_tokens = stats_.batched_tokens - stats_.decode_tokens;
    return kOk;
}

void Scheduler::advance(const Scheduled* batch, int n) {
    for (int i = 0; i < n; ++i) {
        Request& r = req(batch[i].id);
        r.computed += batch[i].count;
        if (batch[i].wants_logits) r.pending += 1;
    }
}

int Scheduler::token(int id, bool is_stop_token) {
    if (find(id) == nullptr) return kAlreadyFinished;
    Request& r = req(id);
    r.pending -= 1;
    r.n_generated += 1;
    int reason = kGoesOn;
    if (is_stop_token) reason = kStop;
    else if (r.n_generated >= r.max_tokens) reason = kLength;
    else if (r.n_prompt + r.n_generated > m_->max_positions()) reason = kContext;  // the next token would pass the last position
    if (reason != kGoesOn) finish(id, nullptr);
    return reason;
}

Status Scheduler::finish(int id, std::string* err) {
    if (find(id) == nullptr) return kOk;  // finished before
    Request& r = req(id);
    if (r.state == kRunning) {
        if (Status s = m_->close(r.slot, err)) return s;
        running_.erase(std::find(running_.begin(), running_.end(), id));
        r.slot = -1;
    } else if (r.state == kWaiting) {
        waiting_.erase(std::find(waiting_.begin(), waiting_.end(), id));
    }
    reqs_.erase(id);
    return kOk;
}

}  // namespace liyab_host
