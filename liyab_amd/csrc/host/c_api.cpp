// The C interface of the host library (cache manager, step metadata), for the Python binding.
// Every function that can fail returns a Status (0 = ok) and leaves a message for
// liyab_host_last_error() on the calling thread.
#include <cstring>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"
#include "attention_plan.h"
#include "step_meta.h"

using namespace liyab_host;

static thread_local std::string g_error;

extern "C" {

const char* liyab_host_last_error() { return g_error.c_str(); }

// -- a pool on its own (used by tests) ----------------------------------------------
void* liyab_pool_create(int num_pages) { return num_pages > 0 ? new PagePool(num_pages) : nullptr; }
void liyab_pool_destroy(void* p) { delete static_cast<PagePool*>(p); }
int liyab_pool_allocate(void* p, int n, int32_t* out) { return static_cast<PagePool*>(p)->allocate(n, out, &g_error); }
int liyab_pool_release(void* p, const int32_t* pages, int n) { return static_cast<PagePool*>(p)->release(pages, n, &g_error); }
int liyab_pool_check(void* p) { return static_cast<PagePool*>(p)->check(&g_error); }
int liyab_pool_free_pages(void* p) { return static_cast<PagePool*>(p)->free_pages(); }
int liyab_pool_peak(void* p) { return static_cast<PagePool*>(p)->peak_in_use(); }

// -- the manager ------------------------------------------------------------------
void* liyab_cm_create(int n_groups, const int* windows, const int* num_pages, int page_size, int max_requests,
                      int max_positions) {
    if (n_groups < 0 || page_size <= 0 || max_requests <= 0 || max_positions <= 0) {
        g_error = "cache manager: page_size, max_requests and max_positions must be positive";
        return nullptr;
    }
    std::vector<GroupConfig> groups;
    for (int g = 0; g < n_groups; ++g) {
        if (num_pages[g] <= 0) {
            g_error = "a page pool needs at least one page";
            return nullptr;
        }
        groups.push_back({windows[g], num_pages[g]});
    }
    return new CacheManager(groups, page_size, max_requests, max_positions);
}
void liyab_cm_destroy(void* h) { delete static_cast<CacheManager*>(h); }
int liyab_cm_open(void* h, int* slot) { return static_cast<CacheManager*>(h)->open(slot, &g_error); }
int liyab_cm_close(void* h, int slot) { return static_cast<CacheManager*>(h)->close(slot, &g_error); }
int liyab_cm_length(void* h, int slot) { return static_cast<CacheManager*>(h)->length(slot); }
void liyab_cm_pages_needed(void* h, int slot, int new_length, int* out) {
    static_cast<CacheManager*>(h)->pages_needed(slot, new_length, out);
}
int liyab_cm_reserve(void* h, const int* slots, const int* new_lengths, int n) {
    return static_cast<CacheManager*>(h)->reserve(slots, new_lengths, n, &g_error);
}
// reserve for requests that each bring extra[i] more positions than they hold; their new lengths go to out
int liyab_cm_reserve_more(void* h, const int* slots, const int* extra, int n, int* new_lengths) {
    auto* m = static_cast<CacheManager*>(h);
    for (int i = 0; i < n; ++i) {
        if (!m->is_open(slots[i])) {
            g_error = "slot " + std::to_string(slots[i]) + " is not open";
            return kInvalidArgument;
        }
        new_lengths[i] = m->length(slots[i]) + extra[i];
    }
    return m->reserve(slots, new_lengths, n, &g_error);
}
int liyab_cm_commit(void* h, int slot, int new_length) { return static_cast<CacheManager*>(h)->commit(slot, new_length, &g_error); }
int liyab_cm_commit_many(void* h, const int* slots, const int* new_lengths, int n) {
    for (int i = 0; i < n; ++i)
        if (int s = static_cast<CacheManager*>(h)->commit(slots[i], new_lengths[i], &g_error)) return s;
    return kOk;
}
int liyab_cm_truncate(void* h, int slot, int length) { return static_cast<CacheManager*>(h)->truncate(slot, length, &g_error); }
const int32_t* liyab_cm_table_rows(void* h, int g) { return static_cast<CacheManager*>(h)->table_rows(g); }
int liyab_cm_table_length(void* h, int slot, int g) { return static_cast<CacheManager*>(h)->table_length(slot, g); }
int liyab_cm_max_blocks(void* h) { return static_cast<CacheManager*>(h)->max_blocks(); }
int liyab_cm_free_slots(void* h) { return static_cast<CacheManager*>(h)->free_slots(); }
int liyab_cm_free_pages(void* h, int g) { return static_cast<CacheManager*>(h)->pool(g).free_pages(); }
int liyab_cm_peak_in_use(void* h, int g) { return static_cast<CacheManager*>(h)->pool(g).peak_in_use(); }
int liyab_cm_check(void* h) { return static_cast<CacheManager*>(h)->check(&g_error); }

// -- a step's metadata --------------------------------------------------------------
int liyab_step_shape(void* h, int n_seqs, const int* slots, const int* q_lens, const int* want_counts, int pad_rows, StepShape* out) {
    return step_shape(*static_cast<CacheManager*>(h), n_seqs, slots, q_lens, want_counts, pad_rows, out, &g_error);
}
int liyab_step_fill(void* h, const StepShape* shape, const int* slots, const int* q_lens, const int64_t* tokens,
                    const int* want_counts, const int* wants, int vocab_size, int32_t* block) {
    return step_fill(*static_cast<CacheManager*>(h), *shape, slots, q_lens, tokens, want_counts, wants, vocab_size, block, &g_error);
}
// attention's own words of a step (attention_plan.h): counts[0] tiles, counts[1] single rows
void liyab_attn_counts(int n_seqs, const int* q_lens, int decode_q_len, int attn_tile, int* counts) {
    attn_counts(n_seqs, q_lens, decode_q_len, attn_tile, &counts[0], &counts[1]);
}
void liyab_attn_fill(int n_seqs, const int* q_lens, const int* first_pos, int decode_q_len, int attn_tile, int32_t* words) {
    attn_fill(n_seqs, q_lens, first_pos, decode_q_len, attn_tile, words);
}

// -- the scheduler --------------------------------------------------------------------
struct SchedulerHandle {
    Scheduler sched;
    std::vector<Scheduled> batch;
    std::vector<int> opened, preempted;
};

void* liyab_sched_create(void* manager, int max_num_seqs, int max_batched_tokens, int prefill_chunk) {
    if (manager == nullptr || max_num_seqs <= 0 || max_batched_tokens <= 0 || prefill_chunk <= 0) {
        g_error = "max_num_seqs, max_batched_tokens and prefill_chunk must be positive";
        return nullptr;
    }
    return new SchedulerHandle{Scheduler(static_cast<CacheManager*>(manager), max_num_seqs, max_batched_tokens, prefill_chunk), {}, {}, {}};
}
void liyab_sched_destroy(void* h) { delete static_cast<SchedulerHandle*>(h); }
int liyab_sched_add(void* h, int n_prompt, int max_tokens, int priority, int* id) {
    return static_cast<SchedulerHandle*>(h)->sched.add(n_prompt, max_tokens, priority, id, &g_error);
}
int liyab_sched_pressure(void* h) { return static_cast<SchedulerHandle*>(h)->sched.pressure() ? 1 : 0; }
// The step's batch; it stays valid until the next call. counts: [batch, opened, preempted].
int liyab_sched_schedule(void* h, const Scheduled** batch, const int** opened, const int** preempted, int* counts) {
    auto* s = static_cast<SchedulerHandle*>(h);
    const int rc = s->sched.schedule(&s->batch, &s->opened, &s->preempted, &g_error);
    *batch = s->batch.data();
    *opened = s->opened.data();
    *preempted = s->preempted.data();
    counts[0] = static_cast<int>(s->batch.size());
    counts[1] = static_cast<int>(s->opened.size());
    counts[2] = static_cast<int>(s->preempted.size());
    return rc;
}
void liyab_sched_advance(void* h, const Scheduled* batch, int n) { static_cast<SchedulerHandle*>(h)->sched.advance(batch, n); }
// One sampled token per request named; reasons[i] as Scheduler::token returns it.
void liyab_sched_tokens(void* h, const int* ids, const int* is_stop, int n, int* reasons) {
    auto& s = static_cast<SchedulerHandle*>(h)->sched;
    for (int i = 0; i < n; ++i) reasons[i] = s.token(ids[i], is_stop[i] != 0);
}
int liyab_sched_finish(void* h, int id) { return static_cast<SchedulerHandle*>(h)->sched.finish(id, &g_error); }
// what: 0 state, 1 computed, 2 pending, 3 generated, 4 preemptions, 5 slot, 6 priority
int liyab_sched_get(void* h, int id, int what) {
    const auto& s = static_cast<SchedulerHandle*>(h)->sched;
    if (id < 0) return -1;
    switch (what) {
        case 0: return s.state(id);
        case 1: return s.computed(id);
        case 2: return s.pending(id);
        case 3: return s.n_generated(id);
        case 4: return s.preemptions(id);
        case 5: return s.slot(id);
        case 6: return s.priority(id);
        default: return -1;
    }
}
// ids of the running requests in order of admission (which = 0) or of the waiting ones in queue order (1)
int liyab_sched_list(void* h, int which, int* out, int cap) {
    const auto& s = static_cast<SchedulerHandle*>(h)->sched;
    int n = 0;
    if (which == 0) {
        for (int id : s.running())
            if (n < cap) out[n++] = id;
    } else {
        for (int id : s.waiting())
            if (n < cap) out[n++] = id;
    }
    return n;
}
void liyab_sched_stats(void* h, long long* out) {
    const SchedulerStats& st = static_cast<SchedulerHandle*>(h)->sched.stats();
    out[0] = st.steps;
    out[1] = st.batched_tokens;
    out[2] = st.prefill_tokens;
    out[3] = st.decode_tokens;
    out[4] = st.preemptions;
}

}  // extern "C"
