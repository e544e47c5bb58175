// The C interface of the host library (cache manager, step metadata), for the Python binding.
// Every function that can fail returns a Status (0 = ok) and leaves a message for
// liyab_host_last_error() on the calling thread.
#include <cstring>
#include <string>
#include <vector>

#include "cache_manager.h"
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
int liyab_step_shape(void* h, int n_seqs, const int* slots, const int* q_lens, const int* want_counts, int decode_q_len,
                     int attn_tile, StepShape* out) {
    return step_shape(*static_cast<CacheManager*>(h), n_seqs, slots, q_lens, want_counts, decode_q_len, attn_tile, out, &g_error);
}
int liyab_step_fill(void* h, const StepShape* shape, const int* slots, const int* q_lens, const int64_t* tokens,
                    const int* want_counts, const int* wants, int vocab_size, int decode_q_len, int attn_tile, int32_t* block) {
    return step_fill(*static_cast<CacheManager*>(h), *shape, slots, q_lens, tokens, want_counts, wants, vocab_size, decode_q_len,
                     attn_tile, block, &g_error);
}

}  // extern "C"
