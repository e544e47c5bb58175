// The cache manager's bookkeeping on the host: page pools, block tables, state slots.
//
// What the reference's KvCache does for one context (include/liyab/kv_cache.h,
// src/core/kv_cache.cpp): fixed pages of `page_size` positions mapped on demand
// (reserve, kv_cache.cpp:249-265), a table from logical page to pool page per
// layer group (kv_cache.h:358-365), groups of layers by what they keep: every
// position, or a window that gives older pages back as the context advances
// (kv_cache.h:10-23, kv_cache.cpp:474-487), and counters (kv_cache.h:347-352).
// Differences, all deliberate: one pool per group is shared by every live
// request (the reference gives each context a pool of its own,
// src/core/transformer.cpp:6529-6545), so pages a finished request gives back
// are used again by the next; pages are not zeroed when mapped (readers mask by
// position); a request that cannot get its pages changes nothing and the caller
// decides, where the reference fails the pass (kv_cache.cpp:192-197).
//
// Requests are known here by their state slot, 0 <= slot < max_requests; the
// caller keeps the map from its own request ids to slots.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace liyab_host {

constexpr int32_t kUnmapped = -1;

enum Status : int {
    kOk = 0,
    kInvalidArgument = 1,
    kOutOfPages = 2,
    kContextFull = 3,
    kBusy = 4,
    kInternal = 5,  // an invariant does not hold
};

// Page ids 0..n-1 with a free stack; a page is held by at most one owner.
class PagePool {
public:
    explicit PagePool(int num_pages);
    int num_pages() const { return num_pages_; }
    int free_pages() const { return static_cast<int>(free_.size()); }
    int pages_in_use() const { return num_pages_ - free_pages(); }
    int peak_in_use() const { return peak_; }
    // n pages into out (lowest ids first from a fresh pool; the most recently freed first after that)
    Status allocate(int n, int32_t* out, std::string* err);
    Status release(const int32_t* pages, int n, std::string* err);
    Status check(std::string* err) const;

private:
    int num_pages_;
    std::vector<int32_t> free_;
    std::vector<uint8_t> held_;
    int peak_ = 0;
};

struct GroupConfig {
    int window;     // 0: every position is kept; W > 0: only the last W are read
    int num_pages;
};

class CacheManager {
public:
    CacheManager(const std::vector<GroupConfig>& groups, int page_size, int max_requests, int max_positions);

    int n_groups() const { return static_cast<int>(pools_.size()); }
    int page_size() const { return page_size_; }
    int max_blocks() const { return max_blocks_; }
    int max_requests() const { return max_requests_; }
    int max_positions() const { return max_positions_; }
    const PagePool& pool(int g) const { return pools_[g]; }
    int window(int g) const { return windows_[g]; }
    int free_slots() const { return static_cast<int>(free_slots_.size()); }

    Status open(int* slot, std::string* err);
    Status close(int slot, std::string* err);
    bool is_open(int slot) const { return slot >= 0 && slot < max_requests_ && reqs_[slot].open; }
    int length(int slot) const { return reqs_[slot].length; }
    // new pages per group that reserve(slot, new_length) would take
    void pages_needed(int slot, int new_length, int* out) const;
    // Maps pages so that each request can hold new_lengths[i] positions: all or nothing.
    Status reserve(const int* slots, const int* new_lengths, int n, std::string* err);
    // The request now holds new_length positions; windowed groups give back the pages no
    // later query can see (a query at p >= length reads [p - W + 1, p]).
    Status commit(int slot, int new_length, std::string* err);
    // Forgets positions >= length; pages wholly past it are given back (kv_cache.cpp:418-439).
    Status truncate(int slot, int length, std::string* err);
    // int32 [max_requests, max_blocks] of group g: the block table of the request in each slot
    const int32_t* table_rows(int g) const { return table_rows_[g].data(); }
    int table_length(int slot, int g) const { return reqs_[slot].mapped[g]; }
    Status check(std::string* err) const;

private:
    struct Request {
        bool open = false;
        int length = 0;                 // positions committed
        std::vector<int> mapped;        // per group: logical pages in the table (mapped or released)
        std::vector<int> first_kept;    // per group: first logical page still mapped
    };
    int pages_for(int n_positions) const { return (n_positions + page_size_ - 1) / page_size_; }
    int32_t* row(int g, int slot) { return table_rows_[g].data() + static_cast<size_t>(slot) * max_blocks_; }
    const int32_t* row(int g, int slot) const { return table_rows_[g].data() + static_cast<size_t>(slot) * max_blocks_; }

    int page_size_, max_requests_, max_positions_, max_blocks_;
    std::vector<int> windows_;
    std::vector<PagePool> pools_;
    std::vector<Request> reqs_;
    std::vector<int> free_slots_;
    std::vector<std::vector<int32_t>> table_rows_;
};

}  // namespace liyab_host
