#include "cache_manager.h"

#include <algorithm>

namespace liyab_host {

static Status fail(std::string* err, Status s, const std::string& msg) {
    if (err != nullptr) *err = msg;
    return s;
}

PagePool::PagePool(int num_pages) : num_pages_(num_pages), held_(static_cast<size_t>(num_pages), 0) {
    free_.reserve(static_cast<size_t>(num_pages));
    for (int p = num_pages - 1; p >= 0; --p) free_.push_back(p);  // the back of the stack is page 0
}

Status PagePool::allocate(int n, int32_t* out, std::string* err) {
    if (n > free_pages())
        return fail(err, kOutOfPages, std::to_string(n) + " pages wanted, " + std::to_string(free_pages()) + " free of " +
                                          std::to_string(num_pages_));
    for (int i = 0; i < n; ++i) {
        const int32_t p = free_.back();
        free_.pop_back();
        if (held_[p]) return fail(err, kInternal, "page " + std::to_string(p) + " handed out twice");
        held_[p] = 1;
        out[i] = p;
    }
    peak_ = std::max(peak_, pages_in_use());
    return kOk;
}

Status PagePool::release(const int32_t* pages, int n, std::string* err) {
    for (int i = 0; i < n; ++i) {
        const int32_t p = pages[i];
        if (p < 0 || p >= num_pages_ || !held_[p]) return fail(err, kInternal, "page " + std::to_string(p) + " freed but not held");
        held_[p] = 0;
        free_.push_back(p);  // the most recently freed is used first
    }
    return kOk;
}

Status PagePool::check(std::string* err) const {
    std::vector<uint8_t> seen(static_cast<size_t>(num_pages_), 0);
    for (int32_t p : free_) {
        if (p < 0 || p >= num_pages_) return fail(err, kInternal, "a free page id is out of range");
        if (seen[p]) return fail(err, kInternal, "a page is on the free list twice");
        seen[p] = 1;
        if (held_[p]) return fail(err, kInternal, "page " + std::to_string(p) + " is free and held");
    }
    int held = 0;
    for (uint8_t h : held_) held += h;
    if (held + free_pages() != num_pages_) return fail(err, kInternal, "a page was lost");
    return kOk;
}

CacheManager::CacheManager(const std::vector<GroupConfig>& groups, int page_size, int max_requests, int max_positions)
    : page_size_(page_size), max_requests_(max_requests), max_positions_(max_positions),
      max_blocks_(std::max(1, (max_positions + page_size - 1) / page_size)), reqs_(static_cast<size_t>(max_requests)) {
    for (const GroupConfig& g : groups) {
        windows_.push_back(g.window);
        pools_.emplace_back(g.num_pages);
        table_rows_.emplace_back(static_cast<size_t>(max_requests) * max_blocks_, kUnmapped);
    }
    for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);  // slot 0 first
    for (Request& r : reqs_) {
        r.mapped.assign(groups.size(), 0);
        r.first_kept.assign(groups.size(), 0);
    }
}

Status CacheManager::open(int* slot, std::string* err) {
    if (free_slots_.empty()) return fail(err, kBusy, "all " + std::to_string(max_requests_) + " request slots are in use");
    *slot = free_slots_.back();
    free_slots_.pop_back();
    Request& r = reqs_[*slot];
    r.open = true;
    r.length = 0;
    std::fill(r.mapped.begin(), r.mapped.end(), 0);
    std::fill(r.first_kept.begin(), r.first_kept.end(), 0);
    return kOk;
}

Status CacheManager::close(int slot, std::string* err) {
    if (!is_open(slot)) return fail(err, kInvalidArgument, "slot " + std::to_string(slot) + " is not open");
    Request& r = reqs_[slot];
    for (int g = 0; g < n_groups(); ++g) {
        int32_t* t = row(g, slot);
        for (int lp = 0; lp < r.mapped[g]; ++lp) {
            if (t[lp] != kUnmapped) {
                if (Status s = pools_[g].release(&t[lp], 1, err)) return s;
                t[lp] = kUnmapped;
            }
        }
        r.mapped[g] = 0;
    }
    r.open = false;
    free_slots_.push_back(slot);
    return kOk;
}

void CacheManager::pages_needed(int slot, int new_length, int* out) const {
    const Request& r = reqs_[slot];
    for (int g = 0; g < n_groups(); ++g) out[g] = std::max(0, pages_for(new_length) - r.mapped[g]);
}

Status CacheManager::reserve(const int* slots, const int* new_lengths, int n, std::string* err) {
    std::vector<int> need(static_cast<size_t>(n_groups()), 0), extra(static_cast<size_t>(n_groups()));
    for (int i = 0; i < n; ++i) {
        if (!is_open(slots[i])) return fail(err, kInvalidArgument, "slot " + std::to_string(slots[i]) + " is not open");
        const Request& r = reqs_[slots[i]];
        if (new_lengths[i] > max_positions_)
            return fail(err, kContextFull, "a request would reach " + std::to_string(new_lengths[i]) + " positions; the context holds " +
                                               std::to_string(max_positions_));
        if (new_lengths[i] < r.length) return fail(err, kInvalidArgument, "reserve cannot shrink a request; use truncate");
        pages_needed(slots[i], new_lengths[i], extra.data());
        for (int g = 0; g < n_groups(); ++g) need[g] += extra[g];
    }
    for (int g = 0; g < n_groups(); ++g)
        if (need[g] > pools_[g].free_pages())
            return fail(err, kOutOfPages, "group " + std::to_string(g) + ": " + std::to_string(need[g]) + " pages wanted, " +
                                              std::to_string(pools_[g].free_pages()) + " free of " + std::to_string(pools_[g].num_pages()));
    for (int i = 0; i < n; ++i) {
        Request& r = reqs_[slots[i]];
        for (int g = 0; g < n_groups(); ++g) {
            const int add = std::max(0, pages_for(new_lengths[i]) - r.mapped[g]);
            if (add == 0) continue;
            if (Status s = pools_[g].allocate(add, row(g, slots[i]) + r.mapped[g], err)) return s;
            r.mapped[g] += add;
        }
    }
    return kOk;
}

Status CacheManager::commit(int slot, int new_length, std::string* err) {
    if (!is_open(slot)) return fail(err, kInvalidArgument, "slot " + std::to_string(slot) + " is not open");
    Request& r = reqs_[slot];
    if (n_groups() > 0 && new_length > r.mapped[0] * page_size_) return fail(err, kInvalidArgument, "commit past the reserved pages");
    r.length = new_length;
    for (int g = 0; g < n_groups(); ++g) {
        if (windows_[g] <= 0) continue;
        const int first_needed = std::max(0, new_length - windows_[g] + 1);
        const int keep_from = std::min(first_needed / page_size_, r.mapped[g]);
        int32_t* t = row(g, slot);
        for (int lp = r.first_kept[g]; lp < keep_from; ++lp) {
            if (t[lp] != kUnmapped) {
                if (Status s = pools_[g].release(&t[lp], 1, err)) return s;
                t[lp] = kUnmapped;
            }
        }
        r.first_kept[g] = std::max(r.first_kept[g], keep_from);
    }
    return kOk;
}

Status CacheManager::truncate(int slot, int length, std::string* err) {
    if (!is_open(slot)) return fail(err, kInvalidArgument, "slot " + std::to_string(slot) + " is not open");
    Request& r = reqs_[slot];
    if (length > r.length) return fail(err, kInvalidArgument, "truncate cannot grow a request");
    const int keep = pages_for(length);
    for (int g = 0; g < n_groups(); ++g)
        if (windows_[g] > 0 && r.first_kept[g] * page_size_ > std::max(0, length - windows_[g] + 1))
            return fail(err, kInvalidArgument, "a windowed group has already released what this truncate needs");
    for (int g = 0; g < n_groups(); ++g) {
        int32_t* t = row(g, slot);
        for (int lp = keep; lp < r.mapped[g]; ++lp) {
            if (t[lp] != kUnmapped) {
                if (Status s = pools_[g].release(&t[lp], 1, err)) return s;
                t[lp] = kUnmapped;
            }
        }
        r.mapped[g] = std::min(r.mapped[g], keep);
        r.first_kept[g] = std::min(r.first_kept[g], r.mapped[g]);
    }
    r.length = length;
    return kOk;
}

Status CacheManager::check(std::string* err) const {
    for (int g = 0; g < n_groups(); ++g) {
        if (Status s = pools_[g].check(err)) return s;
        std::vector<uint8_t> seen(static_cast<size_t>(pools_[g].num_pages()), 0);
        int held = 0;
        for (int slot = 0; slot < max_requests_; ++slot) {
            const int32_t* t = row(g, slot);
            for (int lp = 0; lp < max_blocks_; ++lp) {
                const int32_t p = t[lp];
                if (p == kUnmapped) continue;
                if (!reqs_[slot].open || lp >= reqs_[slot].mapped[g])
                    return fail(err, kInternal, "group " + std::to_string(g) + ": a table outside an open request names a page");
                if (p < 0 || p >= pools_[g].num_pages() || seen[p])
                    return fail(err, kInternal, "group " + std::to_string(g) + ": a page is in two tables");
                seen[p] = 1;
                ++held;
            }
        }
        if (held != pools_[g].pages_in_use())
            return fail(err, kInternal, "group " + std::to_string(g) + ": " + std::to_string(pools_[g].pages_in_use()) +
                                            " pages held, tables name " + std::to_string(held));
    }
    std::vector<uint8_t> free_seen(static_cast<size_t>(max_requests_), 0);
    for (int s : free_slots_) {
        if (s < 0 || s >= max_requests_ || free_seen[s]) return fail(err, kInternal, "a state slot is free twice");
        free_seen[s] = 1;
        if (reqs_[s].open) return fail(err, kInternal, "a state slot is free and held");
    }
    int open = 0;
    for (const Request& r : reqs_) open += r.open ? 1 : 0;
    if (open + free_slots() != max_requests_) return fail(err, kInternal, "a state slot was lost");
    return kOk;
}

}  // namespace liyab_host
