// A step's metadata: one block of int32 words that goes to the device in one copy.
//
// The block here holds what every part may need of a step (tokens, positions, requests, block
// tables, cache slots, wanted rows). What only one kind of part needs (attention's work lists,
// further down) is that part's own: it is laid out behind this block by the step function, from
// what the part's planner says, and goes to the device in the same copy.
//
// The batch is the reference's list of segments flattened (src/core/transformer.h:890-920):
// rows are the items' tokens one after the other; a row's position is its request's length
// before the step plus its index in the item (src/core/transformer.cpp:6689-6693).
#pragma once

#include <cstdint>
#include <string>

#include "cache_manager.h"

namespace liyab_host {

constexpr int kMaxGroups = 16;

// Sizes of a step and where each array starts in the block (offsets in words).
struct StepShape {
    int n_tokens, n_rows, n_seqs, n_logit_rows, n_groups, max_blocks;  // n_rows: the tokens and the padding rows after them
    int max_q_len, max_context;
    int total;       // words in the block
    int off_token_ids, off_positions, off_tok_seq, off_seq_starts, off_context_lens, off_state_slots;
    int off_logit_rows, off_logit_slots;
    int off_block_tables[kMaxGroups], off_slots[kMaxGroups];
};

// From the items' sizes alone (requests by slot, tokens each brings, logits each wants). pad_rows: rows
// after the last token that belong to no request (a step padded to a size that comes back, so that its
// captured graph serves every step of that size): token 0 at position 0 of the step's first request, slot
// -1 in every group, which no kernel writes to; nothing reads what is computed for them.
Status step_shape(const CacheManager& m, int n_seqs, const int* slots, const int* q_lens, const int* want_counts,
                  int pad_rows, StepShape* out, std::string* err);

// Fills the block. `tokens`: the items' token ids one after the other; an id < 0 stands for "the
// token sampled for slot -1 - id, still on the device". `wants`: places within each item.
// Pages of every position the step touches must be mapped (reserve comes first).
Status step_fill(const CacheManager& m, const StepShape& shape, const int* slots, const int* q_lens, const int64_t* tokens,
                 const int* want_counts, const int* wants, int vocab_size, int32_t* block, std::string* err);

}  // namespace liyab_host
