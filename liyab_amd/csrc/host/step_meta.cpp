#include "step_meta.h"

#include <algorithm>
#include <vector>

namespace liyab_host {

static Status fail(std::string* err, Status s, const std::string& msg) {
    if (err != nullptr) *err = msg;
    return s;
}

Status step_shape(const CacheManager& m, int n_seqs, const int* slots, const int* q_lens, const int* want_counts,
                  int pad_rows, StepShape* out, std::string* err) {
    if (n_seqs <= 0) return fail(err, kInvalidArgument, "a step needs at least one item");
    if (pad_rows < 0) return fail(err, kInvalidArgument, "a negative number of padding rows");
    if (m.n_groups() > kMaxGroups) return fail(err, kInvalidArgument, "more cache groups than a step's metadata holds");
    StepShape s{};
    s.n_seqs = n_seqs;
    s.n_groups = m.n_groups();
    s.max_blocks = m.max_blocks();
    for (int i = 0; i < n_seqs; ++i) {
        if (!m.is_open(slots[i])) return fail(err, kInvalidArgument, "slot " + std::to_string(slots[i]) + " is not open");
        if (q_lens[i] <= 0) return fail(err, kInvalidArgument, "an item brings no tokens");
        s.n_tokens += q_lens[i];
        s.n_logit_rows += want_counts[i];
        s.max_q_len = std::max(s.max_q_len, q_lens[i]);
        s.max_context = std::max(s.max_context, m.length(slots[i]) + q_lens[i]);
    }
    int cur = 0;
    auto place = [&cur](int size) {
        const int at = cur;
        cur += size;
        return at;
    };
    s.n_rows = s.n_tokens + pad_rows;
    const int N = s.n_rows, S = n_seqs, R = s.n_logit_rows;
    s.off_token_ids = place(N);
    s.off_positions = place(N);
    s.off_tok_seq = place(N);
    s.off_seq_starts = place(S + 1);
    s.off_context_lens = place(S);
    s.off_state_slots = place(S);
    s.off_logit_rows = place(std::max(R, 1));
    s.off_logit_slots = place(std::max(R, 1));
    for (int g = 0; g < s.n_groups; ++g) {
        s.off_block_tables[g] = place(S * s.max_blocks);
        s.off_slots[g] = place(N);
    }
    s.total = cur;
    *out = s;
    return kOk;
}

Status step_fill(const CacheManager& m, const StepShape& s, const int* slots, const int* q_lens, const int64_t* tokens,
                 const int* want_counts, const int* wants, int vocab_size, int32_t* block, std::string* err) {
    const int S = s.n_seqs, page = m.page_size(), W = s.max_blocks;
    int32_t* tok = block + s.off_token_ids;
    int32_t* pos = block + s.off_positions;
    int32_t* seq = block + s.off_tok_seq;
    int32_t* starts = block + s.off_seq_starts;
    int32_t* rows = block + s.off_logit_rows;
    int32_t* row_slots = block + s.off_logit_slots;
    rows[0] = 0;
    row_slots[0] = 0;
    int row0 = 0, r = 0;
    for (int i = 0; i < S; ++i) {
        const int first = m.length(slots[i]), n = q_lens[i];
        starts[i] = row0;
        block[s.off_context_lens + i] = first + n;
        block[s.off_state_slots + i] = slots[i];
        for (int j = 0; j < n; ++j) {
            const int64_t id = tokens[row0 + j];
            if (id >= vocab_size || (id < 0 && (-1 - id) >= m.max_requests()))
                return fail(err, kInvalidArgument, "token id " + std::to_string(id) + " is outside [0, " + std::to_string(vocab_size) + ")");
            tok[row0 + j] = static_cast<int32_t>(id);
            pos[row0 + j] = first + j;
            seq[row0 + j] = i;
        }
        for (int k = 0; k < want_counts[i]; ++k, ++r) {
            if (wants[r] < 0 || wants[r] >= n)
                return fail(err, kInvalidArgument, "logits wanted at place " + std::to_string(wants[r]) + " of " + std::to_string(n) + " tokens");
            rows[r] = row0 + wants[r];
            row_slots[r] = slots[i];
        }
        row0 += n;
    }
    starts[S] = row0;
    for (int j = row0; j < s.n_rows; ++j) {  // padding rows
        tok[j] = 0;
        pos[j] = 0;
        seq[j] = 0;
    }
    for (int g = 0; g < s.n_groups; ++g) {
        int32_t* bt = block + s.off_block_tables[g];
        int32_t* sl = block + s.off_slots[g];
        const int32_t* all = m.table_rows(g);
        for (int i = 0; i < S; ++i) {
            const int32_t* t = all + static_cast<size_t>(slots[i]) * W;
            std::copy(t, t + W, bt + static_cast<size_t>(i) * W);
            const int first = m.length(slots[i]);
            for (int j = 0; j < q_lens[i]; ++j) {
                const int p = first + j;
                const int32_t pg = p / page < W ? t[p / page] : kUnmapped;
                if (pg < 0) return fail(err, kInternal, "a token of this step maps to a released or unmapped page");
                sl[starts[i] + j] = pg * page + p % page;
            }
        }
        for (int j = s.n_tokens; j < s.n_rows; ++j) sl[j] = -1;
    }
    return kOk;
}

}  // namespace liyab_host
