// A driver for the host library that needs nothing but a C++ compiler: random requests through
// the scheduler, the cache manager and a step's metadata, with the manager's invariants checked
// after every step. It is what the address and undefined-behaviour sanitizers run over
// (`csrc/build.py: build_host_selftest(sanitize=True)`; the reference's build has no sanitizer,
// its determinism tests play that part, tests/test_engine.cpp:4226-4240): out-of-bounds table
// rows, a page used after release, signed overflow in the page arithmetic all end the run.
//
// usage: selftest [seeds] [steps per seed]; exit status 0 when every invariant held.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "../cache_manager.h"
#include "../scheduler.h"
#include "../attention_plan.h"
#include "../step_meta.h"

using namespace liyab_host;

#define CHECK(cond, ...)                                  \
    do {                                                  \
        if (!(cond)) {                                    \
            std::fprintf(stderr, "selftest: " __VA_ARGS__); \
            std::fprintf(stderr, "\n");                   \
            return 1;                                     \
        }                                                 \
    } while (0)

static int run(unsigned seed, int n_steps) {
    std::mt19937 rng(seed);
    auto pick = [&](int lo, int hi) { return lo + static_cast<int>(rng() % static_cast<unsigned>(hi - lo + 1)); };
    const int page = 1 << pick(2, 5), max_positions = pick(40, 300), max_requests = pick(1, 6);
    const int windowed = pick(0, 1), window = pick(5, 60);
    const int need_alone = (max_positions + page - 1) / page;
    std::vector<GroupConfig> groups{{0, need_alone + pick(0, 2 * need_alone)}};
    if (windowed) groups.push_back({window, need_alone + pick(0, need_alone)});
    CacheManager m(groups, page, max_requests, max_positions);
    Scheduler s(&m, pick(1, max_requests), pick(4, 96), pick(2, 64));
    std::string err;
    struct Live {
        int n_prompt, max_tokens;
    };
    std::vector<Live> live;
    std::vector<Scheduled> batch;
    std::vector<int> opened, preempted;
    std::vector<int> waiting_for_token;  // requests whose step has run and whose token has not been read
    long long tokens = 0;
    for (int step = 0; step < n_steps; ++step) {
        // arrivals
        while (pick(0, 3) == 0 && s.n_requests() < 12) {
            int id = -1;
            const int n_prompt = pick(1, max_positions + 3), max_tokens = pick(1, 40);
            const Status st = s.add(n_prompt, max_tokens, static_cast<int>(rng() % 3) - 1, &id, &err);
            CHECK(st == kOk || st == kInvalidArgument || st == kOutOfPages, "seed %u: add: %s", seed, err.c_str());
        }
        // tokens of the step before reach the host before this one is scheduled, or lag one step
        const bool lag = pick(0, 1) == 1 && !s.pressure();
        if (!lag) {
            for (int id : waiting_for_token) s.token(id, pick(0, 30) == 0);
            waiting_for_token.clear();
        }
        const Status st = s.schedule(&batch, &opened, &preempted, &err);
        if (st == kOutOfPages) break;  // "no request can make progress": a legal end of this seed's story
        CHECK(st == kOk, "seed %u step %d: schedule: %s", seed, step, err.c_str());
        if (!batch.empty()) {
            const int n = static_cast<int>(batch.size());
            std::vector<int> slots(n), q_lens(n), wants_n(n), wants, first(n);
            std::vector<int64_t> toks;
            int budget = 0;
            for (int i = 0; i < n; ++i) {
                slots[i] = batch[i].slot;
                q_lens[i] = batch[i].count;
                wants_n[i] = batch[i].wants_logits ? 1 : 0;
                if (batch[i].wants_logits) wants.push_back(batch[i].count - 1);
                first[i] = m.length(batch[i].slot);
                CHECK(first[i] == batch[i].first, "seed %u: the scheduler and the manager disagree on a request's length", seed);
                for (int j = 0; j < batch[i].count; ++j) toks.push_back(pick(0, 99));
                budget += batch[i].count;
            }
            if (wants.empty()) wants.push_back(0);
            std::vector<int> new_lengths(n);
            for (int i = 0; i < n; ++i) new_lengths[i] = first[i] + q_lens[i];
            CHECK(m.reserve(slots.data(), new_lengths.data(), n, &err) == kOk, "seed %u step %d: reserve after schedule: %s", seed, step, err.c_str());
            StepShape shape;
            const int pad = pick(0, 2) == 0 ? pick(1, 70) : 0;  // some steps with padding rows behind their tokens
            CHECK(step_shape(m, n, slots.data(), q_lens.data(), wants_n.data(), pad, &shape, &err) == kOk, "step_shape: %s", err.c_str());
            CHECK(shape.n_tokens == budget && shape.n_rows == budget + pad, "step_shape: %d tokens and %d rows for %d + %d", shape.n_tokens, shape.n_rows, budget, pad);
            std::vector<int32_t> block(static_cast<size_t>(shape.total) + 8, -12345);
            CHECK(step_fill(m, shape, slots.data(), q_lens.data(), toks.data(), wants_n.data(), wants.data(), 100, block.data(), &err) == kOk,
                  "step_fill: %s", err.c_str());
            for (int k = 0; k < 8; ++k) CHECK(block[static_cast<size_t>(shape.total) + k] == -12345, "step_fill wrote past its block");
            for (int j = shape.n_tokens; j < shape.n_rows; ++j) {
                CHECK(block[shape.off_token_ids + j] == 0 && block[shape.off_positions + j] == 0 && block[shape.off_tok_seq + j] == 0, "a padding row's token, position or request");
                for (int g = 0; g < shape.n_groups; ++g) CHECK(block[shape.off_slots[g] + j] == -1, "a padding row with a slot");
            }
            int n_tiles = 0, n_single = 0;
            const int tile = pick(0, 1) ? 64 : 128;
            attn_counts(n, q_lens.data(), 8, tile, &n_tiles, &n_single);
            std::vector<int32_t> words(static_cast<size_t>(4 * std::max(n_tiles, 1) + std::max(n_single, 1)) + 4, -777);
            attn_fill(n, q_lens.data(), first.data(), 8, tile, words.data());
            for (int k = 0; k < 4; ++k) CHECK(words[words.size() - 1 - k] == -777, "attn_fill wrote past its words");
            for (int i = 0; i < n; ++i) CHECK(m.commit(slots[i], new_lengths[i], &err) == kOk, "commit: %s", err.c_str());
            s.advance(batch.data(), n);
            for (int i = 0; i < n; ++i)
                if (batch[i].wants_logits) waiting_for_token.push_back(batch[i].id);
            tokens += budget;
        }
        if (pick(0, 40) == 0 && !s.running().empty()) {
            const int id = s.running()[static_cast<size_t>(pick(0, static_cast<int>(s.running().size()) - 1))];
            CHECK(s.finish(id, &err) == kOk, "finish: %s", err.c_str());
        }
        CHECK(m.check(&err) == kOk, "seed %u step %d: %s", seed, step, err.c_str());
    }
    // drain: read what is pending, end everything, and nothing may be held afterwards
    for (int id : waiting_for_token) s.token(id, false);
    std::vector<int> rest(s.running().begin(), s.running().end());
    rest.insert(rest.end(), s.waiting().begin(), s.waiting().end());
    for (int id : rest) CHECK(s.finish(id, &err) == kOk, "finish at the end: %s", err.c_str());
    CHECK(m.check(&err) == kOk, "seed %u at the end: %s", seed, err.c_str());
    for (int g = 0; g < m.n_groups(); ++g) CHECK(m.pool(g).pages_in_use() == 0, "seed %u: group %d still holds pages", seed, g);
    CHECK(m.free_slots() == max_requests, "seed %u: a state slot was lost", seed);
    return tokens >= 0 ? 0 : 1;
}

int main(int argc, char** argv) {
    const int seeds = argc > 1 ? std::atoi(argv[1]) : 200, steps = argc > 2 ? std::atoi(argv[2]) : 150;
    for (int seed = 0; seed < seeds; ++seed)
        if (int rc = run(static_cast<unsigned>(seed), steps)) return rc;
    std::printf("selftest ok: %d seeds of %d steps\n", seeds, steps);
    return 0;
}
