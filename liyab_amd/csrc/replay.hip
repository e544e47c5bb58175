// A recorded list of launches, run again from one call.
//
// A model's layers of one kind make the same launches with other weights and other cache pages.
// The host's Python composes a layer's launches once a step (kernels chosen, operands checked,
// arguments converted: about 10 us a launch) and records them as words; for each layer that
// follows it writes that layer's addresses over the recorded layer's in a copy of the list
// (models/decoder.py) and the launches run from here. The reference's pass over the layers is
// native code throughout (src/core/transformer.cpp:6589-6769); here the parts stay Python, so
// that a part of a test's own registers like any other, and only the repetition is native.
//
// A list is a sequence of records of 64-bit words:
//   [launcher index, number of arguments, arguments ..., number of block words, block words ...]
// An argument is the value's bits (integers sign-extended, a float's 32 bits in the low half).
// The argument that points at the epilogue's parameter block holds kBlockArg instead; the block's
// bytes follow the arguments, and the launcher gets their address.
#include "launchers.h"
#include "epilogue.h"

#include <cstring>
#include <utility>

namespace liyab {
namespace replay {

constexpr uint64_t kBlockArg = 0xB10CB10CB10CB10Cull;
constexpr int kMaxArgs = 32, kMaxBlockWords = 32;

template <typename T>
struct Arg {
    static T get(uint64_t bits) { return static_cast<T>(static_cast<int64_t>(bits)); }  // integers
};
template <typename T>
struct Arg<T*> {
    static T* get(uint64_t bits) { return reinterpret_cast<T*>(bits); }
};
template <>
struct Arg<float> {
    static float get(uint64_t bits) {
        const uint32_t lo = static_cast<uint32_t>(bits);
        float f;
        std::memcpy(&f, &lo, 4);
        return f;
    }
};

template <typename... A, size_t... I>
int invoke(int (*fn)(A...), const uint64_t* a, std::index_sequence<I...>) {
    return fn(Arg<A>::get(a[I])...);
}
template <typename... A>
constexpr int arity(int (*)(A...)) {
    return static_cast<int>(sizeof...(A));
}

struct Entry {
    const char* name;
    int (*call)(const uint64_t*);
    int n_args;
};

#define LIYAB_ENTRY(fn)                                                                                    \
    {                                                                                                      \
        #fn, [](const uint64_t* a) { return invoke(&fn, a, std::make_index_sequence<arity(&fn)>{}); }, arity(&fn) \
    }

// The launchers a list may name, by index (liyab_replay_index gives a name's).
static const Entry kEntries[] = {
    LIYAB_ENTRY(liyab_fill),
    LIYAB_ENTRY(liyab_add_into),
    LIYAB_ENTRY(liyab_gather_rows),
    LIYAB_ENTRY(liyab_scale),
    LIYAB_ENTRY(liyab_embed),
    LIYAB_ENTRY(liyab_add_rows),
    LIYAB_ENTRY(liyab_kv_write),
    LIYAB_ENTRY(liyab_layernorm),
    LIYAB_ENTRY(liyab_layernorm_parts),
    LIYAB_ENTRY(liyab_sum_parts),
    LIYAB_ENTRY(liyab_gemm_simple),
    LIYAB_ENTRY(liyab_gemm_mfma),
    LIYAB_ENTRY(liyab_gemm_mfma_dl),
    LIYAB_ENTRY(liyab_gemm_mfma_dl_parts),
    LIYAB_ENTRY(liyab_gemm_skinny),
    LIYAB_ENTRY(liyab_gemm_skinny_parts),
    LIYAB_ENTRY(liyab_gemm_att_parts),
    LIYAB_ENTRY(liyab_gemm_skinny_ln),
    LIYAB_ENTRY(liyab_attention_generic),
    LIYAB_ENTRY(liyab_attention_decode),
    LIYAB_ENTRY(liyab_attention_merge),
    LIYAB_ENTRY(liyab_attention_prefill),
};
constexpr int kNumEntries = static_cast<int>(sizeof(kEntries) / sizeof(kEntries[0]));

}  // namespace replay
}  // namespace liyab

using namespace liyab;
using namespace liyab::replay;

// The index of a launcher in the lists' numbering and the number of its arguments; -1 for a
// name the replay does not know (a launch of it cannot be recorded).
extern "C" int liyab_replay_index(const char* name, int* n_args) {
    for (int i = 0; i < kNumEntries; ++i)
        if (std::strcmp(kEntries[i].name, name) == 0) {
            if (n_args != nullptr) *n_args = kEntries[i].n_args;
            return i;
        }
    return -1;
}

// Runs the `n_words` words of `list` (see above). Stops at the first launcher that fails and
// returns its code (its message is liyab_last_error's); a malformed list is refused before
// anything of it is launched.
extern "C" int liyab_replay(const uint64_t* list, int64_t n_words) {
    LIYAB_REQUIRE(list != nullptr && n_words >= 0, "replay: null operand");
    // the whole list is looked over first
    int64_t at = 0;
    int n_launches = 0;
    while (at < n_words) {
        LIYAB_REQUIRE(at + 2 <= n_words, "replay: a record is cut short at word %lld", static_cast<long long>(at));
        const uint64_t index = list[at], n_args = list[at + 1];
        LIYAB_REQUIRE(index < static_cast<uint64_t>(kNumEntries), "replay: unknown launcher %llu", static_cast<unsigned long long>(index));
        LIYAB_REQUIRE(n_args == static_cast<uint64_t>(kEntries[index].n_args) && n_args <= kMaxArgs, "replay: %s takes %d arguments, the record has %llu",
                      kEntries[index].name, kEntries[index].n_args, static_cast<unsigned long long>(n_args));
        LIYAB_REQUIRE(at + 2 + static_cast<int64_t>(n_args) + 1 <= n_words, "replay: a record is cut short at word %lld", static_cast<long long>(at));
        const uint64_t n_block = list[at + 2 + n_args];
        LIYAB_REQUIRE(n_block <= kMaxBlockWords && at + 3 + static_cast<int64_t>(n_args + n_block) <= n_words, "replay: a parameter block of %llu words",
                      static_cast<unsigned long long>(n_block));
        LIYAB_REQUIRE(n_block == 0 || n_block * sizeof(uint64_t) >= sizeof(EpiParams), "replay: a parameter block of %llu words is shorter than the launchers read",
                      static_cast<unsigned long long>(n_block));
        int blocks = 0;
        for (uint64_t i = 0; i < n_args; ++i) blocks += list[at + 2 + i] == kBlockArg ? 1 : 0;
        LIYAB_REQUIRE(blocks == (n_block > 0 ? 1 : 0), "replay: %s: %d arguments point at a parameter block of %llu words", kEntries[index].name, blocks,
                      static_cast<unsigned long long>(n_block));
        at += 3 + static_cast<int64_t>(n_args + n_block);
        ++n_launches;
    }
    at = 0;
    for (int l = 0; l < n_launches; ++l) {
        const uint64_t index = list[at], n_args = list[at + 1], n_block = list[at + 2 + n_args];
        uint64_t args[kMaxArgs];
        alignas(16) uint64_t block[kMaxBlockWords];  // (the list itself may not be aligned for the block's type)
        for (uint64_t i = 0; i < n_block; ++i) block[i] = list[at + 3 + n_args + i];
        for (uint64_t i = 0; i < n_args; ++i) {
            const uint64_t word = list[at + 2 + i];
            args[i] = word == kBlockArg ? reinterpret_cast<uint64_t>(block) : word;
        }
        if (const int rc = kEntries[index].call(args)) return rc;
        at += 3 + static_cast<int64_t>(n_args + n_block);
    }
    return 0;
}
