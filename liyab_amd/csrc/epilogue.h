// What a matrix product does with its accumulators.
//
// Every product kernel ends in the same epilogue: add the bias, then one of
//   none / GELU          -> out[m, n] in the output type
//   residual             -> residual[m, n] += value (the 32-bit residual stream)
//   paged QKV            -> columns [0, q_dim) go to out[m, n] (queries);
//                           columns of keys and values go straight to token
//                           m's slot of the cache pages, so the projection's
//                           output is never copied (the reference splits the
//                           fused output per token and then stores the rows,
//                           src/core/transformer.cpp:2657-2673, 2875-2890).
#pragma once

#include "activations.h"
#include "common.h"

namespace liyab {

enum : int { kEpiQkvPaged = 4 };

struct EpiParams {
    int mode;
    int out_dtype;            // of out and of the cache pages
    const float* bias;        // [N] or null
    void* out;                // [M, ldo]
    int64_t ldo;
    float* residual;          // [M, ldr]
    int64_t ldr;
    // paged QKV
    void* kc;
    void* vc;
    const int* slots;         // [M]: page * page_size + offset
    int q_dim, kv_dim, hd, n_kv_head, page_size;
    int exact;                // erf in double (32-bit path)
    uint32_t num_slots;       // pages x page_size of the caches: a slot outside [0, num_slots) is not written
};

// `MODE` >= 0 fixes the epilogue at compile time (straight-line code in the kernels' store
// loops); -1 reads it from the parameters.
// The bias of column n (0 without one). Kernels that store several rows of a column load it
// once, ahead of their store loop: a load between two stores would have to wait for the first
// store, since the compiler cannot know that outputs and bias do not overlap.
__device__ __forceinline__ float epilogue_bias(const EpiParams& p, int n) { return p.bias != nullptr ? p.bias[n] : 0.0f; }

template <typename OutT, int MODE = -1>
__device__ __forceinline__ void epilogue_store_biased(const EpiParams& p, int m, int n, float v);

template <typename OutT, int MODE = -1>
__device__ __forceinline__ void epilogue_store(const EpiParams& p, int m, int n, float v) {
    epilogue_store_biased<OutT, MODE>(p, m, n, v + epilogue_bias(p, n));
}

// `v` already holds the bias.
template <typename OutT, int MODE>
__device__ __forceinline__ void epilogue_store_biased(const EpiParams& p, int m, int n, float v) {
    switch (MODE >= 0 ? MODE : p.mode) {
        case kEpiGeluTanh: v = p.exact ? gelu_tanh(v) : gelu_tanh_fast(v); break;
        case kEpiGeluErf: v = p.exact ? gelu_erf_exact(v) : gelu_erf_fast(v); break;
        case kEpiResidual:
            p.residual[static_cast<int64_t>(m) * p.ldr + n] += v;
            return;
        case kEpiQkvPaged:
            if (n >= p.q_dim) {
                const bool is_v = n >= p.q_dim + p.kv_dim;
                const int c = n - p.q_dim - (is_v ? p.kv_dim : 0);
                const int64_t slot = p.slots[m];
                if (static_cast<uint64_t>(slot) >= p.num_slots) return;  // no slot (-1), or none of these caches
                const int64_t page = slot / p.page_size;
                const int off = static_cast<int>(slot % p.page_size);
                const int64_t dst = ((page * p.n_kv_head + c / p.hd) * p.page_size + off) * p.hd + c % p.hd;
                static_cast<OutT*>(is_v ? p.vc : p.kc)[dst] = from_float<OutT>(v);
                return;
            }
            break;
        default: break;
    }
    static_cast<OutT*>(p.out)[static_cast<int64_t>(m) * p.ldo + n] = from_float<OutT>(v);
}

// The paged QKV epilogue for kernels whose lanes hold several rows of one column: what depends
// on the row (its slot's place in the pages) is computed once per row, ahead of the stores.
// Element offset of row m's slot for head 0, dimension 0; -1 for a token without a slot (or with
// one past the caches' pages: a wrong word in the slots must not become a store outside them).
__device__ __forceinline__ int64_t qkv_row_base(const EpiParams& p, int m) {
    const int64_t slot = p.slots[m];
    if (static_cast<uint64_t>(slot) >= p.num_slots) return -1;
    return (slot / p.page_size) * (static_cast<int64_t>(p.n_kv_head) * p.page_size * p.hd) + (slot % p.page_size) * p.hd;
}
// What depends on the column: -1 for a query column, else the offset of (head, dimension)
// within a page, with bit 62 set for values.
__device__ __forceinline__ int64_t qkv_col_offset(const EpiParams& p, int n) {
    if (n < p.q_dim) return -1;
    const bool is_v = n >= p.q_dim + p.kv_dim;
    const int c = n - p.q_dim - (is_v ? p.kv_dim : 0);
    return (static_cast<int64_t>(c / p.hd) * p.page_size * p.hd + c % p.hd) | (is_v ? (int64_t{1} << 62) : 0);
}
template <typename OutT>
__device__ __forceinline__ void qkv_store(const EpiParams& p, int m, int n, int64_t row_base, int64_t col_offset, float v) {
    if (col_offset < 0) {
        static_cast<OutT*>(p.out)[static_cast<int64_t>(m) * p.ldo + n] = from_float<OutT>(v);
    } else if (row_base >= 0) {
        const bool is_v = (col_offset >> 62) & 1;
        static_cast<OutT*>(is_v ? p.vc : p.kc)[row_base + (col_offset & ~(int64_t{1} << 62))] = from_float<OutT>(v);
    }
}

// Host-side check shared by the launchers.
inline int check_epilogue(const EpiParams& p, int M, int N) {
    (void)M;
    if (p.mode == kEpiResidual) {
        LIYAB_REQUIRE(p.residual != nullptr && p.ldr >= N, "gemm: the residual epilogue needs a residual of row stride >= N");
    } else if (p.mode == kEpiQkvPaged) {
        LIYAB_REQUIRE(p.out && p.kc && p.vc && p.slots, "gemm: the paged QKV epilogue needs out, caches and slots");
        LIYAB_REQUIRE(p.q_dim > 0 && p.kv_dim > 0 && p.hd > 0 && p.page_size > 0 && p.n_kv_head * p.hd == p.kv_dim &&
                          p.q_dim + 2 * p.kv_dim == N && p.ldo >= p.q_dim,
                      "gemm: the paged QKV epilogue's sizes do not fit N = %d", N);
        LIYAB_REQUIRE(p.num_slots > 0 && p.num_slots % static_cast<uint32_t>(p.page_size) == 0,
                      "gemm: the paged QKV epilogue needs the caches' slots (pages x page size), got %u", p.num_slots);
    } else {
        LIYAB_REQUIRE(p.mode >= kEpiNone && p.mode <= kEpiGeluErf, "gemm: unknown epilogue %d", p.mode);
        LIYAB_REQUIRE(p.out != nullptr && p.ldo >= N, "gemm: needs an output of row stride >= N");
    }
    return 0;
}

}  // namespace liyab
