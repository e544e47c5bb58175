// Token embedding gather (+ learned positions) and the write of keys and
// values into cache pages.
//
// x[t] = scale * tok[id_t] (+ pos[p_t]): the reference's `embed` followed by
// `add_positions` (src/core/transformer.cpp:5495-5512, 2791-2808), one pass
// over the row. The sum is formed in 32-bit and the residual stream it
// starts is 32-bit on both paths.
#include "common.h"
#include "launchers.h"

#include <algorithm>

namespace liyab {

// An id below zero is a reference: -1 - id indexes `last_tokens`, where the sampler left the
// token a request drew in the step before (the host may not have seen it yet).
// WIDE: rows whose width is a multiple of 16 bytes' worth of elements are read 16 bytes a lane,
// all of a lane's loads asked for before the first is used (one element a lane and trip, a
// row of 4,096 took 14 us of waiting for one load after the other).
template <typename T, bool WIDE>
__global__ void embed_kernel(float* __restrict__ x, const T* __restrict__ tok, const T* __restrict__ pos,
                             const int* __restrict__ ids, const int* __restrict__ positions, int d, float scale,
                             const int* __restrict__ last_tokens) {
    const int t = blockIdx.x;
    int64_t id = ids[t];
    if (id < 0) id = last_tokens[-1 - id];
    const T* trow = tok + id * d;
    const T* prow = pos != nullptr ? pos + static_cast<int64_t>(positions[t]) * d : nullptr;
    float* out = x + static_cast<int64_t>(t) * d;
    if constexpr (WIDE) {
        constexpr int V = 16 / sizeof(T);
        struct alignas(16) Piece {
            T e[V];
        };
        for (int i = threadIdx.x * V; i < d; i += blockDim.x * V) {
            const Piece a = *reinterpret_cast<const Piece*>(trow + i);
            Piece b = a;
            if (prow != nullptr) b = *reinterpret_cast<const Piece*>(prow + i);
            float v[V];
#pragma unroll
            for (int j = 0; j < V; ++j) {
                v[j] = to_float<T>(a.e[j]) * scale;
                if (prow != nullptr) v[j] += to_float<T>(b.e[j]);
            }
#pragma unroll
            for (int j = 0; j < V; j += 4) *reinterpret_cast<float4*>(out + i + j) = make_float4(v[j], v[j + 1], v[j + 2], v[j + 3]);
        }
    } else {
        for (int i = threadIdx.x; i < d; i += blockDim.x) {
            float v = to_float<T>(trow[i]) * scale;
            if (prow != nullptr) v += to_float<T>(prow[i]);
            out[i] = v;
        }
    }
}

// x[t] += table[p_t]  (a residual position encoding applied on its own)
template <typename T>
__global__ void add_rows_kernel(float* __restrict__ x, const T* __restrict__ table, const int* __restrict__ rows, int d) {
    const int t = blockIdx.x;
    const T* r = table + static_cast<int64_t>(rows[t]) * d;
    float* out = x + static_cast<int64_t>(t) * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] += to_float<T>(r[i]);
}

// Token t's keys and values, read from its row of the projection output at
// column offsets k_off and v_off, go to slot[t] = page * page_size + offset
// of a cache laid out [page][kv_head][page_size][head_dim]
// (the reference's store_kv, src/core/transformer.cpp:2875-2890).
template <typename T>
__global__ void kv_write_kernel(T* __restrict__ kc, T* __restrict__ vc, const T* __restrict__ src, int64_t src_stride,
                                int k_off, int v_off, const int* __restrict__ slots, int n_kv_head, int hd,
                                int page_size, uint32_t num_slots) {
    const int t = blockIdx.x;
    const int64_t slot = slots[t];
    if (static_cast<uint64_t>(slot) >= num_slots) return;  // no slot (-1), or none of these caches
    const int64_t page = slot / page_size;
    const int off = static_cast<int>(slot % page_size);
    const T* row = src + static_cast<int64_t>(t) * src_stride;
    const int kv_dim = n_kv_head * hd;
    for (int i = threadIdx.x; i < kv_dim; i += blockDim.x) {
        const int h = i / hd, e = i % hd;
        const int64_t dst = ((page * n_kv_head + h) * page_size + off) * hd + e;
        kc[dst] = row[k_off + i];
        vc[dst] = row[v_off + i];
    }
}

// out[r] = x[rows[r]] (or x[r]) in the output's precision: the rows whose logits are wanted, for a
// head that no norm stands before (a norm gathers them itself).
template <typename T>
__global__ void gather_rows_kernel(T* __restrict__ out, const float* __restrict__ x, const int* __restrict__ rows, int d) {
    const int r = blockIdx.x;
    const float* src = x + static_cast<int64_t>(rows != nullptr ? rows[r] : r) * d;
    T* dst = out + static_cast<int64_t>(r) * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = from_float<T>(src[i]);
}

// p[i] *= scale (logits times a model's logit scale, the reference's finish_logits,
// src/core/transformer.cpp:2613-2620)
__global__ void scale_kernel(float* __restrict__ p, float scale, int64_t n) {
    int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += step) p[i] *= scale;
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_gather_rows(void* out, int out_dtype, const float* x, const int* rows, int n, int d, hipStream_t stream) {
    LIYAB_REQUIRE(out && x, "gather_rows: null pointer");
    LIYAB_REQUIRE(d > 0 && n >= 0, "gather_rows: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(out_dtype == kF32 || out_dtype == kBF16, "gather_rows: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    const int threads = d >= 256 ? 256 : 64;
    if (out_dtype == kF32) gather_rows_kernel<float><<<n, threads, 0, stream>>>(static_cast<float*>(out), x, rows, d);
    else gather_rows_kernel<bf16_t><<<n, threads, 0, stream>>>(static_cast<bf16_t*>(out), x, rows, d);
    return check_launch("gather_rows");
}

extern "C" int liyab_scale(float* p, float scale, int64_t n, hipStream_t stream) {
    LIYAB_REQUIRE(p != nullptr || n == 0, "scale: null pointer");
    LIYAB_REQUIRE(n >= 0, "scale: negative count");
    if (n == 0) return 0;
    const int blocks = static_cast<int>(std::min<int64_t>((n + 255) / 256, 4096));
    scale_kernel<<<blocks, 256, 0, stream>>>(p, scale, n);
    return check_launch("scale");
}

extern "C" int liyab_embed(float* x, const void* tok, const void* pos, int dtype, const int* ids, const int* positions,
                           int n, int d, float scale, const int* last_tokens, hipStream_t stream) {
    LIYAB_REQUIRE(x && tok && ids, "embed: null pointer");
    LIYAB_REQUIRE(pos == nullptr || positions != nullptr, "embed: a position table needs positions");
    LIYAB_REQUIRE(d > 0 && n >= 0, "embed: bad sizes n=%d d=%d", n, d);
    if (n == 0) return 0;
    auto aligned = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool wide = d % (dtype == kF32 ? 4 : 8) == 0 && aligned(x) && aligned(tok) && aligned(pos);
    auto launch = [&](auto* table, auto* positions_table) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(table)>>;
        const int lanes = wide ? d / static_cast<int>(16 / sizeof(T)) : d;
        const int threads = lanes > 512 ? 1024 : (lanes > 256 ? 512 : (lanes > 64 ? 256 : 64));
        if (wide) embed_kernel<T, true><<<n, threads, 0, stream>>>(x, table, positions_table, ids, positions, d, scale, last_tokens);
        else embed_kernel<T, false><<<n, threads, 0, stream>>>(x, table, positions_table, ids, positions, d, scale, last_tokens);
    };
    if (dtype == kF32) {
        launch(static_cast<const float*>(tok), static_cast<const float*>(pos));
    } else if (dtype == kBF16) {
        launch(static_cast<const bf16_t*>(tok), static_cast<const bf16_t*>(pos));
    } else {
        return fail(1, "embed: unknown dtype %d", dtype);
    }
    return check_launch("embed");
}

extern "C" int liyab_add_rows(float* x, const void* table, int dtype, const int* rows, int n, int d,
                              hipStream_t stream) {
    LIYAB_REQUIRE(x && table && rows, "add_rows: null pointer");
    LIYAB_REQUIRE(d > 0 && n >= 0, "add_rows: bad sizes n=%d d=%d", n, d);
    if (n == 0) return 0;
    const int threads = d >= 256 ? 256 : 64;
    if (dtype == kF32) {
        add_rows_kernel<float><<<n, threads, 0, stream>>>(x, static_cast<const float*>(table), rows, d);
    } else if (dtype == kBF16) {
        add_rows_kernel<bf16_t><<<n, threads, 0, stream>>>(x, static_cast<const bf16_t*>(table), rows, d);
    } else {
        return fail(1, "add_rows: unknown dtype %d", dtype);
    }
    return check_launch("add_rows");
}

extern "C" int liyab_kv_write(void* kc, void* vc, const void* src, int dtype, int64_t src_stride, int k_off, int v_off,
                              const int* slots, int n, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream) {
    LIYAB_REQUIRE(kc && vc && src && slots, "kv_write: null pointer");
    LIYAB_REQUIRE(num_pages > 0 && static_cast<int64_t>(num_pages) * page_size < (int64_t{1} << 31), "kv_write: the caches hold %d pages", num_pages);
    const uint32_t num_slots = static_cast<uint32_t>(num_pages) * static_cast<uint32_t>(page_size);
    LIYAB_REQUIRE(n >= 0 && n_kv_head > 0 && hd > 0 && page_size > 0, "kv_write: bad sizes");
    LIYAB_REQUIRE(k_off >= 0 && v_off >= 0 && k_off + n_kv_head * hd <= src_stride && v_off + n_kv_head * hd <= src_stride,
                  "kv_write: column offsets %d/%d with %d values do not fit a row of %lld", k_off, v_off, n_kv_head * hd,
                  static_cast<long long>(src_stride));
    if (n == 0) return 0;
    const int threads = n_kv_head * hd >= 256 ? 256 : 64;
    if (dtype == kF32) {
        kv_write_kernel<float><<<n, threads, 0, stream>>>(static_cast<float*>(kc), static_cast<float*>(vc),
                                                          static_cast<const float*>(src), src_stride, k_off, v_off,
                                                          slots, n_kv_head, hd, page_size, num_slots);
    } else if (dtype == kBF16) {
        kv_write_kernel<bf16_t><<<n, threads, 0, stream>>>(static_cast<bf16_t*>(kc), static_cast<bf16_t*>(vc),
                                                           static_cast<const bf16_t*>(src), src_stride, k_off, v_off,
                                                           slots, n_kv_head, hd, page_size, num_slots);
    } else {
        return fail(1, "kv_write: unknown dtype %d", dtype);
    }
    return check_launch("kv_write");
}
