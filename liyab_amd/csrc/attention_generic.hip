// Causal attention over paged keys and values: the plain kernel.
//
// One workgroup per (token, query head). The token's query sees the keys of
// its own request at positions [first, pos], first = 0 or pos - window + 1
// (the reference's attention, src/core/transformer.cpp:2162-2453: scores
// s_j = (k_j . q) * scale :2303-2313, softmax with the maximum subtracted
// :2327-2341, weighted values :2344-2358). Keys are visited in tiles of 256
// positions with a running maximum and sum, in position order, so the way a
// query's attention rounds depends on its position only: not on how the
// prompt was cut into steps, on the rest of the batch, or on which pages
// hold the keys (the property the reference states at :2136-2139).
// Scores, exponentials, sums and the output are 32-bit; keys and values are
// read at the cache's precision. It serves the true 32-bit path and any
// head size up to 256 on the bfloat16 path.
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int ATT_THREADS = 256;

template <typename T>
__global__ void __launch_bounds__(ATT_THREADS)
attention_generic_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
                         const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ block_tables,
                         int max_blocks, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, float scale,
                         int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages) {
    extern __shared__ float smem[];
    float* qs = smem;                    // [hd]
    float* sc = qs + hd;                 // [ATT_THREADS]
    float* red = sc + ATT_THREADS;       // [ATT_THREADS / kWave]
    float* accs = red + ATT_THREADS / kWave;  // [G][hd] for the final sum over groups

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int pos = static_cast<int>(min(static_cast<int64_t>(max(tok_pos[t], 0)), static_cast<int64_t>(max_blocks) * page_size - 1));  // within the table's reach
    const int* bt = block_tables + static_cast<int64_t>(tok_seq[t]) * max_blocks;
    const int hkv = h / (n_head / n_kv_head);
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const T* qrow = q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * hd;
    for (int e = tid; e < hd; e += ATT_THREADS) qs[e] = to_float<T>(qrow[e]);
    __syncthreads();

    const int G = ATT_THREADS / hd;  // groups of hd threads sharing the keys of a tile
    const int g = tid / hd, e = tid % hd;
    const bool vthread = g < G;
    float m = -INFINITY, l = 0.0f, acc = 0.0f;

    for (int j0 = first; j0 <= pos; j0 += ATT_THREADS) {
        const int j = j0 + tid;
        float s = -INFINITY;
        if (j <= pos) {
            const int64_t page = min(max(bt[j / page_size], 0), num_pages - 1);  // whatever the table holds, a page of the caches
            const T* kr = kc + ((page * n_kv_head + hkv) * page_size + j % page_size) * hd;
            float dot = 0.0f;
            for (int i = 0; i < hd; ++i) dot = fmaf(to_float<T>(kr[i]), qs[i], dot);
            s = dot * scale;
        }
        // tile maximum
        float tm = wave_max(s);
        if (lane == 0) red[wave] = tm;
        __syncthreads();
        tm = red[0];
#pragma unroll
        for (int i = 1; i < ATT_THREADS / kWave; ++i) tm = fmaxf(tm, red[i]);
        const float m_new = fmaxf(m, tm);
        const float p = j <= pos ? expf(s - m_new) : 0.0f;
        sc[tid] = p;
        float ps = wave_sum(p);
        __syncthreads();  // every thread has read red[] for the maximum
        if (lane == 0) red[wave] = ps;
        __syncthreads();
        ps = 0.0f;
#pragma unroll
        for (int i = 0; i < ATT_THREADS / kWave; ++i) ps += red[i];
        const float corr = expf(m - m_new);  // 0 on the first tile (m = -inf)
        l = l * corr + ps;
        acc *= corr;
        m = m_new;
        if (vthread) {
            const int len = min(ATT_THREADS, pos - j0 + 1);
            for (int jj = g; jj < len; jj += G) {
                const int jv = j0 + jj;
                const int64_t page = min(max(bt[jv / page_size], 0), num_pages - 1);
                const T* vr = vc + ((page * n_kv_head + hkv) * page_size + jv % page_size) * hd;
                acc = fmaf(sc[jj], to_float<T>(vr[e]), acc);
            }
        }
        __syncthreads();  // sc[] and red[] are rewritten by the next tile
    }
    if (vthread) accs[g * hd + e] = acc;
    __syncthreads();
    if (tid < hd) {
        float o = 0.0f;
        for (int i = 0; i < G; ++i) o += accs[i * hd + tid];
        out[static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * hd + tid] = from_float<T>(o / l);
    }
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_attention_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc,
                                       const void* vc, int dtype, const int* block_tables, int max_blocks,
                                       const int* tok_seq, const int* tok_pos, int n, float scale, int window,
                                       int n_head, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream) {
    LIYAB_REQUIRE(out && q && kc && vc && block_tables && tok_seq && tok_pos, "attention: null pointer");
    LIYAB_REQUIRE(num_pages > 0, "attention: the caches hold %d pages", num_pages);
    LIYAB_REQUIRE(n >= 0 && n_head > 0 && n_kv_head > 0 && page_size > 0 && max_blocks > 0, "attention: bad sizes");
    LIYAB_REQUIRE(n_head % n_kv_head == 0, "attention: %d query heads are no multiple of %d key/value heads", n_head,
                  n_kv_head);
    LIYAB_REQUIRE(hd > 0 && hd <= 256, "attention: head size %d is outside 1..256", hd);
    LIYAB_REQUIRE(out_stride >= static_cast<int64_t>(n_head) * hd && q_stride >= static_cast<int64_t>(n_head) * hd,
                  "attention: row strides are shorter than heads x head size");
    LIYAB_REQUIRE(window >= 0, "attention: negative window");
    if (n == 0) return 0;
    const int G = ATT_THREADS / hd;
    const size_t smem = sizeof(float) * (hd + ATT_THREADS + ATT_THREADS / kWave + static_cast<size_t>(G) * hd);
    dim3 grid(n, n_head);
    if (dtype == kF32) {
        attention_generic_kernel<float><<<grid, ATT_THREADS, smem, stream>>>(
            static_cast<float*>(out), out_stride, static_cast<const float*>(q), q_stride, static_cast<const float*>(kc),
            static_cast<const float*>(vc), block_tables, max_blocks, tok_seq, tok_pos, scale, window, n_head, n_kv_head,
            hd, page_size, num_pages);
    } else if (dtype == kBF16) {
        attention_generic_kernel<bf16_t><<<grid, ATT_THREADS, smem, stream>>>(
            static_cast<bf16_t*>(out), out_stride, static_cast<const bf16_t*>(q), q_stride,
            static_cast<const bf16_t*>(kc), static_cast<const bf16_t*>(vc), block_tables, max_blocks, tok_seq, tok_pos,
            scale, window, n_head, n_kv_head, hd, page_size, num_pages);
    } else {
        return fail(1, "attention: unknown dtype %d", dtype);
    }
    return check_launch("attention_generic");
}
