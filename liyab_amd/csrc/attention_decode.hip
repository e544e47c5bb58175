// Attention for tokens taken one at a time (decoding, short prompt portions)
// over paged keys and values (bfloat16, or 32-bit for the 32-bit path), with
// the keys of a token cut into splits so that few tokens still fill the chip.
//
// Grid (token, query head, split). A workgroup of 4 or 16 waves walks its split's
// keys; LPK lanes share a key (each holds 8 consecutive dimensions, 16
// bytes), so a wave takes 64 / LPK keys a pass, read straight from the pages
// through the block table. Each lane group keeps a running maximum, sum and
// weighted values (the reference's per-span partial softmax,
// src/core/transformer.cpp:2327-2358); groups, then waves, then splits are
// merged in a fixed order by rescaling to the common maximum (:2367-2385).
// With `chunk` keys a split (instead of the token's keys divided by the number of
// splits) and four waves, which lane adds which key and which sums are merged
// follow from the token's position alone, as the reference cuts (:2136-2139):
// the form of the 32-bit path and of the batch-invariant mode.
// The reference cuts a token's keys by its position only (:2136-2139,
// 2225-2227) to keep bits equal; here the number of splits follows the batch
// (more splits when few tokens are in flight), which moves results by
// rounding only. Scores, exponentials and sums are 32-bit.
#include "common.h"
#include "launchers.h"

namespace liyab {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int AD_MAX_BLOCKS = 2048;  // page ids of a request kept in LDS
constexpr int AD_LOOP_CHUNKS = 16;   // splits by position that one workgroup walks in turn, at most


__device__ __forceinline__ void unpack8(const u32x4& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(v[i] << 16);
        f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
}

// 8 consecutive elements of a row as they are loaded (bfloat16 stays packed until it is used), and as floats
typedef __attribute__((ext_vector_type(4))) float f32x4;
struct Raw8F { f32x4 a, b; };
__device__ __forceinline__ u32x4 fetch8(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ Raw8F fetch8(const float* p) {
    return Raw8F{*reinterpret_cast<const f32x4*>(p), *reinterpret_cast<const f32x4*>(p + 4)};
}
__device__ __forceinline__ void unpack8(const Raw8F& v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) { f[i] = v.a[i]; f[4 + i] = v.b[i]; }
}
template <typename T> struct Raw8 { typedef u32x4 type; };
template <> struct Raw8<float> { typedef Raw8F type; };
// exponentials of scores: the fast one beside bfloat16 data, the library's beside 32-bit data
template <typename T> __device__ __forceinline__ float exp_for(float x) { return __expf(x); }
template <> __device__ __forceinline__ float exp_for<float>(float x) { return expf(x); }

struct Partial {
    float m, l;
    float acc[8];
};

// this <- merge(this, other): both rescaled to the larger maximum; this comes first.
template <typename T>
__device__ __forceinline__ void merge_partial(Partial& a, float mo, float lo, const float* acco) {
    const float M = fmaxf(a.m, mo);
    const float wa = a.m == -INFINITY ? 0.0f : exp_for<T>(a.m - M);
    const float wb = mo == -INFINITY ? 0.0f : exp_for<T>(mo - M);
    a.l = wa * a.l + wb * lo;
#pragma unroll
    for (int e = 0; e < 8; ++e) a.acc[e] = wa * a.acc[e] + wb * acco[e];
    a.m = M;
}

template <typename T, int LPK, int AD_WAVES, int AD_U>
__global__ void __launch_bounds__(64 * AD_WAVES)
attention_decode_kernel(T* __restrict__ out, int64_t out_stride, const T* __restrict__ q, int64_t q_stride,
                        const T* __restrict__ kc, const T* __restrict__ vc,
                        const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ tok_list,
                        const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, float scale, int window,
                        int n_head, int n_kv_head, int hd, int page_size, int page_shift, int rows_are_requests,
                        int n_splits, int chunk, float* __restrict__ partials, int num_pages) {
    constexpr int KPP = 64 / LPK;  // keys per wave and pass
    __shared__ float lds2[2][AD_WAVES][LPK][10];  // the waves' sums, for the first wave to merge; two of them in turn, so that one barrier a split is enough
    const int t = tok_list != nullptr ? tok_list[blockIdx.x] : blockIdx.x;
    const int h = blockIdx.y, z = blockIdx.z;
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int c = lane % LPK, kg = lane / LPK;
    const bool active = c * 8 < hd;
    // The request's page ids go to LDS first, so that fetching a key is one load deep; they are
    // loaded together with the position and the query (when every row is its own request the
    // block-table row is known without looking the request up).
    __shared__ int sbt[AD_MAX_BLOCKS];
    const int seq = rows_are_requests ? t : tok_seq[t];
    const int* bt = block_tables + static_cast<int64_t>(seq) * max_blocks;
    // (an id outside the caches' pages, an unmapped -1 or a wrong word, becomes a page that exists:
    // whatever a table holds, no fetch leaves the caches)
    for (int i = tid; i < max_blocks; i += 64 * AD_WAVES) sbt[i] = min(max(bt[i], 0), num_pages - 1);
    // (a position past the block table's reach would index the staged ids out of range)
    const int pos = static_cast<int>(min(static_cast<int64_t>(max(tok_pos[t], 0)), static_cast<int64_t>(max_blocks) * page_size - 1));
    const int hkv = h / (n_head / n_kv_head);
    // lanes past the head dimension read column 0 and multiply it by a zero query
    const int col = active ? c * 8 : 0;
    float qf[8];
    unpack8(fetch8(q + static_cast<int64_t>(t) * q_stride + static_cast<int64_t>(h) * hd + col), qf);
    if (!active) {
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[e] = 0.0f;
    }
    __syncthreads();
    const int first = window > 0 ? max(0, pos - window + 1) : 0;
    const int n_keys = pos - first + 1;
    // Splits by position launched as one (chunk > 0, n_splits == 1): the workgroup walks the token's
    // splits one after the other, keeps each one's sums apart and merges them at the end as the merge
    // kernel would, operation for operation: the bits of the split launch without its traffic, for
    // steps of many tokens.
    const bool walks_all = chunk > 0 && n_splits == 1;
    const int z_count = walks_all ? min(AD_LOOP_CHUNKS, max(1, (n_keys + chunk - 1) / chunk)) : 1;  // (the launcher has checked that they fit)
    __shared__ float stash[AD_LOOP_CHUNKS][LPK][10];
    for (int zi = 0; zi < z_count; ++zi) {
    float (&lds)[AD_WAVES][LPK][10] = lds2[zi & 1];
    const int zz = walks_all ? zi : z;
    // split zz: its share of the keys, or keys [zz * chunk, (zz + 1) * chunk) of them (none, for a short context)
    const int k_begin = first + (chunk > 0 ? zz * chunk : static_cast<int>(static_cast<int64_t>(n_keys) * zz / n_splits));
    const int k_end = chunk > 0 ? min(pos + 1, k_begin + chunk) : first + static_cast<int>(static_cast<int64_t>(n_keys) * (zz + 1) / n_splits);
    Partial st;
    st.m = -INFINITY;
    st.l = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) st.acc[e] = 0.0f;

    const int64_t head_off = static_cast<int64_t>(hkv) * page_size * hd + col;
    const int64_t page_stride = static_cast<int64_t>(n_kv_head) * page_size * hd;
    for (int j0 = k_begin + wave * KPP; j0 < k_end; j0 += AD_WAVES * KPP * AD_U) {
        typename Raw8<T>::type kv[AD_U], vv[AD_U];
        bool valid[AD_U];
#pragma unroll
        for (int u = 0; u < AD_U; ++u) {
            const int j = j0 + u * AD_WAVES * KPP + kg;
            valid[u] = j < k_end;
            const int jc = valid[u] ? j : pos;  // a mapped position; its values are not used
            // no branch around the loads: a load under a branch is waited for where the branch ends
            const int lp = page_shift >= 0 ? jc >> page_shift : jc / page_size;
            const int off = page_shift >= 0 ? jc & (page_size - 1) : jc % page_size;
            const int64_t at = static_cast<int64_t>(sbt[lp]) * page_stride + head_off + static_cast<int64_t>(off) * hd;
            kv[u] = fetch8(kc + at);
            vv[u] = fetch8(vc + at);
        }
        float s[AD_U];
        float m_new = st.m;
#pragma unroll
        for (int u = 0; u < AD_U; ++u) {
            float kf[8];
            unpack8(kv[u], kf);
            float d = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) d = fmaf(kf[e], qf[e], d);
            d = group_sum<LPK>(d);  // over the lanes that share the key
            s[u] = valid[u] ? d * scale : -INFINITY;
            m_new = fmaxf(m_new, s[u]);
        }
        if (m_new == -INFINITY) continue;  // this lane group had no key in this trip (and none before)
        const float corr = st.m == -INFINITY ? 0.0f : exp_for<T>(st.m - m_new);
        st.l *= corr;
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[e] *= corr;
#pragma unroll
        for (int u = 0; u < AD_U; ++u) {
            if (!valid[u]) continue;
            const float p = exp_for<T>(s[u] - m_new);
            st.l += p;
            float vf[8];
            unpack8(vv[u], vf);
#pragma unroll
            for (int e = 0; e < 8; ++e) st.acc[e] = fmaf(p, vf[e], st.acc[e]);
        }
        st.m = m_new;
    }
    // lane groups of the wave, in a fixed tree
#pragma unroll
    for (int off = LPK; off < 64; off <<= 1) {
        const float mo = __shfl_xor(st.m, off, 64), lo = __shfl_xor(st.l, off, 64);
        float ao[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) ao[e] = __shfl_xor(st.acc[e], off, 64);
        merge_partial<T>(st, mo, lo, ao);
    }
    if (kg == 0) {
        lds[wave][c][0] = st.m;
        lds[wave][c][1] = st.l;
#pragma unroll
        for (int e = 0; e < 8; ++e) lds[wave][c][2 + e] = st.acc[e];
    }
    __syncthreads();
    if (wave == 0 && kg == 0 && active) {
#pragma unroll
        for (int w = 1; w < AD_WAVES; ++w) merge_partial<T>(st, lds[w][c][0], lds[w][c][1], &lds[w][c][2]);
        if (z_count > 1) {
            stash[zi][c][0] = st.m;
            stash[zi][c][1] = st.l;
#pragma unroll
            for (int e = 0; e < 8; ++e) stash[zi][c][2 + e] = st.acc[e];
        } else if (n_splits == 1) {
            T* o = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * hd + c * 8;
            if (chunk > 0) {
                // as the merge of several splits divides: a token has the same bits alone in one split
                // and beside longer contexts, its later splits empty
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = from_float<T>(st.acc[e] / st.l);
            } else {
                const float inv = 1.0f / st.l;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = from_float<T>(st.acc[e] * inv);
            }
        } else {
            // partials [token slot][head][split][hd + 4]: values, then maximum and sum (and two
            // unused, which keep every split's values 16-byte aligned)
            float* p = partials + ((static_cast<int64_t>(blockIdx.x) * n_head + h) * n_splits + z) * (hd + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) p[c * 8 + e] = st.acc[e];
            if (c == 0) {
                p[hd] = st.m;
                p[hd + 1] = st.l;
            }
        }
    }
    }
    if (z_count > 1 && wave == 0 && kg == 0 && active) {
        // (each lane reads what it wrote itself)
        float M = -INFINITY;
        for (int zi = 0; zi < z_count; ++zi) M = fmaxf(M, stash[zi][c][0]);
        float sum = 0.0f, o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = 0.0f;
        for (int zi = 0; zi < z_count; ++zi) {
            const float m = stash[zi][c][0];
            if (m == -INFINITY) continue;
            const float w = exp_for<T>(m - M);
            sum = fmaf(w, stash[zi][c][1], sum);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = fmaf(w, stash[zi][c][2 + e], o[e]);
        }
        T* dst = out + static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * hd + c * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = from_float<T>(o[e] / sum);
    }
}

// Splits of a (token, head) merged in split order (the same operations as the end of the kernel above).
template <typename T>
__global__ void attention_merge_kernel(T* __restrict__ out, int64_t out_stride, const int* __restrict__ tok_list,
                                       const float* __restrict__ partials, int n_head, int hd, int n_splits) {
    // The splits' maxima and sums go to LDS first, a lane a split, and the values are fetched
    // eight splits at a time before they are used: the sums below are one chain in split order,
    // and a load at a time inside it would cost its latency once a split.
    __shared__ float sm[64], sl[64];
    const int slot = blockIdx.x, h = blockIdx.y, e = threadIdx.x;
    const int t = tok_list != nullptr ? tok_list[slot] : slot;
    const float* p = partials + (static_cast<int64_t>(slot) * n_head + h) * n_splits * (hd + 4);
    const int ec = min(e, hd - 1);
    float a[8];  // the first eight splits' values are on their way while the maxima and sums go through LDS
#pragma unroll
    for (int u = 0; u < 8; ++u) a[u] = p[min(u, n_splits - 1) * (hd + 4) + ec];
    for (int z = e; z < n_splits; z += blockDim.x) {
        sm[z] = p[z * (hd + 4) + hd];
        sl[z] = p[z * (hd + 4) + hd + 1];
    }
    __syncthreads();
    if (e >= hd) return;
    float M = -INFINITY;
    for (int z = 0; z < n_splits; ++z) M = fmaxf(M, sm[z]);
    float sum = 0.0f, o = 0.0f;
    for (int z0 = 0; z0 < n_splits; z0 += 8) {
        if (z0 > 0) {
#pragma unroll
            for (int u = 0; u < 8; ++u) a[u] = p[min(z0 + u, n_splits - 1) * (hd + 4) + e];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (z0 + u >= n_splits) break;
            const float m = sm[z0 + u];
            if (m == -INFINITY) continue;
            const float w = exp_for<T>(m - M);
            sum = fmaf(w, sl[z0 + u], sum);
            o = fmaf(w, a[u], o);
        }
    }
    out[static_cast<int64_t>(t) * out_stride + static_cast<int64_t>(h) * hd + e] = from_float<T>(o / sum);
}

template <typename T>
int launch_attention_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc,
                            const int* block_tables, int max_blocks, const int* tok_list, const int* tok_seq,
                            const int* tok_pos, int n, float scale, int window, int n_head, int n_kv_head, int hd,
                            int page_size, int n_splits, int chunk, int waves, int rows_are_requests, float* partials,
                            int leave_splits, int num_pages, hipStream_t stream) {
    int page_shift = -1;
    for (int b = 0; b < 31; ++b)
        if ((1 << b) == page_size) page_shift = b;
    dim3 grid(n, n_head, n_splits);
    auto* o = static_cast<T*>(out);
    auto* pq = static_cast<const T*>(q);
    auto* pk = static_cast<const T*>(kc);
    auto* pv = static_cast<const T*>(vc);
#define LIYAB_GO(L)                                                                                                  \
    do {                                                                                                             \
        if (waves == 4)                                                                                              \
            attention_decode_kernel<T, L, 4, 4><<<grid, 256, 0, stream>>>(o, out_stride, pq, q_stride, pk, pv, block_tables, \
                                                                    max_blocks, tok_list, tok_seq, tok_pos, scale,   \
                                                                    window, n_head, n_kv_head, hd, page_size, page_shift, rows_are_requests, n_splits, chunk, partials, num_pages); \
        else if (waves == 8)                                                                                         \
            attention_decode_kernel<T, L, 8, 4><<<grid, 512, 0, stream>>>(o, out_stride, pq, q_stride, pk, pv, block_tables, \
                                                                    max_blocks, tok_list, tok_seq, tok_pos, scale,   \
                                                                    window, n_head, n_kv_head, hd, page_size, page_shift, rows_are_requests, n_splits, chunk, partials, num_pages); \
        else                                                                                                         \
            attention_decode_kernel<T, L, 16, sizeof(T) == 2 ? 8 : 4><<<grid, 1024, 0, stream>>>(o, out_stride, pq, q_stride, pk, pv, block_tables, \
                                                                      max_blocks, tok_list, tok_seq, tok_pos, scale, \
                                                                      window, n_head, n_kv_head, hd, page_size, page_shift, rows_are_requests, n_splits, chunk, partials, num_pages); \
    } while (0)
    if (hd <= 8) LIYAB_GO(1);
    else if (hd <= 16) LIYAB_GO(2);
    else if (hd <= 32) LIYAB_GO(4);
    else if (hd <= 64) LIYAB_GO(8);
    else if (hd <= 128) LIYAB_GO(16);
    else LIYAB_GO(32);
#undef LIYAB_GO
    if (int rc = check_launch("attention_decode")) return rc;
    if (n_splits > 1 && !leave_splits) {
        attention_merge_kernel<T><<<dim3(n, n_head), ((hd + 63) / 64) * 64, 0, stream>>>(o, out_stride, tok_list, partials, n_head, hd, n_splits);
        return check_launch("attention_merge");
    }
    return 0;
}
}  // namespace liyab

using namespace liyab;

// Tokens tok_list[0..n) (or 0..n-1 when tok_list is null), each on its own. `partials` must hold
// n * n_head * n_splits * (hd + 4) floats when n_splits > 1. With `leave_splits` (n_splits > 1)
// the splits are not merged and `out` is not written: partials[token slot][head][split] holds
// hd weighted values, then the split's maximum and sum (an empty split: -inf and 0), for a
// reader that merges them as it loads them (the output projection cut over its inner dimension).
// dtype: the element type of out, q and the caches (bfloat16 or 32-bit floats). chunk: 0 = each
// split an equal share of the token's keys; > 0 = split z takes keys [z * chunk, (z + 1) * chunk)
// of the token's (n_splits * chunk must cover the longest context: keys beyond are not read).
// num_pages: the pages the caches hold; page ids of the block tables are brought into [0, num_pages).
extern "C" int liyab_attention_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc,
                                      const void* vc, int dtype, const int* block_tables, int max_blocks, const int* tok_list,
                                      const int* tok_seq, const int* tok_pos, int n, float scale, int window,
                                      int n_head, int n_kv_head, int hd, int page_size, int n_splits, int chunk, int waves,
                                      int rows_are_requests, float* partials, int leave_splits, int num_pages, hipStream_t stream) {
    LIYAB_REQUIRE(num_pages > 0, "attention_decode: the caches hold %d pages", num_pages);
    LIYAB_REQUIRE((out || leave_splits) && q && kc && vc && block_tables && tok_seq && tok_pos, "attention_decode: null pointer");
    LIYAB_REQUIRE(dtype == kBF16 || dtype == kF32, "attention_decode: unknown dtype %d", dtype);
    LIYAB_REQUIRE(!leave_splits || n_splits > 1, "attention_decode: splits are left only when there are several");
    LIYAB_REQUIRE(n >= 0 && n_head > 0 && n_kv_head > 0 && page_size > 0 && max_blocks > 0, "attention_decode: bad sizes");
    LIYAB_REQUIRE(n_head % n_kv_head == 0, "attention_decode: %d query heads are no multiple of %d key/value heads", n_head, n_kv_head);
    LIYAB_REQUIRE(hd >= 8 && hd <= 256 && hd % 8 == 0, "attention_decode: head size %d is not a multiple of 8 in 8..256", hd);
    const int per16 = dtype == kBF16 ? 8 : 4;  // elements in 16 bytes
    LIYAB_REQUIRE(q_stride % per16 == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0 && (reinterpret_cast<uintptr_t>(kc) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(vc) & 15) == 0,
                  "attention_decode: queries and caches must be 16-byte aligned with a query stride that is a multiple of 16 bytes");
    LIYAB_REQUIRE(out_stride >= static_cast<int64_t>(n_head) * hd && q_stride >= static_cast<int64_t>(n_head) * hd,
                  "attention_decode: row strides are shorter than heads x head size");
    LIYAB_REQUIRE(n_splits >= 1 && n_splits <= 64 && (n_splits == 1 || partials != nullptr), "attention_decode: bad split count %d", n_splits);
    LIYAB_REQUIRE(window >= 0 && n_head <= 65535, "attention_decode: bad window or head count");
    LIYAB_REQUIRE(chunk >= 0, "attention_decode: a negative number of keys a split");
    LIYAB_REQUIRE(chunk == 0 || n_splits > 1 || static_cast<int64_t>(chunk) * AD_LOOP_CHUNKS >= static_cast<int64_t>(max_blocks) * page_size ||
                      (window > 0 && static_cast<int64_t>(chunk) * AD_LOOP_CHUNKS >= window),
                  "attention_decode: one workgroup walks at most %d splits of %d keys; contexts of %lld need a launch in splits", AD_LOOP_CHUNKS,
                  chunk, static_cast<long long>(max_blocks) * page_size);
    LIYAB_REQUIRE(max_blocks <= AD_MAX_BLOCKS, "attention_decode: block tables of %d pages; at most %d are taken", max_blocks, AD_MAX_BLOCKS);
    LIYAB_REQUIRE(!rows_are_requests || tok_list == nullptr, "attention_decode: rows_are_requests does not go with a row list");
    LIYAB_REQUIRE(waves == 4 || waves == 8 || waves == 16, "attention_decode: %d waves per workgroup is not 4, 8 or 16", waves);
    if (n == 0) return 0;
    if (dtype == kF32)
        return launch_attention_decode<float>(out, out_stride, q, q_stride, kc, vc, block_tables, max_blocks, tok_list, tok_seq,
                                              tok_pos, n, scale, window, n_head, n_kv_head, hd, page_size, n_splits, chunk, waves,
                                              rows_are_requests, partials, leave_splits, num_pages, stream);
    return launch_attention_decode<bf16_t>(out, out_stride, q, q_stride, kc, vc, block_tables, max_blocks, tok_list, tok_seq,
                                           tok_pos, n, scale, window, n_head, n_kv_head, hd, page_size, n_splits, chunk, waves,
                                           rows_are_requests, partials, leave_splits, num_pages, stream);
}

// out[m, h * hd + e] = the splits of (m, h) merged in split order: for splits that
// liyab_attention_decode left unmerged and no reader takes as they are.
extern "C" int liyab_attention_merge(void* out, int out_dtype, int64_t out_stride, const float* partials, int n, int n_head,
                                     int hd, int n_splits, hipStream_t stream) {
    LIYAB_REQUIRE(out && partials, "attention_merge: null pointer");
    LIYAB_REQUIRE(n >= 0 && n_head > 0 && n_head <= 65535 && hd > 0 && hd <= 1024 && n_splits >= 1 && n_splits <= 64, "attention_merge: bad sizes (at most 64 splits)");
    LIYAB_REQUIRE(out_stride >= static_cast<int64_t>(n_head) * hd, "attention_merge: the row stride is shorter than heads x head size");
    LIYAB_REQUIRE(out_dtype == kBF16 || out_dtype == kF32, "attention_merge: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    const dim3 grid(n, n_head);
    const int threads = ((hd + 63) / 64) * 64;
    if (out_dtype == kF32)
        attention_merge_kernel<float><<<grid, threads, 0, stream>>>(static_cast<float*>(out), out_stride, nullptr, partials, n_head, hd, n_splits);
    else
        attention_merge_kernel<bf16_t><<<grid, threads, 0, stream>>>(static_cast<bf16_t*>(out), out_stride, nullptr, partials, n_head, hd, n_splits);
    return check_launch("attention_merge");
}
