// Causal attention of prompt portions over paged bfloat16 keys and values, on
// the matrix cores (the formulas of the reference's attention,
// src/core/transformer.cpp:2303-2358, blocked as in flash attention: the
// reference's own remark on flash decoding is at :2146-2153).
//
// A work item is (tile of up to 128 consecutive queries of one request, head).
// A workgroup has QG x KS waves: wave (qg, ks) owns the 32 queries of group qg
// and, of every KS consecutive blocks of 32 keys, block ks; the KS partial
// results of a query group are merged at the end in a fixed order. With few
// tiles in flight KS > 1 puts more waves on the longest tile, whose walk over
// the keys is the kernel's critical path. Keys are staged in LDS with their
// values, KS blocks a step. Scores are computed transposed, S^T = K Q^T with
// v_mfma_f32_32x32x16_bf16 (contraction over the head dimension, both operands
// contiguous along it), so that a lane holds 16 scores of ONE query: the
// running maximum and sum of a query need one exchange with the lane 32 apart
// instead of a reduction over 32 lanes. The accumulators then serve, rounded to
// bfloat16, directly as the second operand of O^T = V^T P^T (contraction over
// the keys); V lies in LDS as it lies in the pages, and a wave reads its operand, four keys
// of one dimension a lane, through gfx950's transposing read.
// Exponentials are taken against a reference value that follows the running
// maximum from below by at most 2^8: the outputs are rescaled only when a
// query's maximum jumps past that, which is rare, instead of at every block.
// Maximum, exponentials, sums and outputs are 32-bit. A query's result depends
// on its position and the block grid (multiples of 32 from the window's start),
// not on the batch or the pages. Head sizes: multiples of 16 up to 128.
//
// A block's work is one chain: fragments from LDS, four products into one accumulator, the
// maximum across two lanes, sixteen exponentials, fragments of the values, four products; alone
// it takes about 2,000 cycles for 600 of arithmetic (measured: a tile that walks 1,024 keys took
// 24 us on an otherwise idle chip, 0.018 us a key). With NS = 2 a wave walks two blocks a step
// as two streams with a running maximum, sum and output each: nothing in one stream waits for the
// other, so their chains overlap, and the streams are merged once at the end (in registers, then
// the KS partial results as before).
#include "common.h"
#include "launchers.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// Four 16-bit values through the transposing read of LDS: see where it is used.
__device__ __forceinline__ uint2 tr_read4(const bf16_t* p) {
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s* lds_v4s;
    const v4s v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(p));
    return __builtin_bit_cast(uint2, v);
}

union QFrag {
    u32x4 u;
    bf16x8 v;
    bf16_t h[8];
};

constexpr int AP_KEYS = 32;     // keys per block
constexpr int AP_QUERIES = 128; // queries per tile (4 waves x 32)
constexpr int kDepth = 6;       // blocks of keys and values in flight in registers
constexpr int AP_MAX_BLOCKS = 2048;  // page ids of a tile's keys are kept in LDS

template <int DB, int QG, int KS, int NS = 1>  // head dimension padded to 32 * DB; 32 * QG queries a tile; KS x NS blocks of keys a step, NS a wave
__global__ void __launch_bounds__(64 * QG * KS)
attention_prefill_kernel(bf16_t* __restrict__ out, int64_t out_stride, const bf16_t* __restrict__ q, int64_t q_stride,
                         const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc,
                         const int* __restrict__ block_tables, int max_blocks, const int* __restrict__ work, float scale,
                         int window, int n_head, int n_kv_head, int hd, int page_size, int page_shift, int num_pages) {
    constexpr int HDP = 32 * DB;
    constexpr int LDK = HDP + 8;  // padded row: 16-byte reads of 16 lanes fall in distinct banks
    constexpr int WAVES = QG * KS, THREADS = 64 * WAVES;
    constexpr int AP_DEPTH = kDepth / NS;  // the same bytes in flight whatever a step holds
    constexpr int STEP_KEYS = AP_KEYS * KS * NS;  // keys staged a step
    constexpr int STAGE = STEP_KEYS * LDK;
    // values lie as the keys do, [key of the step][dimension]; the product's operand wants four
    // keys of one dimension a lane, which the transposing read gives (ds_read_b64_tr_b16: 16 lanes
    // that point at 4 keys x 16 dimensions get them back as 16 dimensions x 4 keys)
    constexpr int VSTAGE = STAGE;
    // two stages of keys and of values (the next step's load while this one is used); after the
    // walk the same memory carries the partial results of the waves with ks > 0
    constexpr int PARTIAL = DB * 16 * 64 + 2 * 64;  // floats a wave: outputs, then maximum and sum
    constexpr int KV_BYTES = 2 * (STAGE + VSTAGE) * 2, MERGE_BYTES = (KS - 1) * QG * PARTIAL * 4;
    __shared__ __attribute__((aligned(16))) unsigned char kv_raw[KV_BYTES > MERGE_BYTES ? KV_BYTES : MERGE_BYTES];
    bf16_t* const Kb = reinterpret_cast<bf16_t*>(kv_raw);  // [2][STAGE]
    bf16_t* const Vb = Kb + 2 * STAGE;                     // [2][VSTAGE]
    __shared__ __attribute__((aligned(16))) bf16_t Os[QG][32 * LDK];

    // heads vary fastest: the work list has the longest tiles first, and workgroups start in the
    // grid's order, so that every head's longest tile starts before anybody's short one
    const int* wk = work + 4 * blockIdx.y;
    // (queries and positions within what the tile and the block table hold, whatever the list says)
    const int seq = wk[0], row0 = wk[1], nq = min(max(wk[3], 1), 32 * QG);
    const int pos0 = static_cast<int>(min(static_cast<int64_t>(max(wk[2], 0)), static_cast<int64_t>(max_blocks) * page_size - nq));
    const int h = blockIdx.x;
    const int hkv = h / (n_head / n_kv_head);
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int qg = wave % QG, ks = wave / QG;
    const int ql = lane % 32, g2 = lane / 32;
    const int* bt = block_tables + static_cast<int64_t>(seq) * max_blocks;

    const int my_q = 32 * qg + ql;
    const int qpos = pos0 + min(my_q, nq - 1);  // lanes past the tile's end repeat its last query; never stored
    const int wave_last = pos0 + min(32 * qg + 31, nq - 1);  // the wave's latest query position
    const bool wave_has = 32 * qg < nq;
    const int n_slabs = hd / 16;
    const float scale2 = scale * 1.4426950408889634f;  // log2(e): exp(x) = 2^(x log2 e)

    QFrag qf[2 * DB];
    {
        const bf16_t* qrow = q + static_cast<int64_t>(row0 + min(my_q, nq - 1)) * q_stride + static_cast<int64_t>(h) * hd;
#pragma unroll
        for (int s = 0; s < 2 * DB; ++s) {
            qf[s].u = u32x4{0, 0, 0, 0};
            if (s < n_slabs) qf[s].u = *reinterpret_cast<const u32x4*>(qrow + 16 * s + 8 * g2);
        }
    }
    // per stream: outputs, the reference the exponentials are taken against, and this lane's part
    // of the sum (its own keys: the two lanes of a query add theirs up at the end)
    floatx16 o_s[NS][DB];
    float m_s[NS], l_s[NS];
#pragma unroll
    for (int z = 0; z < NS; ++z) {
        m_s[z] = -INFINITY;
        l_s[z] = 0.0f;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 16; ++r) o_s[z][d][r] = 0.0f;
    }

    const int k_hi = pos0 + nq - 1;  // last key any query of the tile sees
    const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int64_t page_stride = static_cast<int64_t>(n_kv_head) * page_size * hd;
    const int64_t head_off = static_cast<int64_t>(hkv) * page_size * hd;
    constexpr int CHUNKS = 4 * DB;  // 16-byte pieces per padded row
    // a block's keys and values go global -> registers -> LDS (zeros past the head dimension,
    // before the window and past the last key). AP_DEPTH register sets form a ring: a block is
    // fetched AP_DEPTH - 1 blocks before it is multiplied, which covers the latency of the pages.
    constexpr int PER = (STEP_KEYS * CHUNKS + THREADS - 1) / THREADS;
    u32x4 rk[AP_DEPTH][PER], rv[AP_DEPTH][PER];
    // The request's page ids wait in LDS, so that a fetch is one load deep; and a fetch is
    // branch-free (a position outside the range reads a valid one and is zeroed when it is
    // put into LDS): a load under a branch would have to be waited for where the branch ends.
    __shared__ int sbt[AP_MAX_BLOCKS];
    const int first_page = k_lo / page_size, n_pages = k_hi / page_size - first_page + 1;
    // (the host has checked that they fit; an id outside the caches' pages becomes one that exists)
    for (int i = tid; i < n_pages; i += THREADS) sbt[i] = min(max(bt[first_page + i], 0), num_pages - 1);
    __syncthreads();
    auto fetch = [&](int kb, u32x4 (&fk)[PER], u32x4 (&fv)[PER]) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = min(tid + THREADS * i, STEP_KEYS * CHUNKS - 1), key = c / CHUNKS, col = min((c % CHUNKS) * 8, hd - 8);
            const int kp = min(max(kb + key, k_lo), k_hi);
            // page_shift >= 0: the page size is a power of two (no integer division)
            const int lp = page_shift >= 0 ? kp >> page_shift : kp / page_size;
            const int off = page_shift >= 0 ? kp & (page_size - 1) : kp % page_size;
            const int64_t page = sbt[lp - first_page];
            const int64_t at = page * page_stride + head_off + static_cast<int64_t>(off) * hd + col;
            fk[i] = *reinterpret_cast<const u32x4*>(kc + at);
            fv[i] = *reinterpret_cast<const u32x4*>(vc + at);
        }
    };
    auto stash = [&](int buf, int kb, const u32x4 (&fk)[PER], const u32x4 (&fv)[PER]) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int c = tid + THREADS * i, key = c / CHUNKS, col = (c % CHUNKS) * 8;
            if (c < STEP_KEYS * CHUNKS) {
                const int kp = kb + key;
                const bool ok = kp >= k_lo && kp <= k_hi && col < hd;
                const u32x4 zero = {0, 0, 0, 0};
                *reinterpret_cast<u32x4*>(&Kb[buf * STAGE + key * LDK + col]) = ok ? fk[i] : zero;
                *reinterpret_cast<u32x4*>(&Vb[buf * VSTAGE + key * LDK + col]) = ok ? fv[i] : zero;
            }
        }
    };
    const int kb0 = (k_lo / AP_KEYS) * AP_KEYS;
#pragma unroll
    for (int d = 0; d < AP_DEPTH; ++d) fetch(kb0 + d * STEP_KEYS, rk[d], rv[d]);
    stash(0, kb0, rk[0], rv[0]);
    __syncthreads();
    int cur = 0;
    for (int kbase = kb0; kbase <= k_hi; kbase += AP_DEPTH * STEP_KEYS) {
#pragma unroll
      for (int ring = 0; ring < AP_DEPTH; ++ring) {
        const int kb_step = kbase + ring * STEP_KEYS;
        if (kb_step > k_hi) break;
        const bool more = kb_step + STEP_KEYS <= k_hi;
        fetch(kb_step + AP_DEPTH * STEP_KEYS, rk[ring], rv[ring]);  // this set's keys are in LDS already
        const int kb0w = kb_step + ks * NS * AP_KEYS;  // this wave's first block of the step; its NS blocks are consecutive
        const bf16_t* Ks = Kb + cur * STAGE + ks * NS * AP_KEYS * LDK;
        const bf16_t* Vs = Vb + cur * VSTAGE + ks * NS * AP_KEYS * LDK;
        if (wave_has && kb0w <= wave_last) {
            // S^T[key][query] = sum_d K[key][d] Q[query][d], a block a stream. Every slab of the
            // padded head dimension, without a branch (queries and staged keys are zero past the head
            // dimension); the reads of LDS go out together, ahead of the products, and the streams'
            // products alternate. A stream whose block lies past the wave's last query sees every
            // key masked and changes nothing.
            floatx16 st[NS];
            QFrag kf[NS][2 * DB];
#pragma unroll
            for (int z = 0; z < NS; ++z) {
#pragma unroll
                for (int r = 0; r < 16; ++r) st[z][r] = 0.0f;
#pragma unroll
                for (int sl = 0; sl < 2 * DB; ++sl)
                    kf[z][sl].u = *reinterpret_cast<const u32x4*>(Ks + (z * AP_KEYS + ql) * LDK + 16 * sl + 8 * g2);
            }
#pragma unroll
            for (int sl = 0; sl < 2 * DB; ++sl)
#pragma unroll
                for (int z = 0; z < NS; ++z) st[z] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[z][sl].v, qf[sl].v, st[z], 0, 0, 0);
            // this lane: query ql, keys kb + 8 (r / 4) + 4 g2 + r % 4. A block every query of the
            // wave sees whole needs no mask. The maximum is taken over the raw scores (the scale is
            // positive); exponentials are 2^(score * scale2 - reference), one fused multiply-add and
            // one v_exp_f32 a score.
            float bm[NS];
#pragma unroll
            for (int z = 0; z < NS; ++z) {
                const int kb = kb0w + z * AP_KEYS;
                const bool whole = kb + AP_KEYS - 1 <= pos0 + 32 * qg && (window <= 0 || kb > wave_last - window);
                bm[z] = -INFINITY;
                if (whole) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) bm[z] = fmaxf(bm[z], st[z][r]);
                } else {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int kp = kb + 8 * (r / 4) + 4 * g2 + r % 4;
                        const bool ok = kp <= qpos && (window <= 0 || kp > qpos - window);
                        st[z][r] = ok ? st[z][r] : -INFINITY;
                        bm[z] = fmaxf(bm[z], st[z][r]);
                    }
                }
            }
            float other[NS];
#pragma unroll
            for (int z = 0; z < NS; ++z) other[z] = __shfl_xor(bm[z], 32, 64);  // the query's other lane: both exchanges in flight together
            // the reference m_s is raised only when the block's maximum passes it by more than
            // kLag: until then exponentials may reach 2^kLag, which 32-bit sums and bfloat16
            // products hold as well as values below 1
            constexpr float kLag = 8.0f;
            float corr[NS];
            QFrag pf[NS][2];
            bool any = false;
#pragma unroll
            for (int z = 0; z < NS; ++z) {
                const float b = fmaxf(bm[z], other[z]) * scale2;
                corr[z] = 1.0f;
                if (b > m_s[z] + kLag) {  // also the first block with a visible key (m_s = -inf)
                    corr[z] = m_s[z] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_s[z] - b);
                    m_s[z] = b;
                }
                const float ref = m_s[z] == -INFINITY ? 0.0f : m_s[z];  // nothing visible yet: every score is -inf, 2^-inf = 0
                float bs = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pr = __builtin_amdgcn_exp2f(fmaf(st[z][r], scale2, -ref));  // 0 for masked keys
                    bs += pr;
                    pf[z][r / 8].h[r % 8] = float_to_bf16(pr);
                }
                l_s[z] = l_s[z] * corr[z] + bs;  // the reference, and so corr, is the same in both lanes of a query
                any = any || corr[z] != 1.0f;
            }
            const bool rescale = __builtin_amdgcn_ballot_w64(any) != 0;
            // O^T[d][query] += sum_key V[key][d] P[key][query]; instruction s2 contracts the keys
            // of accumulator registers 8 s2 .. 8 s2 + 7: rows 16 s2 + 4 g2 + {0..3} and + 8
#pragma unroll
            for (int d = 0; d < DB; ++d) {
                if (rescale) {
#pragma unroll
                    for (int z = 0; z < NS; ++z)
#pragma unroll
                        for (int r = 0; r < 16; ++r) o_s[z][d][r] *= corr[z];
                }
                union { uint2 u[2]; bf16x8 v; } vf[NS][2];
#pragma unroll
                for (int z = 0; z < NS; ++z)
#pragma unroll
                    for (int s2 = 0; s2 < 2; ++s2) {
                        // this lane gets: dimension 32 d + ql, keys 16 s2 + 4 g2 + {0..3} and the same + 8 of the
                        // stream's block. It points at: of its 16 lanes' 4 keys x 16 dimensions, key (lane % 16) / 4,
                        // dimensions 4 (lane % 4) .. + 3.
                        const bf16_t* vat = Vs + (z * AP_KEYS + 16 * s2 + 4 * g2 + (lane % 16) / 4) * LDK + 32 * d + 16 * ((lane % 32) / 16) + 4 * (lane % 4);
                        vf[z][s2].u[0] = tr_read4(vat);
                        vf[z][s2].u[1] = tr_read4(vat + 8 * LDK);
                    }
#pragma unroll
                for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
                    for (int z = 0; z < NS; ++z)
                        o_s[z][d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[z][s2].v, pf[z][s2].v, o_s[z][d], 0, 0, 0);
            }
        }
        if (more) stash(cur ^ 1, kb_step + STEP_KEYS, rk[(ring + 1) % AP_DEPTH], rv[(ring + 1) % AP_DEPTH]);  // the next step's keys, fetched long ago
        lds_barrier();  // the blocks still in flight stay in flight
        cur ^= 1;
      }
    }
    // the streams of a wave into the first, in their order; then the two lanes of a query add up
    // their parts of the sum
    floatx16 (&o)[DB] = o_s[0];
    float m_run = m_s[0], l_run = l_s[0];
#pragma unroll
    for (int z = 1; z < NS; ++z) {
        const float M = fmaxf(m_run, m_s[z]);
        const float wa = m_run == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run - M);
        const float wb = m_s[z] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_s[z] - M);
        l_run = wa * l_run + wb * l_s[z];
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[d][r] = wa * o[d][r] + wb * o_s[z][d][r];
        m_run = M;
    }
    l_run += __shfl_xor(l_run, 32, 64);
    if constexpr (KS > 1) {
        // the query group's partial results, merged into wave (qg, 0) in the order of ks (the
        // walk's last barrier has passed: nobody reads keys or values any more)
        float* part = reinterpret_cast<float*>(kv_raw);
        if (ks > 0 && wave_has) {
            float* mine = part + ((ks - 1) * QG + qg) * PARTIAL;
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
                for (int r = 0; r < 16; ++r) mine[(d * 16 + r) * 64 + lane] = o[d][r];
            mine[DB * 16 * 64 + lane] = m_run;
            mine[DB * 16 * 64 + 64 + lane] = l_run;
        }
        __syncthreads();
        if (ks == 0 && wave_has) {
#pragma unroll
            for (int k2 = 1; k2 < KS; ++k2) {
                const float* other = part + ((k2 - 1) * QG + qg) * PARTIAL;
                const float mo = other[DB * 16 * 64 + lane], lo = other[DB * 16 * 64 + 64 + lane];
                const float M = fmaxf(m_run, mo);
                const float wa = m_run == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run - M);
                const float wb = mo == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mo - M);
                l_run = wa * l_run + wb * lo;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[d][r] = wa * o[d][r] + wb * other[(d * 16 + r) * 64 + lane];
                m_run = M;
            }
        }
    }
    // o[d][r] = O^T[dim = 32 d + 8 (r / 4) + 4 g2 + r % 4][query ql]: through LDS to rows of 16-byte pieces
    const bool writes = wave_has && ks == 0;
    if (writes) {
        const float inv = 1.0f / l_run;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                Os[qg][ql * LDK + 32 * d + 8 * (r / 4) + 4 * g2 + r % 4] = float_to_bf16(o[d][r] * inv);
    }
    __syncthreads();
    if (writes) {
        const int chunks_row = hd / 8;
        for (int c = lane; c < 32 * chunks_row; c += 64) {
            const int qq = c / chunks_row, col = (c % chunks_row) * 8;
            if (32 * qg + qq < nq) {
                *reinterpret_cast<u32x4*>(out + static_cast<int64_t>(row0 + 32 * qg + qq) * out_stride +
                                          static_cast<int64_t>(h) * hd + col) =
                    *reinterpret_cast<const u32x4*>(&Os[qg][qq * LDK + col]);
            }
        }
    }
}

}  // namespace liyab

using namespace liyab;

// work: n_tiles x (request index, first row, first position, queries <= tile), int32; tile = 64 or 128
// queries (2 or 4 groups of 32); ksplit = 1, 2 or 4 waves share a query group's keys (128-query tiles: 1 or 2).
// num_pages: the pages the caches hold; page ids of the block tables are brought into [0, num_pages).
extern "C" int liyab_attention_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc,
                                       const void* vc, const int* block_tables, int max_blocks, const int* work,
                                       int n_tiles, int tile, int ksplit, float scale, int window, int n_head, int n_kv_head, int hd,
                                       int page_size, int num_pages, hipStream_t stream) {
    LIYAB_REQUIRE(out && q && kc && vc && block_tables && work, "attention_prefill: null pointer");
    LIYAB_REQUIRE(num_pages > 0, "attention_prefill: the caches hold %d pages", num_pages);
    LIYAB_REQUIRE(n_tiles >= 0 && n_head > 0 && n_kv_head > 0 && page_size > 0 && max_blocks > 0, "attention_prefill: bad sizes");
    LIYAB_REQUIRE(n_head % n_kv_head == 0 && n_head <= 65535, "attention_prefill: %d query heads are no multiple of %d key/value heads", n_head, n_kv_head);
    LIYAB_REQUIRE(hd >= 16 && hd <= 128 && hd % 16 == 0, "attention_prefill: head size %d is not a multiple of 16 in 16..128", hd);
    LIYAB_REQUIRE(q_stride % 8 == 0 && out_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(q) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (reinterpret_cast<uintptr_t>(kc) & 15) == 0 &&
                      (reinterpret_cast<uintptr_t>(vc) & 15) == 0,
                  "attention_prefill: operands must be 16-byte aligned with strides that are multiples of 8");
    LIYAB_REQUIRE(out_stride >= static_cast<int64_t>(n_head) * hd && q_stride >= static_cast<int64_t>(n_head) * hd,
                  "attention_prefill: row strides are shorter than heads x head size");
    LIYAB_REQUIRE(window >= 0, "attention_prefill: negative window");
    LIYAB_REQUIRE(scale > 0.0f, "attention_prefill: the scale must be positive (the maximum is taken before scaling), not %g", scale);
    LIYAB_REQUIRE(tile == 64 || tile == 128, "attention_prefill: tiles of %d queries; 64 or 128 are taken", tile);
    LIYAB_REQUIRE(ksplit == 1 || ksplit == 2 || (ksplit == 4 && tile == 64), "attention_prefill: %d waves a query group do not go with tiles of %d", ksplit, tile);
    LIYAB_REQUIRE(ksplit < 4 || hd <= 64, "attention_prefill: 4 waves a query group are taken up to head size 64, not %d", hd);
    LIYAB_REQUIRE(max_blocks <= AP_MAX_BLOCKS, "attention_prefill: block tables of %d pages; at most %d are taken", max_blocks, AP_MAX_BLOCKS);
    if (n_tiles == 0) return 0;
    int page_shift = -1;
    for (int b = 0; b < 31; ++b)
        if ((1 << b) == page_size) page_shift = b;
    dim3 grid(n_head, n_tiles);
    auto* o = static_cast<bf16_t*>(out);
    auto* pq = static_cast<const bf16_t*>(q);
    auto* pk = static_cast<const bf16_t*>(kc);
    auto* pv = static_cast<const bf16_t*>(vc);
#define LIYAB_RUN(D, Q, S)                                                                                          \
    attention_prefill_kernel<D, Q, S, (D <= 2 && Q == 4 && S <= 2) ? 2 : 1><<<grid, 64 * Q * S, 0, stream>>>(                          \
        o, out_stride, pq, q_stride, pk, pv, block_tables, max_blocks, work, scale, window, n_head, n_kv_head, hd, page_size, page_shift, num_pages)
#define LIYAB_RUN4(D) LIYAB_RUN(D, 2, 4)
#define LIYAB_SKIP4(D) (void)0  // four stages of 128 keys do not fit LDS at these head sizes (refused above)
#define LIYAB_GO(D, FOUR)                           \
    do {                                            \
        if (tile == 64) {                           \
            if (ksplit == 1) LIYAB_RUN(D, 2, 1);    \
            else if (ksplit == 2) LIYAB_RUN(D, 2, 2); \
            else FOUR(D);                           \
        } else {                                    \
            if (ksplit == 1) LIYAB_RUN(D, 4, 1);    \
            else LIYAB_RUN(D, 4, 2);                \
        }                                           \
    } while (0)
    if (hd <= 32) LIYAB_GO(1, LIYAB_RUN4);
    else if (hd <= 64) LIYAB_GO(2, LIYAB_RUN4);
    else if (hd <= 96) LIYAB_GO(3, LIYAB_SKIP4);
    else LIYAB_GO(4, LIYAB_SKIP4);
#undef LIYAB_GO
#undef LIYAB_RUN4
#undef LIYAB_SKIP4
#undef LIYAB_RUN
    return check_launch("attention_prefill");
}
