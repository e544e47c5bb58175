// Sampling on the device: argmax, and temperature -> top-k -> top-p ->
// renormalise -> inverse CDF over ascending ids, the order and rules of the
// reference's Sampler (src/core/sampling.cpp:12-79):
//   * greedy (temperature <= 0): the first maximal element, so ties go to
//     the lowest id (:12-14);
//   * top-k keeps the k largest logits (:28-32), top-p the shortest prefix
//     of the descending order whose share reaches top_p (:43-60); ties in
//     either order are taken by ascending id here (the reference leaves
//     them to its sort);
//   * p_i = exp((l_i - l_max) / T) in float, sums in double (:34-41);
//   * the draw r in [0, total) walks the ids upwards subtracting p_i and
//     stops at the first r < 0; the last id with mass is the fallback
//     (:65-79).
// The uniform number of a row comes from the host (a counter-based
// generator keyed by the request's seed and token index), so a request
// draws the same tokens alone or in any batch. One workgroup per row; every
// count and sum is reduced in a fixed order.
#include "common.h"

namespace liyab {

constexpr int S_THREADS = 1024;
constexpr int S_WAVES = S_THREADS / kWave;

__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// Sum over the workgroup; every thread gets the result. `red` holds S_WAVES values.
__device__ __forceinline__ double block_sum_d(double v, double* red) {
    v = wave_sum_d(v);
    __syncthreads();
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    double t = 0.0;
#pragma unroll
    for (int i = 0; i < S_WAVES; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ int block_sum_i(int v, int* red) {
    v = wave_sum_i(v);
    __syncthreads();
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < S_WAVES; ++i) t += red[i];
    return t;
}

// The first maximal element of the row; every thread gets (value, index).
__device__ __forceinline__ void block_argmax(const float* row, int V, float& best_v, int& best_i, float* redv, int* redi) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += S_THREADS) {
        const float v = row[i];
        if (v > bv) { bv = v; bi = i; }  // strict: an equal later id does not replace
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    __syncthreads();
    if (threadIdx.x % kWave == 0) { redv[threadIdx.x / kWave] = bv; redi[threadIdx.x / kWave] = bi; }
    __syncthreads();
    bv = redv[0]; bi = redi[0];
#pragma unroll
    for (int i = 1; i < S_WAVES; ++i) {
        if (redv[i] > bv || (redv[i] == bv && redi[i] < bi)) { bv = redv[i]; bi = redi[i]; }
    }
    best_v = bv;
    best_i = bi == 0x7fffffff ? 0 : bi;
}

__global__ void __launch_bounds__(S_THREADS)
sample_kernel(int* __restrict__ out, const float* __restrict__ logits, int64_t ld, int V,
              const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
              const double* __restrict__ uniform, const int* __restrict__ scatter_index, int* __restrict__ scatter_out) {
    __shared__ double redd[S_WAVES];
    __shared__ int redi[S_WAVES];
    __shared__ float redf[S_WAVES];
    __shared__ double chunk_mass[S_THREADS];
    __shared__ int chunk_ties[S_THREADS];
    __shared__ int result;

    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + static_cast<int64_t>(r) * ld;
    float lmax;
    int imax;
    block_argmax(row, V, lmax, imax, redf, redi);
    const float T = temperature != nullptr ? temperature[r] : 0.0f;
    if (!(T > 0.0f)) {
        if (tid == 0) {
            out[r] = imax;
            if (scatter_index != nullptr) scatter_out[scatter_index[r]] = imax;
        }
        return;
    }
    const float inv_t = 1.0f / T;
    int k = top_k != nullptr ? top_k[r] : 0;
    const float tp = top_p != nullptr ? top_p[r] : 1.0f;
    const bool use_k = k > 0 && k < V;
    const bool use_p = tp < 1.0f;

    // ---- top-k: the k-th largest key, and how many of its ties are kept ----
    uint32_t tau_k = 0;
    int ties_k = 0x7fffffff;
    if (use_k) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau_k | (1u << bit);
            int c = 0;
            for (int i = tid; i < V; i += S_THREADS) c += ordered_key(row[i]) >= cand;
            if (block_sum_i(c, redi) >= k) tau_k = cand;
        }
        int c = 0;
        for (int i = tid; i < V; i += S_THREADS) c += ordered_key(row[i]) > tau_k;
        ties_k = k - block_sum_i(c, redi);
    }
    // mass of {key >= tau} within the top-k set (ties at tau_k counted ties_k times)
    auto mass_ge = [&](uint32_t tau) -> double {
        double s = 0.0;
        for (int i = tid; i < V; i += S_THREADS) {
            const uint32_t key = ordered_key(row[i]);
            if (key >= tau && key > tau_k) s += static_cast<double>(expf((row[i] - lmax) * inv_t));
        }
        s = block_sum_d(s, redd);
        if (use_k && tau <= tau_k) s += static_cast<double>(ties_k) * static_cast<double>(expf((key_value(tau_k) - lmax) * inv_t));
        return s;
    };

    // ---- top-p: the key where the descending cumulative share reaches top_p ----
    uint32_t tau = tau_k;
    int ties = ties_k;
    if (use_p) {
        const double total = mass_ge(0u);
        const double target = static_cast<double>(tp) * total;
        uint32_t tau_p = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau_p | (1u << bit);
            if (mass_ge(cand) >= target) tau_p = cand;
        }
        if (tau_p < tau_k) tau_p = tau_k;
        const double above = tau_p == 0xffffffffu ? 0.0 : mass_ge(tau_p + 1u);
        int avail;
        if (use_k && tau_p == tau_k) {
            avail = ties_k;
        } else {
            int c = 0;
            for (int i = tid; i < V; i += S_THREADS) c += ordered_key(row[i]) == tau_p;
            avail = block_sum_i(c, redi);
        }
        const double p_tie = static_cast<double>(expf((key_value(tau_p) - lmax) * inv_t));
        // the prefix grows one tie at a time until its share reaches top_p
        int need = 1;
        if (p_tie > 0.0) {
            double cum = above;
            need = 0;
            while (need < avail) {
                cum += p_tie;
                ++need;
                if (cum >= target) break;
            }
            if (need < 1) need = 1;
        }
        tau = tau_p;
        ties = need < avail ? need : avail;
    }

    // ---- inverse CDF over ascending ids among the kept ----
    const int chunk = (V + S_THREADS - 1) / S_THREADS;
    const int i0 = tid * chunk, i1 = min(V, i0 + chunk);
    int my_ties = 0;
    for (int i = i0; i < i1; ++i) my_ties += ordered_key(row[i]) == tau;
    chunk_ties[tid] = my_ties;
    __syncthreads();
    int tie_rank = 0;
    for (int i = 0; i < tid; ++i) tie_rank += chunk_ties[i];
    double mine = 0.0;
    {
        int rank = tie_rank;
        for (int i = i0; i < i1; ++i) {
            const uint32_t key = ordered_key(row[i]);
            const bool kept = key > tau || (key == tau && rank++ < ties);
            if (kept) mine += static_cast<double>(expf((row[i] - lmax) * inv_t));
        }
    }
    chunk_mass[tid] = mine;
    if (tid == 0) result = -1;
    __syncthreads();
    double before = 0.0, total = 0.0;
    for (int i = 0; i < S_THREADS; ++i) {
        if (i == tid) before = total;
        total += chunk_mass[i];
    }
    double rr = uniform[r] * total - before;
    // the walk stops in the chunk where the running remainder first goes below 0
    if (rr >= 0.0 && rr - mine < 0.0) {
        int rank = tie_rank;
        for (int i = i0; i < i1; ++i) {
            const uint32_t key = ordered_key(row[i]);
            const bool kept = key > tau || (key == tau && rank++ < ties);
            if (!kept) continue;
            rr -= static_cast<double>(expf((row[i] - lmax) * inv_t));
            if (rr < 0.0) { atomicMax(&result, i); break; }
        }
    }
    __syncthreads();
    if (result < 0) {
        // floating-point slack: the last id with mass
        int rank = tie_rank, last = -1;
        for (int i = i0; i < i1; ++i) {
            const uint32_t key = ordered_key(row[i]);
            const bool kept = key > tau || (key == tau && rank++ < ties);
            if (kept && expf((row[i] - lmax) * inv_t) > 0.0f) last = i;
        }
        if (last >= 0) atomicMax(&result, last);
        __syncthreads();
    }
    if (tid == 0) {
        const int token = result < 0 ? imax : result;
        out[r] = token;
        if (scatter_index != nullptr) scatter_out[scatter_index[r]] = token;
    }
}

// Argmax in two stages so that a few rows still use many CUs: chunks of a row give partial
// (value, id) pairs, then one wave per row picks among them; ties go to the lowest id.
constexpr int AM_CHUNKS = 64;

__global__ void __launch_bounds__(256)
argmax_partial_kernel(float* __restrict__ pv, int* __restrict__ pi, const float* __restrict__ logits, int64_t ld, int V) {
    __shared__ float redv[4];
    __shared__ int redi[4];
    const int r = blockIdx.x, c = blockIdx.y;
    const int per = (V + AM_CHUNKS - 1) / AM_CHUNKS;
    const int i0 = c * per, i1 = min(V, i0 + per);
    const float* row = logits + static_cast<int64_t>(r) * ld;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = i0 + threadIdx.x; i < i1; i += 256) {
        const float v = row[i];
        if (v > bv) { bv = v; bi = i; }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (threadIdx.x % kWave == 0) { redv[threadIdx.x / kWave] = bv; redi[threadIdx.x / kWave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (redv[w] > bv || (redv[w] == bv && redi[w] < bi)) { bv = redv[w]; bi = redi[w]; }
        pv[r * AM_CHUNKS + c] = bv;
        pi[r * AM_CHUNKS + c] = bi;
    }
}

__global__ void __launch_bounds__(64)
argmax_final_kernel(int* __restrict__ out, const float* __restrict__ pv, const int* __restrict__ pi,
                    const int* __restrict__ scatter_index, int* __restrict__ scatter_out) {
    const int r = blockIdx.x;
    float bv = pv[r * AM_CHUNKS + threadIdx.x];
    int bi = pi[r * AM_CHUNKS + threadIdx.x];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, kWave);
        const int oi = __shfl_xor(bi, off, kWave);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (threadIdx.x == 0) {
        const int token = bi == 0x7fffffff ? 0 : bi;
        out[r] = token;
        if (scatter_index != nullptr) scatter_out[scatter_index[r]] = token;
    }
}

}  // namespace liyab

using namespace liyab;

// scratch_v / scratch_i: rows * 64 floats / ints of workspace. With scatter_index, row r's token
// also goes to scatter_out[scatter_index[r]] (the requests' last-token table).
extern "C" int liyab_argmax(int* out, const float* logits, int64_t ld, int rows, int V, float* scratch_v,
                            int* scratch_i, const int* scatter_index, int* scatter_out, hipStream_t stream) {
    LIYAB_REQUIRE(out && logits && scratch_v && scratch_i, "argmax: null pointer");
    LIYAB_REQUIRE(rows >= 0 && V > 0 && ld >= V, "argmax: bad sizes rows=%d V=%d", rows, V);
    LIYAB_REQUIRE(rows <= 65535 * 16, "argmax: too many rows");
    if (rows == 0) return 0;
    static_assert(AM_CHUNKS == kWave, "the final stage is one wave over the chunks");
    argmax_partial_kernel<<<dim3(rows, AM_CHUNKS), 256, 0, stream>>>(scratch_v, scratch_i, logits, ld, V);
    if (int rc = check_launch("argmax_partial")) return rc;
    argmax_final_kernel<<<rows, 64, 0, stream>>>(out, scratch_v, scratch_i, scatter_index, scatter_out);
    return check_launch("argmax_final");
}

// Per-row parameters; a row with temperature <= 0 is greedy. top_k <= 0 and
// top_p >= 1 switch those filters off. uniform[r] is in [0, 1).
extern "C" int liyab_sample(int* out, const float* logits, int64_t ld, int rows, int V, const float* temperature,
                            const int* top_k, const float* top_p, const double* uniform, const int* scatter_index,
                            int* scatter_out, hipStream_t stream) {
    LIYAB_REQUIRE(out && logits && temperature && uniform, "sample: null pointer");
    LIYAB_REQUIRE(rows >= 0 && V > 0 && ld >= V, "sample: bad sizes rows=%d V=%d", rows, V);
    if (rows == 0) return 0;
    LIYAB_REQUIRE(scatter_index == nullptr || scatter_out != nullptr, "sample: a scatter index needs a target");
    sample_kernel<<<rows, S_THREADS, 0, stream>>>(out, logits, ld, V, temperature, top_k, top_p, uniform, scatter_index, scatter_out);
    return check_launch("sample");
}
