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
#include "no_alloc.h"

#include <mutex>

namespace liyab {

constexpr int S_THREADS = 1024;
constexpr int S_WAVES = S_THREADS / kWave;

// Unsigned keys in the order of the floats. -0 becomes +0 first (x + 0 does that and nothing
// else), so that the two zeros are one value with one key, ties like any others.
__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t u = __float_as_uint(f + 0.0f);
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
    wave_argmax(bv, bi);
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

// The same rules with the row held in registers, for vocabularies up to THREADS * EPT entries
// (1024 threads up to 16 ids each, 512 threads up to 128: the registers of a wave must hold
// them). Wave w owns the ids [w * 64 * chunk, (w + 1) * 64 * chunk); within it lane l holds
// groups of 4 consecutive ids, its g-th group starting at (g * 64 + l) * 4, so the order of
// ids within a wave is (group, lane, place in the group). The row is read once; the
// bisections for the k-th largest key and for the top-p threshold then cost compares on
// registers instead of passes over memory. With top-k of at most 64 (the usual case) the
// kept logits are gathered into LDS and one wave finishes: nucleus cut and draw among at most
// 64 candidates. Masses are fixed-point integers, exp((l - l_max) / T) * 2^44 rounded down, so
// that every sum is exact and independent of the order of the additions; a probability below
// 2^-44 of the largest counts as none.
constexpr int kMassBits = 44;
constexpr int kWaveCandidates = 64;
constexpr int kPoolMax = 1024;  // keys that may be among the k largest, for one wave to choose from (half of them on 1,024 threads, whose waves have half the registers)
// Top-p over many candidates: masses are first added up in bins by the logit's distance below
// the largest, kBins of them over the 44 powers of two that a mass can lie under the largest
// (a bin is a monotone function of the key, so the bins are intervals of the descending order).
constexpr int kBins = 2048;
constexpr int kBinPad = 32;  // one word of padding every 32 bins: a lane's 32 bins in a row, the lanes' on different banks
__device__ __forceinline__ int bin_slot(int b) { return b + b / kBinPad; }

__device__ __forceinline__ unsigned long long fixed_mass(uint32_t key, float lmax, float scale2) {
    // exp((l - l_max) / T) through the hardware's 2^x (scale2 = log2(e) / T), in [0, 1]; times
    // 2^44 (exact), then split into the words of a 64-bit integer: the part above 2^32 has at
    // most 13 bits, so its product with 2^32 and the remainder are exact in 32-bit floats
    const float x = __builtin_amdgcn_exp2f((key_value(key) - lmax) * scale2) * static_cast<float>(1ull << kMassBits);
    const uint32_t hi = static_cast<uint32_t>(x * (1.0f / 4294967296.0f));
    const uint32_t lo = static_cast<uint32_t>(fmaf(-static_cast<float>(hi), 4294967296.0f, x));
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// The same value, opaque to the compiler: what is computed from it is computed again instead of
// being kept in registers from an earlier pass over the row (two more registers per id held).
__device__ __forceinline__ uint32_t again(uint32_t key) {
    asm volatile("" : "+v"(key));
    return key;
}

__device__ __forceinline__ unsigned long long shfl_up_u64(unsigned long long v, int delta) {
    const uint32_t lo = __shfl_up(static_cast<uint32_t>(v), delta, kWave);
    const uint32_t hi = __shfl_up(static_cast<uint32_t>(v >> 32), delta, kWave);
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}
__device__ __forceinline__ unsigned long long shfl_u64(unsigned long long v, int src) {
    const uint32_t lo = __shfl(static_cast<uint32_t>(v), src, kWave);
    const uint32_t hi = __shfl(static_cast<uint32_t>(v >> 32), src, kWave);
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}
// Lane `src`'s value for every lane, `src` being the same for the whole wave: a register read,
// where an exchange through the lanes' crossbar would take a hundred cycles to come back.
__device__ __forceinline__ uint32_t lane_value(uint32_t v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ int lane_value(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ unsigned long long lane_value64(unsigned long long v, int src) {
    const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), src);
    const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), src);
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}
__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
    // within rows of 16 lanes through DPP, the rows' sums as scalars (integer sums: any order gives the same)
    auto step = [&](auto ctrl) {
        constexpr int CTRL = decltype(ctrl)::value;
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(v)), CTRL, 0xf, 0xf, false));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(static_cast<uint32_t>(v >> 32)), CTRL, 0xf, 0xf, false));
        v += (static_cast<unsigned long long>(hi) << 32) | lo;
    };
    step(std::integral_constant<int, 0xB1>{});
    step(std::integral_constant<int, 0x4E>{});
    step(std::integral_constant<int, 0x141>{});
    step(std::integral_constant<int, 0x140>{});
    return (lane_value64(v, 0) + lane_value64(v, 16)) + (lane_value64(v, 32) + lane_value64(v, 48));
}

// Sums over a workgroup of WAVES waves, exact; every thread gets the result. `red`: WAVES values.
template <int WAVES>
__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* red) {
    v = wave_sum_u64(v);
    __syncthreads();
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    unsigned long long t = 0;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) t += red[i];
    return t;
}
template <int WAVES>
__device__ __forceinline__ int block_count(int v, int* red) {
    v = wave_sum_i(v);
    __syncthreads();
    if (threadIdx.x % kWave == 0) red[threadIdx.x / kWave] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) t += red[i];
    return t;
}

// PLAIN: no row asks for top-k or top-p (the caller's word): every logit is kept, and what serves
// the cuts is not compiled in, which leaves the registers to the row (what serves the cuts costs registers,
// and time in every pass over the keys a thread holds).
template <int EPT, int THREADS, bool PLAIN>
__global__ void __launch_bounds__(THREADS)
sample_registers_kernel(int* __restrict__ out, const float* __restrict__ logits, int64_t ld, int V,
                        const float* __restrict__ temperature, const int* __restrict__ top_k, const float* __restrict__ top_p,
                        const double* __restrict__ uniform, const int* __restrict__ scatter_index, int* __restrict__ scatter_out) {
    static_assert(EPT % 4 == 0, "ids are held in groups of 4");
    constexpr int WAVES = THREADS / kWave, GROUPS = EPT / 4;
    __shared__ unsigned long long red64[WAVES];
    __shared__ uint32_t redk[WAVES];
    __shared__ int redi[WAVES];
    __shared__ int result, n_cand;
    __shared__ uint32_t cand_key[kWaveCandidates];
    __shared__ int cand_id[kWaveCandidates];
    // top-k of at most 64: the threads' largest keys, and the pool of keys that may be among the k largest
    __shared__ uint32_t thread_max[THREADS];
    constexpr int kPool = THREADS >= 1024 ? kPoolMax / 2 : kPoolMax;
    __shared__ uint32_t pool_key[kPool];
    __shared__ int pool_id[kPool];
    __shared__ int n_pool;
    __shared__ uint32_t pool_floor;
    // top-p over many candidates: the bins' masses, and what one wave finds for all
    __shared__ unsigned long long bin_mass[PLAIN ? 1 : kBins + kBins / kBinPad];
    __shared__ unsigned long long bins_above;
    __shared__ double bins_target;
    __shared__ int bin_star, bins_ok, found_ties;
    __shared__ uint32_t found_tau;

    const int r = blockIdx.x, tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
    const float* row = logits + static_cast<int64_t>(r) * ld;
    // A thread's groups of 4 ids are read as 16 bytes each, so the groups start at addresses that
    // are multiples of 16: the ids are counted from `shift` entries before the row (a row of an odd
    // width starts anywhere), and an id before the row is no element.
    const int shift = static_cast<int>((reinterpret_cast<uintptr_t>(row) >> 2) & 3u);
    const int chunk = (((V + shift + THREADS - 1) / THREADS + 3) / 4) * 4;  // ids a thread, <= EPT (the launcher's check)
    const int span0 = wave * kWave * chunk - shift;
    auto id_of = [&](int j) { return span0 + ((j / 4) * kWave + lane) * 4 + j % 4; };
    // keys of this thread's ids; 0 stands for "no element" (no real logit has that key)
    uint32_t keys[EPT];
    // every load from a valid address (a group past the row reads the row's last group), so that no
    // condition has to live while the loads are in flight; what is outside the row is dropped after.
    // The first and the last group may reach up to 12 bytes outside the row, within its aligned 16.
    {
        typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
        const int last_group = ((V - 1 + shift) / 4) * 4 - shift;  // first id of the group that holds the row's last entry
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(row + min(id_of(4 * g), last_group));
#pragma unroll
            for (int e = 0; e < 4; ++e) keys[4 * g + e] = v[e];
        }
    }
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        const uint32_t raw = again(keys[j]);
        keys[j] = (j < chunk && id_of(j) >= 0 && id_of(j) < V) ? ordered_key(__uint_as_float(raw)) : 0u;
    }
    // the largest key and its lowest id
    uint32_t kmax = 0;
    int imax = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < EPT; ++j)
        if (keys[j] > kmax) { kmax = keys[j]; imax = id_of(j); }
    thread_max[tid] = kmax;
    wave_argmax(kmax, imax);
    if (lane == 0) { redk[wave] = kmax; redi[wave] = imax; }
    if (tid == 0) { result = -1; n_cand = 0; n_pool = 0; }
    __syncthreads();
    kmax = redk[0]; imax = redi[0];
#pragma unroll
    for (int i = 1; i < WAVES; ++i)
        if (redk[i] > kmax || (redk[i] == kmax && redi[i] < imax)) { kmax = redk[i]; imax = redi[i]; }
    if (imax == 0x7fffffff) imax = 0;
    const float T = temperature != nullptr ? temperature[r] : 0.0f;
    if (!(T > 0.0f)) {
        if (tid == 0) {
            out[r] = imax;
            if (scatter_index != nullptr) scatter_out[scatter_index[r]] = imax;
        }
        return;
    }
    const float lmax = key_value(kmax), inv_t = 1.4426950408889634f / T;  // exponentials are taken in base 2
    const int k = top_k != nullptr ? top_k[r] : 0;
    const float tp = top_p != nullptr ? top_p[r] : 1.0f;
    const bool use_k = !PLAIN && k > 0 && k < V, use_p = !PLAIN && tp < 1.0f;
    const unsigned long long lanes_below = (1ull << lane) - 1ull;

    // Which of this thread's ids are kept, as bits: key > t, or key == t and among the first
    // `ties` of the ids with that key (ascending ids: waves in order, within a wave groups, lanes,
    // places). When every tie is kept no ranks are needed.
    auto kept_bits = [&](uint32_t t, int ties, uint32_t (&bits)[(EPT + 31) / 32]) {
        int n_ties = 0;
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            // (compared afresh: the same comparisons come again in the ranks below, and kept from here to
            // there they are a lane mask an id, more scalar registers than there are)
            const uint32_t key = again(keys[j]);
            n_ties += key == t && key != 0u;
        }
        const int all_ties = block_count<WAVES>(n_ties, redi);
#pragma unroll
        for (int w = 0; w < (EPT + 31) / 32; ++w) bits[w] = 0u;
        if (ties >= all_ties) {
#pragma unroll
            for (int j = 0; j < EPT; ++j)
                if (keys[j] != 0u && keys[j] >= t) bits[j / 32] |= 1u << (j % 32);
            return;
        }
        const int in_wave = wave_sum_i(n_ties);
        __syncthreads();
        if (lane == 0) redi[wave] = in_wave;
        __syncthreads();
        int rank = 0;  // ties before this wave, then before the group at hand
        for (int w = 0; w < wave; ++w) rank += redi[w];
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            unsigned long long tied[4];
            int below = 0, in_group = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                tied[e] = __ballot(keys[4 * g + e] == t && keys[4 * g + e] != 0u);
                below += __popcll(tied[e] & lanes_below);
                in_group += __popcll(tied[e]);
            }
            int mine = rank + below;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t key = keys[4 * g + e];
                const bool tie = key == t && key != 0u;
                if (key > t || (tie && mine < ties)) bits[(4 * g + e) / 32] |= 1u << ((4 * g + e) % 32);
                mine += tie;
            }
            rank += in_group;
        }
    };

    uint32_t bits[(EPT + 31) / 32];
    // is id j of this thread kept? (PLAIN: every element of the row is)
    // (the word of bits is read afresh each time, for the same reason: no lane mask an id is kept between the passes)
    auto is_kept = [&](int j) { return PLAIN ? again(keys[j]) != 0u : ((again(bits[j / 32]) >> (j % 32)) & 1u) != 0u; };
    if constexpr (!PLAIN) {
    // ---- one wave among at most 64 candidates in cand_key / cand_id: nucleus cut and draw ----
    auto wave_finish = [&]() {
        const int n = n_cand;  // = k
        const bool has = lane < n;
        const uint32_t key = has ? cand_key[lane] : 0u;
        const int id = has ? cand_id[lane] : 0x7fffffff;
        const unsigned long long q = has ? fixed_mass(key, lmax, inv_t) : 0ull;
        // place in the descending order of keys (ties by ascending id) and in the ascending order of ids
        int desc = 0, asc = 0;
        for (int o = 0; o < n; ++o) {
            const uint32_t ok = lane_value(key, o);
            const int oi = lane_value(id, o);
            desc += ok > key || (ok == key && oi < id);
            asc += oi < id;
        }
        bool kept = has;
        if (use_p) {
            // cum = mass of the candidates before this one in descending order, itself included
            unsigned long long cum = 0, total = 0;
            for (int o = 0; o < n; ++o) {
                const unsigned long long oq = lane_value64(q, o);
                const int od = lane_value(desc, o);
                total += oq;
                if (od <= desc) cum += oq;
            }
            const double target = static_cast<double>(tp) * static_cast<double>(total);
            // the shortest prefix whose mass reaches the target: an element is kept when the prefix
            // before it has not reached it yet; the first is always kept
            kept = has && (desc == 0 || static_cast<double>(cum - q) < target);
        }
        const unsigned long long mass = kept ? q : 0ull;
        unsigned long long before = 0, total = 0;
        for (int o = 0; o < n; ++o) {
            const unsigned long long om = lane_value64(mass, o);
            const int oa = lane_value(asc, o);
            total += om;
            if (oa < asc) before += om;
        }
        int token = imax;
        if (total > 0ull) {
            unsigned long long rr = static_cast<unsigned long long>(uniform[r] * static_cast<double>(total));
            if (rr >= total) rr = total - 1;
            const bool mine = kept && rr >= before && rr - before < mass;
            const unsigned long long pick = __ballot(mine);
            if (pick != 0ull) token = __shfl(id, __ffsll(static_cast<long long>(pick)) - 1, kWave);
        }
        if (lane == 0) {
            out[r] = token;
            if (scatter_index != nullptr) scatter_out[scatter_index[r]] = token;
        }
    };

    // ---- top-k of at most 64 (the usual case) without passes of the whole workgroup over the row ----
    // The k-th largest of the threads' largest keys is a floor for the k-th largest key of the
    // row (k keys reach it): one wave finds it among THREADS values; every thread then puts its
    // keys from that floor up into a pool (about k of them, unless many keys are equal); one wave
    // finds the k-th largest of the pool exactly, keeps ties by ascending id, and finishes. A pool
    // that overflows falls through to the bisection over the whole row below.
    if (use_k && k <= kWaveCandidates) {
        if (wave == 0) {
            constexpr int PER = THREADS / kWave;
            uint32_t mine[PER];
#pragma unroll
            for (int i = 0; i < PER; ++i) mine[i] = thread_max[lane + kWave * i];
            uint32_t floor_key = 0;
            for (int bit = 31; bit >= 0; --bit) {
                const uint32_t cand = floor_key | (1u << bit);
                int c = 0;  // counted through the lanes' votes: sums across lanes would cost six dependent exchanges a bit
#pragma unroll
                for (int i = 0; i < PER; ++i) c += __popcll(__ballot(mine[i] >= cand));
                if (c >= k) floor_key = cand;
            }
            if (lane == 0) pool_floor = floor_key;
        }
        __syncthreads();
        const uint32_t floor_key = pool_floor;
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            if (keys[j] != 0u && keys[j] >= floor_key) {
                const int at = atomicAdd(&n_pool, 1);  // the order of arrival does not matter: ranks below are by key and id
                if (at < kPool) {
                    pool_key[at] = keys[j];
                    pool_id[at] = id_of(j);
                }
            }
        }
        __syncthreads();
        const int n = n_pool;
        if (n <= kPool) {
            if (wave == 0) {
                constexpr int PER = kPool / kWave;
                uint32_t pk[PER];
                int pid[PER];
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const int e = lane + kWave * i;
                    pk[i] = e < n ? pool_key[e] : 0u;
                    pid[i] = e < n ? pool_id[e] : 0x7fffffff;
                }
                uint32_t tau = 0;
                for (int bit = 31; bit >= 0; --bit) {
                    const uint32_t cand = tau | (1u << bit);
                    int c = 0;
#pragma unroll
                    for (int i = 0; i < PER; ++i) c += __popcll(__ballot(pk[i] >= cand));
                    if (c >= k) tau = cand;
                }
                int above = 0, tied = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    above += __popcll(__ballot(pk[i] > tau));
                    tied += __popcll(__ballot(pk[i] == tau && pk[i] != 0u));
                }
                const int ties = k - above;  // ties at tau that are kept: those of the lowest ids
                int base = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    bool keep = pk[i] != 0u && pk[i] >= tau;
                    if (ties < tied && pk[i] == tau && pk[i] != 0u) {
                        int rank = 0;  // ties of a lower id
                        for (int o = 0; o < n; ++o) rank += pool_key[o] == tau && pool_id[o] < pid[i];
                        keep = rank < ties;
                    }
                    const unsigned long long kept_lanes = __ballot(keep);
                    if (keep) {
                        const int at = base + __popcll(kept_lanes & lanes_below);
                        cand_key[at] = pk[i];
                        cand_id[at] = pid[i];
                    }
                    base += __popcll(kept_lanes);
                }
                if (lane == 0) n_cand = base;
            }
            __syncthreads();
            if (wave == 0) wave_finish();
            return;
        }
    }

    // ---- top-k: the k-th largest key, and how many of its ties are kept ----
    uint32_t tau_k = 0;
    int ties_k = 0x7fffffff;
    // the bin of a key: its logit's distance under the largest, in kBins steps over the kMassBits powers
    // of two that a mass can lie under the largest one's (a monotone function of the key)
    auto bin_of = [&](uint32_t key) {
        const float below = (lmax - key_value(key)) * inv_t;  // powers of two under the largest mass, >= 0
        return static_cast<int>(fminf(below * (static_cast<float>(kBins) / kMassBits), static_cast<float>(kBins - 1)));
    };
    bool k_found = false;
    if (use_k) {
        // by bins, as top-p below: the keys are counted in bins, one wave finds the bin that holds the
        // k-th largest, that bin's keys alone are gathered, and the wave picks among them. A bin with
        // more keys than the pool leaves it to the counting passes over the whole row.
        uint32_t* bin_count = reinterpret_cast<uint32_t*>(bin_mass);
        __syncthreads();
        for (int i = tid; i < kBins + kBins / kBinPad; i += THREADS) bin_count[i] = 0u;
        if (tid == 0) { bins_ok = 0; n_pool = 0; }
        __syncthreads();
        // (the last bin takes every key from 2^-44 of the largest mass down, often most of the row: those are
        // counted in a register and added once a wave, not one atomic each on the same word)
        int last_bin = 0;
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            const uint32_t key = again(keys[j]);
            if (key != 0u) {
                const int b = bin_of(key);
                if (b == kBins - 1) ++last_bin;
                else atomicAdd(&bin_count[bin_slot(b)], 1u);
            }
        }
        last_bin = wave_sum_i(last_bin);
        if (lane == 0 && last_bin != 0) atomicAdd(&bin_count[bin_slot(kBins - 1)], static_cast<uint32_t>(last_bin));
        __syncthreads();
        if (wave == 0) {
            constexpr int PER_LANE = kBins / kWave;
            int mine_sum = 0;
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) mine_sum += static_cast<int>(bin_count[bin_slot(lane * PER_LANE + i)]);
            int incl = mine_sum;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                const int o = __shfl_up(incl, d, kWave);
                if (lane >= d) incl += o;
            }
            const unsigned long long reached = __ballot(incl >= k);
            if (reached != 0ull && lane == __ffsll(static_cast<long long>(reached)) - 1) {
                int cum = incl - mine_sum;
                for (int i = 0; i < PER_LANE; ++i) {
                    const int next = cum + static_cast<int>(bin_count[bin_slot(lane * PER_LANE + i)]);
                    if (next >= k) {
                        bin_star = lane * PER_LANE + i;
                        bins_above = static_cast<unsigned long long>(cum);
                        bins_ok = 1;
                        break;
                    }
                    cum = next;
                }
            }
        }
        __syncthreads();
        if (bins_ok != 0) {
            const int star = bin_star;
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const uint32_t key = again(keys[j]);
                if (key != 0u && bin_of(key) == star) {
                    const int at = atomicAdd(&n_pool, 1);  // the order of arrival does not matter: only keys count here
                    if (at < kPool) pool_key[at] = key;
                }
            }
            __syncthreads();
            const int n = n_pool;
            if (n <= kPool) {
                if (wave == 0) {
                    constexpr int PER = kPool / kWave;
                    const int want = k - static_cast<int>(bins_above);  // the k-th largest of the row is the want-th largest of this bin
                    uint32_t pk[PER];
                    uint32_t lo = 0xffffffffu, hi = 0u;
#pragma unroll
                    for (int i = 0; i < PER; ++i) {
                        const int e = lane + kWave * i;
                        pk[i] = e < n ? pool_key[e] : 0u;
                        if (e < n) { lo = min(lo, pk[i]); hi = max(hi, pk[i]); }
                    }
#pragma unroll
                    for (int off = kWave / 2; off > 0; off >>= 1) {
                        lo = min(lo, static_cast<uint32_t>(__shfl_xor(static_cast<int>(lo), off, kWave)));
                        hi = max(hi, static_cast<uint32_t>(__shfl_xor(static_cast<int>(hi), off, kWave)));
                    }
                    const int open_bits = lo == hi ? 0 : 32 - __clz(lo ^ hi);
                    uint32_t t = open_bits >= 32 ? 0u : (hi >> open_bits) << open_bits;
                    for (int bit = open_bits - 1; bit >= 0; --bit) {
                        const uint32_t cand = t | (1u << bit);
                        int c = 0;
#pragma unroll
                        for (int i = 0; i < PER; ++i)
                            if (i * kWave < n) c += __popcll(__ballot(pk[i] >= cand));
                        if (c >= want) t = cand;
                    }
                    int above = 0;
#pragma unroll
                    for (int i = 0; i < PER; ++i)
                        if (i * kWave < n) above += __popcll(__ballot(pk[i] > t));
                    if (lane == 0) {
                        found_tau = t;
                        found_ties = want - above;
                    }
                }
                __syncthreads();
                tau_k = found_tau;
                ties_k = found_ties;
                k_found = true;
            }
        }
        __syncthreads();
        if (tid == 0) n_pool = 0;  // (the pool serves top-p next)
        __syncthreads();
    }
    if (use_k && !k_found) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau_k | (1u << bit);
            int c = 0;
#pragma unroll
            for (int j = 0; j < EPT; ++j) c += keys[j] >= cand;
            if (block_count<WAVES>(c, redi) >= k) tau_k = cand;
        }
        int c = 0;
#pragma unroll
        for (int j = 0; j < EPT; ++j) c += keys[j] > tau_k;
        ties_k = k - block_count<WAVES>(c, redi);
    }

    if (use_k && k <= kWaveCandidates) {
        // ---- few candidates (the pool overflowed): gathered, then one wave does the rest ----
        kept_bits(tau_k, ties_k, bits);
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            if (bits[j / 32] >> (j % 32) & 1u) {
                const int at = atomicAdd(&n_cand, 1);  // the order of arrival does not matter: ranks below are by key and id
                cand_key[at] = keys[j];
                cand_id[at] = id_of(j);
            }
        }
        __syncthreads();
        if (wave == 0) wave_finish();
        return;
    }

    // ---- top-p over many candidates: the key where the descending cumulative mass reaches top_p ----
    uint32_t tau = tau_k;
    int ties = ties_k;
    bool cut_found = false;
    if (use_p) {
        // ---- by bins: one pass adds the masses up in bins, one wave finds the bin in which the
        // descending cumulative mass reaches top_p, the keys of that bin alone are gathered, and the
        // same wave finds the key among them. The sums are integers, so the bins' total and every
        // prefix are the sums the bisection below would find, and so are the key and the ties kept.
        // A bin with more keys than the pool holds (thousands of nearly equal logits), or nothing
        // to cut, leaves it to the bisection.
        const unsigned long long tie_mass = use_k ? static_cast<unsigned long long>(ties_k) * fixed_mass(tau_k, lmax, inv_t) : 0ull;
        for (int i = tid; i < kBins + kBins / kBinPad; i += THREADS) bin_mass[i] = 0ull;
        if (tid == 0) bins_ok = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < EPT; ++j) {
            const uint32_t key = again(keys[j]);
            if (key != 0u && key > tau_k) {
                const unsigned long long m = fixed_mass(key, lmax, inv_t);
                if (m != 0ull) atomicAdd(&bin_mass[bin_slot(bin_of(key))], m);
            }
        }
        if (tid == 0 && tie_mass != 0ull) atomicAdd(&bin_mass[bin_slot(bin_of(tau_k))], tie_mass);
        __syncthreads();
        if (wave == 0) {
            constexpr int PER_LANE = kBins / kWave;
            unsigned long long mine_sum = 0;
#pragma unroll
            for (int i = 0; i < PER_LANE; ++i) mine_sum += bin_mass[bin_slot(lane * PER_LANE + i)];
            unsigned long long incl = mine_sum;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                const unsigned long long o = shfl_up_u64(incl, d);
                if (lane >= d) incl += o;
            }
            const unsigned long long total = lane_value64(incl, kWave - 1);
            const double target = static_cast<double>(tp) * static_cast<double>(total);
            const unsigned long long reached = __ballot(static_cast<double>(incl) >= target);
            if (total > 0ull && target > 0.0 && reached != 0ull && lane == __ffsll(static_cast<long long>(reached)) - 1) {
                unsigned long long cum = incl - mine_sum;
                for (int i = 0; i < PER_LANE; ++i) {
                    const unsigned long long next = cum + bin_mass[bin_slot(lane * PER_LANE + i)];
                    if (static_cast<double>(next) >= target) {
                        bin_star = lane * PER_LANE + i;
                        bins_above = cum;
                        bins_target = target;
                        bins_ok = 1;
                        break;
                    }
                    cum = next;
                }
            }
        }
        __syncthreads();
        if (bins_ok != 0) {
            const int star = bin_star;
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const uint32_t key = again(keys[j]);
                if (key != 0u && key > tau_k && bin_of(key) == star) {
                    const int at = atomicAdd(&n_pool, 1);  // the order of arrival does not matter: only keys count here
                    if (at < kPool) pool_key[at] = key;
                }
            }
            __syncthreads();
            const int n = n_pool;
            if (n <= kPool) {
                if (wave == 0) {
                    constexpr int PER = kPool / kWave;
                    const bool k_here = tie_mass != 0ull && bin_of(tau_k) == star;  // the top-k ties lie in this bin
                    const unsigned long long k_mass = k_here ? tie_mass : 0ull;
                    uint32_t pk[PER];  // (their masses are taken again wherever they are needed: registers are short here)
                    auto pm = [&](int i) { return pk[i] != 0u ? fixed_mass(again(pk[i]), lmax, inv_t) : 0ull; };
                    uint32_t lo = k_here ? tau_k : 0xffffffffu, hi = k_here ? tau_k : 0u;
#pragma unroll
                    for (int i = 0; i < PER; ++i) {
                        const int e = lane + kWave * i;
                        pk[i] = e < n ? pool_key[e] : 0u;
                        if (e < n) { lo = min(lo, pk[i]); hi = max(hi, pk[i]); }
                    }
#pragma unroll
                    for (int off = kWave / 2; off > 0; off >>= 1) {
                        lo = min(lo, static_cast<uint32_t>(__shfl_xor(static_cast<int>(lo), off, kWave)));
                        hi = max(hi, static_cast<uint32_t>(__shfl_xor(static_cast<int>(hi), off, kWave)));
                    }
                    const unsigned long long above_bin = bins_above;
                    const double target = bins_target;
                    // the largest key whose mass from it upwards reaches the target: it lies in this bin,
                    // so only the bits in which the bin's keys differ are open
                    const int open_bits = lo == hi ? 0 : 32 - __clz(lo ^ hi);
                    uint32_t tau_p = open_bits >= 32 ? 0u : (hi >> open_bits) << open_bits;
                    for (int bit = open_bits - 1; bit >= 0; --bit) {
                        const uint32_t cand = tau_p | (1u << bit);
                        unsigned long long m = 0;
#pragma unroll
                        for (int i = 0; i < PER; ++i)
                            if (i * kWave < n) m += pk[i] >= cand ? pm(i) : 0ull;  // (the same for the whole wave: a bin mostly holds far fewer keys than the pool)
                        m = wave_sum_u64(m) + (k_here && tau_k >= cand ? k_mass : 0ull) + above_bin;
                        if (static_cast<double>(m) >= target) tau_p = cand;
                    }
                    unsigned long long above = 0;
                    int avail = 0;
#pragma unroll
                    for (int i = 0; i < PER; ++i) {
                        if (i * kWave < n) {
                            above += pk[i] > tau_p ? pm(i) : 0ull;
                            avail += __popcll(__ballot(pk[i] == tau_p && pk[i] != 0u));
                        }
                    }
                    above = wave_sum_u64(above) + above_bin;
                    if (k_here && tau_p == tau_k) avail = ties_k;
                    // the prefix grows one tie at a time until its share reaches top_p
                    const unsigned long long p_tie = fixed_mass(tau_p, lmax, inv_t);
                    int need = 1;
                    if (p_tie > 0ull) {
                        unsigned long long cum = above;
                        need = 0;
                        while (need < avail) {
                            cum += p_tie;
                            ++need;
                            if (static_cast<double>(cum) >= target) break;
                        }
                        if (need < 1) need = 1;
                    }
                    if (lane == 0) {
                        found_tau = tau_p;
                        found_ties = need < avail ? need : avail;
                    }
                }
                __syncthreads();
                tau = found_tau;
                ties = found_ties;
                cut_found = true;
            }
        }
    }
    if (use_p && !cut_found) {
        const unsigned long long tie_mass_k = use_k ? static_cast<unsigned long long>(ties_k) * fixed_mass(tau_k, lmax, inv_t) : 0ull;
        // mass of {key >= cand} within the top-k set (ties at tau_k counted ties_k times)
        auto mass_ge = [&](uint32_t cand) -> unsigned long long {
            unsigned long long m = 0;
#pragma unroll
            for (int j = 0; j < EPT; ++j) {
                const uint32_t key = again(keys[j]);
                if (key >= cand && key > tau_k) m += fixed_mass(key, lmax, inv_t);
            }
            m = block_sum_u64<WAVES>(m, red64);
            return (use_k && cand <= tau_k) ? m + tie_mass_k : m;
        };
        const double target = static_cast<double>(tp) * static_cast<double>(mass_ge(0u));
        uint32_t tau_p = 0;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau_p | (1u << bit);
            if (static_cast<double>(mass_ge(cand)) >= target) tau_p = cand;
        }
        if (tau_p < tau_k) tau_p = tau_k;
        const unsigned long long above = tau_p == 0xffffffffu ? 0ull : mass_ge(tau_p + 1u);
        int avail;
        if (use_k && tau_p == tau_k) {
            avail = ties_k;
        } else {
            int c = 0;
#pragma unroll
            for (int j = 0; j < EPT; ++j) c += keys[j] == tau_p;
            avail = block_count<WAVES>(c, redi);
        }
        // the prefix grows one tie at a time until its share reaches top_p
        const unsigned long long p_tie = fixed_mass(tau_p, lmax, inv_t);
        int need = 1;
        if (p_tie > 0ull) {
            unsigned long long cum = above;
            need = 0;
            while (need < avail) {
                cum += p_tie;
                ++need;
                if (static_cast<double>(cum) >= target) break;
            }
            if (need < 1) need = 1;
        }
        tau = tau_p;
        ties = need < avail ? need : avail;
    }

        kept_bits(tau, ties, bits);
    }

    // ---- inverse CDF over ascending ids among the kept ----
    unsigned long long mine = 0;
#pragma unroll
    for (int j = 0; j < EPT; ++j)
        if (is_kept(j)) mine += fixed_mass(again(keys[j]), lmax, inv_t);
    // the wave where the walk ends, from the waves' masses in order; then that wave alone walks
    // its ids in their order: group by group, a scan over the lanes' four ids each
    const unsigned long long wave_mass = wave_sum_u64(mine);
    __syncthreads();
    if (lane == 0) red64[wave] = wave_mass;
    __syncthreads();
    unsigned long long total = 0, before = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
        if (w < wave) before += red64[w];
        total += red64[w];
    }
    if (total > 0ull) {
        unsigned long long rr = static_cast<unsigned long long>(uniform[r] * static_cast<double>(total));
        if (rr >= total) rr = total - 1;
        if (rr >= before && rr - before < wave_mass) {  // wave-uniform
            unsigned long long left = rr - before;
            // The group where the walk ends, from the groups' masses in order. The sums over the
            // lanes are taken for 8 groups at a time, their exchanges interleaved: one after the
            // other (a scan per group, each waiting for the one before) they cost 16 us a row.
            int gstar = -1;
#pragma unroll
            for (int g0 = 0; g0 < GROUPS; g0 += 8) {
                unsigned long long tot[8];
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    tot[b] = 0ull;
                    if (g0 + b < GROUPS) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int j = 4 * (g0 + b) + e;
                            if (is_kept(j)) tot[b] += fixed_mass(again(keys[j]), lmax, inv_t);
                        }
                    }
                }
#pragma unroll
                for (int off = kWave / 2; off > 0; off >>= 1) {
#pragma unroll
                    for (int b = 0; b < 8; ++b) {
                        if (g0 + b < GROUPS) {
                            const uint32_t lo = __shfl_xor(static_cast<uint32_t>(tot[b]), off, kWave);
                            const uint32_t hi = __shfl_xor(static_cast<uint32_t>(tot[b] >> 32), off, kWave);
                            tot[b] += (static_cast<unsigned long long>(hi) << 32) | lo;
                        }
                    }
                }
#pragma unroll
                for (int b = 0; b < 8; ++b) {
                    if (g0 + b < GROUPS && gstar < 0) {
                        if (left < tot[b]) gstar = g0 + b;
                        else left -= tot[b];
                    }
                }
            }
            // within that group: a scan over the lanes' four ids each
            int found = -1;
#pragma unroll
            for (int g = 0; g < GROUPS; ++g) {
                if (g != gstar) continue;  // the same for the whole wave
                unsigned long long q[4], q4 = 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int j = 4 * g + e;
                    q[e] = is_kept(j) ? fixed_mass(again(keys[j]), lmax, inv_t) : 0ull;
                    q4 += q[e];
                }
                unsigned long long inc = q4;
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1) {
                    const unsigned long long o = shfl_up_u64(inc, d);
                    if (lane >= d) inc += o;
                }
                const unsigned long long pick = __ballot(q4 > 0ull && left >= inc - q4 && left < inc);
                if (pick != 0ull) {
                    const int src = __ffsll(static_cast<long long>(pick)) - 1;
                    // within the lane's four ids
                    unsigned long long rest = left - (inc - q4);
                    int e_pick = 3;
#pragma unroll
                    for (int e = 3; e >= 0; --e) {
                        unsigned long long upto = 0;
#pragma unroll
                        for (int e2 = 0; e2 <= e; ++e2) upto += q[e2];
                        if (q[e] > 0ull && rest < upto) e_pick = e;
                    }
                    found = __shfl(id_of(4 * g) + e_pick, src, kWave);
                }
            }
            if (lane == 0) result = found;
        }
    }
    __syncthreads();
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
    wave_argmax(bv, bi);
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
    wave_argmax(bv, bi);
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

// The scratch of liyab_argmax_static: 64 values, then 64 ids, for each of up to
// LIYAB_ARGMAX_STATIC_MAX_ROWS rows. In host code this name is a stand-in for the symbol, not a
// device address: the address is asked for once a device (each GPU holds its own copy) and only
// that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[LIYAB_ARGMAX_STATIC_MAX_ROWS * AM_CHUNKS * (sizeof(float) + sizeof(int))];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};  // the array's address on each device, once looked up

// The array's address on the current device (nullptr after fail(...)).
void* scratch_of_current_device() {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { fail(2, "argmax_static: hipGetDevice: %s", hipGetErrorString(e)); return nullptr; }
    if (dev < 0 || dev >= kMaxDevices) { fail(1, "argmax_static: device %d is beyond the %d this library keeps track of", dev, kMaxDevices); return nullptr; }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            fail(2, "argmax_static: hipGetSymbolAddress on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int liyab_argmax_static_init(void) { return scratch_of_current_device() != nullptr ? 0 : 2; }

extern "C" int liyab_argmax_static(int* out, const float* logits, int64_t ld, int rows, int V, const int* scatter_index,
                                   int* scatter_out, hipStream_t stream) {
    LIYAB_REQUIRE(out && logits, "argmax_static: null pointer");
    LIYAB_REQUIRE(rows >= 0 && V > 0 && ld >= V, "argmax_static: bad sizes rows=%d V=%d", rows, V);
    LIYAB_REQUIRE(rows <= LIYAB_ARGMAX_STATIC_MAX_ROWS, "argmax_static: %d rows; the library's own scratch holds %d (use liyab_argmax with a workspace beyond)",
                  rows, LIYAB_ARGMAX_STATIC_MAX_ROWS);
    LIYAB_REQUIRE(scatter_index == nullptr || scatter_out != nullptr, "argmax_static: a scatter index needs a target");
    if (rows == 0) return 0;
    void* ptr = scratch_of_current_device();
    if (ptr == nullptr) return 2;
    float* pv = static_cast<float*>(ptr);
    int* pi = reinterpret_cast<int*>(pv + static_cast<size_t>(LIYAB_ARGMAX_STATIC_MAX_ROWS) * AM_CHUNKS);
    argmax_partial_kernel<<<dim3(rows, AM_CHUNKS), 256, 0, stream>>>(pv, pi, logits, ld, V);
    if (int rc = check_launch("argmax_partial")) return rc;
    argmax_final_kernel<<<rows, 64, 0, stream>>>(out, pv, pi, scatter_index, scatter_out);
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
    const bool plain = top_k == nullptr && top_p == nullptr;  // no row cuts its candidates
    // the row in registers where it fits; the general kernel beyond
#define LIYAB_REGS(E, T)                                                                                                              \
    do {                                                                                                                              \
        if (plain) sample_registers_kernel<E, T, true><<<rows, T, 0, stream>>>(out, logits, ld, V, temperature, top_k, top_p, uniform, scatter_index, scatter_out); \
        else sample_registers_kernel<E, T, false><<<rows, T, 0, stream>>>(out, logits, ld, V, temperature, top_k, top_p, uniform, scatter_index, scatter_out); \
    } while (0)
    // (3 more ids than the row has: a row may start up to 3 entries past a multiple of 16 bytes)
    if (V + 3 <= 8 * 1024) LIYAB_REGS(8, 1024);
    else if (V + 3 <= 16 * 1024) LIYAB_REGS(16, 1024);
    else if (V + 3 <= 48 * 512) LIYAB_REGS(48, 512);
    else if (V + 3 <= 72 * 512) LIYAB_REGS(72, 512);
    // (GPT-2's 50,257 on 1,024 threads with 52 ids each rather than 512 with 104; us a step of 8 rows: no cuts 21.9
    // against 30.7, top_k 40 with top_p 0.95 29.3 against 32.0, top_p 0.95 alone 49.4 against 64.6, top_k 100 58.0 against 66.5)
    else if (V + 3 <= 52 * 1024) LIYAB_REGS(52, 1024);
    else if (V + 3 <= 128 * 512) LIYAB_REGS(128, 512);
    else sample_kernel<<<rows, S_THREADS, 0, stream>>>(out, logits, ld, V, temperature, top_k, top_p, uniform, scatter_index, scatter_out);
#undef LIYAB_REGS
    return check_launch("sample");
}
