// Attention's output projection for steps of at most 32 tokens, cut over its inner
// dimension, reading attention's output as the decode kernel's splits leave it.
//
// With few tokens in flight a (token, head) pair's keys are cut into splits over several
// workgroups so that the chip is covered; each split leaves its weighted values with its
// maximum and sum (the reference's per-span partial softmax, src/core/transformer.cpp:2327-2358),
// and somebody has to merge them (:2367-2385). A kernel of its own for that costs as much as the
// attention it follows. Here the projection merges them as it loads its first operand: a
// workgroup owns 16 output features and one part of K, which is a few heads' worth of
// attention output for every token; it reads those heads' splits, merges them in split order
// into bfloat16 rows in LDS, and multiplies. The splits are asked for before the weights
// (loads are counted in order: a wait for the splits does not wait for the weights, which come
// from further away). The sums go to one plane a part, the first plane also taking the bias
// and the rows of the residual stream the product is added to, as in the plain cut product.
#include "common.h"
#include "launchers.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(2))) float floatx2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

namespace att_proj {

union Frag {
    u32x4 u;
    bf16x8 v;
};

constexpr int WAVES = 8;
constexpr int MAX_SPLITS = 8;

struct Splits {
    const float* partials;  // [M][n_head][n_splits][hd + 4]: values, maximum, sum, two unused
    int n_splits, n_head, hd;
};
struct BaseSum {
    const float* planes;  // rows the product is added to, a sum of planes [n][M][N]; or null
    int n;
    int64_t stride;
};

template <int MT>  // tiles of 16 rows
__global__ void __launch_bounds__(64 * WAVES)
gemm_att_parts_kernel(Splits att, const bf16_t* __restrict__ w, int M, int N, int K, float* __restrict__ out, int part_k,
                      int64_t part_stride, const float* __restrict__ bias, BaseSum base) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const int k_begin = blockIdx.z * part_k, k_end = min(K, k_begin + part_k);
    const int pk = k_end - k_begin, units = (pk + 63) / 64;
    const int ldx = pk + 8;
    bf16_t* xs = reinterpret_cast<bf16_t*>(smem);  // [M][pk + 8]
    float* red = reinterpret_cast<float*>(smem + ((static_cast<size_t>(M) * ldx * 2 + 15) / 16) * 16);  // [waves][MT][256]
    out += blockIdx.z * part_stride;
    const u32x4 zero = {0, 0, 0, 0};
    const int S = att.n_splits, hd4 = att.hd + 4;

    // -- the first operand: four consecutive k of a token a thread, merged over the splits ----
    const int per = pk / 4, items = M * per;
    struct Item {
        floatx4 acc[MAX_SPLITS];
        floatx2 ml[MAX_SPLITS];
        const float* p;
        int m, kk, e;
        bool valid;
    };
    auto fetch = [&](int it) {
        Item x;
        x.valid = it < items;
        const int itc = min(it, items - 1);  // past the end: the last one again, computed and dropped
        x.m = itc / per;
        x.kk = (itc - x.m * per) * 4;
        const int k = k_begin + x.kk, head = k / att.hd;
        x.e = k - head * att.hd;
        x.p = att.partials + (static_cast<int64_t>(x.m) * att.n_head + head) * S * hd4;
#pragma unroll
        for (int s = 0; s < MAX_SPLITS; ++s) x.ml[s] = *reinterpret_cast<const floatx2*>(x.p + min(s, S - 1) * hd4 + att.hd);
        // every split's values are asked for here, ahead of the weights: asked for after them
        // (loads are counted in order) a wait for a split would be a wait for the weights
#pragma unroll
        for (int s = 0; s < MAX_SPLITS; ++s) x.acc[s] = *reinterpret_cast<const floatx4*>(x.p + min(s, S - 1) * hd4 + x.e);
        return x;
    };
    auto finish = [&](const Item& x) {
        float mx = -INFINITY;
#pragma unroll
        for (int s = 0; s < MAX_SPLITS; ++s)
            if (s < S) mx = fmaxf(mx, x.ml[s][0]);
        float wgt[MAX_SPLITS];
        float sum = 0.0f;
#pragma unroll
        for (int s = 0; s < MAX_SPLITS; ++s) {
            wgt[s] = (s < S && x.ml[s][0] != -INFINITY) ? __expf(x.ml[s][0] - mx) : 0.0f;  // an empty split weighs nothing
            sum += wgt[s] * x.ml[s][1];
        }
        floatx4 o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int s = 0; s < MAX_SPLITS; ++s) o += wgt[s] * x.acc[s];  // a split past the last weighs nothing
        if (x.valid) {
            uint2 packed;
            packed.x = static_cast<uint32_t>(float_to_bf16(o[0] / sum)) | (static_cast<uint32_t>(float_to_bf16(o[1] / sum)) << 16);
            packed.y = static_cast<uint32_t>(float_to_bf16(o[2] / sum)) | (static_cast<uint32_t>(float_to_bf16(o[3] / sum)) << 16);
            *reinterpret_cast<uint2*>(xs + x.m * ldx + x.kk) = packed;
        }
    };
    const Item first = fetch(tid);

    // -- this wave's share of the weights, and what the epilogue will read -----------------
    const bf16_t* wrow = w + static_cast<int64_t>(min(n0 + i, N - 1)) * K;
    // 8 consecutive k of a row; past the part's end it is the last piece, read and dropped
    auto piece = [&](const bf16_t* row, int k, int end) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + min(k, end - 8));
        return k < end ? v : zero;
    };
    auto load_w = [&](int u0, Frag (&f)[2][2]) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int k = k_begin + (u0 + p) * 64 + g * 8;
            f[p][0].u = piece(wrow, k, k_end);
            f[p][1].u = piece(wrow, k + 32, k_end);
        }
    };
    // K goes to the waves as in gemm_skinny_kernel (trips of consecutive units, or, where rows
    // lie a multiple of 32 KB apart, a block of trips a wave begun blockIdx.x mod trips trips
    // in): the same bits
    const bool blocks = K % 16384 == 0;
    const int trips = max(1, (units + 2 * WAVES - 1) / (2 * WAVES));
    int trip = blocks ? static_cast<int>(blockIdx.x % trips) : 0;
    auto unit_of = [&](int t) { return blocks ? (wave * trips + t) * 2 : (t * WAVES + wave) * 2; };
    Frag wc[2][2];
    load_w(unit_of(trip), wc);
    const int e_m = 16 * (tid / 256) + (tid % 256) / 16, e_n = n0 + tid % 16;  // tile tid / 256 of rows
    const bool e_mine = tid < MT * 256 && e_m < M && e_n < N;
    const bool based = base.planes != nullptr && blockIdx.z == 0;
    const float e_bias = (e_mine && based && bias != nullptr) ? bias[e_n] : 0.0f;
    float e_base[4];
    {
        // no branch around the loads: whoever has nothing to add reads a word of the weights and drops it
        const float* src = based ? base.planes : reinterpret_cast<const float*>(w);
        const int64_t at = (based && e_mine) ? static_cast<int64_t>(e_m) * N + e_n : 0;
        const int64_t stride = based ? base.stride : 0;
        const int last = based ? base.n - 1 : 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) e_base[q] = src[min(q, last) * stride + at];
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the loads in this order: the scheduler would sink them to their use

    finish(first);
    for (int it = tid + 64 * WAVES; it < items; it += 64 * WAVES) finish(fetch(it));
    lds_barrier();  // the weights may still be on their way

    // -- the product ---------------------------------------------------------------------
    const bf16_t* arow[MT];
    floatx4 acc[MT];
#pragma unroll
    for (int r = 0; r < MT; ++r) {
        arow[r] = xs + min(16 * r + i, M - 1) * ldx;
        acc[r] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    auto multiply = [&](int u0) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int kk = (u0 + p) * 64 + g * 8;  // within the part
#pragma unroll
            for (int r = 0; r < MT; ++r) {
                Frag x0, x1;
                x0.u = piece(arow[r], kk, pk);
                x1.u = piece(arow[r], kk + 32, pk);
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][0].v, x0.v, acc[r], 0, 0, 0);
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][1].v, x1.v, acc[r], 0, 0, 0);
            }
        }
    };
    const int my_trips = blocks ? trips : max(1, (units - wave * 2 + 2 * WAVES - 1) / (2 * WAVES));  // (as gemm_skinny_kernel stops a wave early)
    for (int left = my_trips - 1; left > 0; --left) {
        const int u0 = unit_of(trip);
        trip = trip + 1 == trips ? 0 : trip + 1;
        Frag wn[2][2];
        load_w(unit_of(trip), wn);
        multiply(u0);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            wc[p][0] = wn[p][0];
            wc[p][1] = wn[p][1];
        }
    }
    multiply(unit_of(trip));  // a wave past the end of the part holds zeros
    // acc[r][c] = partial C^T[n = 4 g + c][m = 16 r + i]; kept [tile][m][n] per wave, added up in wave order
#pragma unroll
    for (int r = 0; r < MT; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) red[(wave * MT + r) * 256 + i * 16 + 4 * g + c] = acc[r][c];
    __syncthreads();
    if (tid < MT * 256) {
        float v = 0.0f;
#pragma unroll
        for (int q = 0; q < WAVES; ++q) v += red[q * MT * 256 + tid];
        if (e_mine) {
            if (based) {
                // this plane = (sums + bias) + (base planes added up in their order)
                const float* bp = base.planes + static_cast<int64_t>(e_m) * N + e_n;
                float b = e_base[0];
#pragma unroll
                for (int q = 1; q < 4; ++q)
                    if (q < base.n) b += e_base[q];
                for (int q = 4; q < base.n; ++q) b += bp[q * base.stride];
                v = (v + e_bias) + b;
            }
            out[static_cast<int64_t>(e_m) * N + e_n] = v;
        }
    }
}

}  // namespace att_proj
}  // namespace liyab

using namespace liyab;

// parts[p] = merged(partials) . w^T summed over the p-th of `kparts` parts of K = n_head * hd,
// one plane [M, N] of 32-bit sums a part. partials [M][n_head][n_splits][hd + 4] float32 as
// liyab_attention_decode leaves them with `leave_splits` (row m is token slot m); w [N, K]
// bfloat16. M <= 32, n_splits <= 8, hd a multiple of 8. With `base` (n_base planes [M, N],
// base_stride floats apart, not overlapping `parts`) the first plane also takes bias[n] and the
// rows base[0] + base[1] + ...; without it `bias` must be null.
extern "C" int liyab_gemm_att_parts(const float* partials, int n_splits, int n_head, int hd, const void* w, int M, int N,
                                    int kparts, float* parts, int64_t part_stride, const float* bias, const float* base,
                                    int n_base, int64_t base_stride, hipStream_t stream) {
    LIYAB_REQUIRE(partials && w && parts, "gemm_att_parts: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 32 && N > 0 && n_head > 0, "gemm_att_parts: bad sizes M=%d (at most 32) N=%d heads=%d", M, N, n_head);
    LIYAB_REQUIRE(hd >= 8 && hd <= 256 && hd % 8 == 0, "gemm_att_parts: head size %d is not a multiple of 8 in 8..256", hd);
    LIYAB_REQUIRE(n_splits >= 1 && n_splits <= att_proj::MAX_SPLITS, "gemm_att_parts: %d splits (1 to %d)", n_splits, att_proj::MAX_SPLITS);
    const int K = n_head * hd;
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(partials) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_att_parts: operands must be 16-byte aligned");
    const int units = (K + 63) / 64;
    LIYAB_REQUIRE(kparts >= 1 && kparts <= 16 && (kparts - 1) * ((units + kparts - 1) / kparts) < units,
                  "gemm_att_parts: K = %d does not cut into %d parts of whole units of 64", K, kparts);
    LIYAB_REQUIRE(part_stride >= static_cast<int64_t>(M) * N, "gemm_att_parts: planes of %lld overlap", static_cast<long long>(part_stride));
    LIYAB_REQUIRE(base != nullptr || bias == nullptr, "gemm_att_parts: a bias needs the rows it is added to");
    if (base != nullptr) {
        LIYAB_REQUIRE(n_base >= 1 && n_base <= 16 && (n_base == 1 || base_stride >= static_cast<int64_t>(M) * N),
                      "gemm_att_parts: bad planes of rows to add to (%d, %lld apart)", n_base, static_cast<long long>(base_stride));
        const float* base_end = base + (n_base - 1) * base_stride + static_cast<int64_t>(M) * N;
        const float* parts_end = parts + (kparts - 1) * part_stride + static_cast<int64_t>(M) * N;
        LIYAB_REQUIRE(base_end <= parts || parts_end <= base, "gemm_att_parts: the rows to add to overlap the planes written");
    }
    if (M == 0) return 0;
    const int part_k = (units + kparts - 1) / kparts * 64;
    const int mt = M <= 16 ? 1 : 2;
    const size_t smem = ((static_cast<size_t>(M) * (part_k + 8) * 2 + 15) / 16) * 16 + att_proj::WAVES * mt * 256 * sizeof(float);
    LIYAB_REQUIRE(smem <= 64 * 1024, "gemm_att_parts: %d rows of a part of %d do not fit LDS", M, part_k);
    const dim3 grid((N + 15) / 16, 1, kparts);
    const att_proj::Splits att{partials, n_splits, n_head, hd};
    const att_proj::BaseSum bs{base, n_base, base_stride};
    auto* pw = static_cast<const bf16_t*>(w);
    if (mt == 1) att_proj::gemm_att_parts_kernel<1><<<grid, 64 * att_proj::WAVES, smem, stream>>>(att, pw, M, N, K, parts, part_k, part_stride, bias, bs);
    else att_proj::gemm_att_parts_kernel<2><<<grid, 64 * att_proj::WAVES, smem, stream>>>(att, pw, M, N, K, parts, part_k, part_stride, bias, bs);
    return check_launch("gemm_att_parts");
}
