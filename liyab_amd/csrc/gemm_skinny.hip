// out[M,N] = a[M,K] . w[N,K]^T in bfloat16 for steps of few tokens (M <= 64):
// decoding, where the product is a stream of the weights.
//
// A workgroup owns 16 * NT output features (rows of `w`) and all M tokens as
// MT tiles of 16; its waves split K and add their partial sums through LDS in
// wave order. With v_mfma_f32_16x16x32_bf16 the weights are the first
// operand (16 rows) and the tokens the second (16), so an accumulator is a
// transposed output tile. A lane holds 8 consecutive k of its row per
// instruction, the four lane groups of a row 32 consecutive k: one load
// instruction reads 64 contiguous bytes of each of 16 rows (whole sectors;
// a lane reading 32 contiguous bytes in two instructions touched every
// sector twice). Weights are
// read once, straight from global memory into registers, 16 bytes a lane,
// one trip ahead of the multiplies; the tokens' rows come from L2 (every
// workgroup reads all of them: few, wide tiles of N would starve most CUs).
// K must be a multiple of 8. The order of the sum depends on the output feature, K and the
// split only, never on M.
//
// The product may be cut over K into parts (blockIdx.z), each part's sums going to its own
// plane of 32-bit sums; the first plane may take the bias and the rows the product is to be
// added to (themselves a sum of planes), so that the planes together are the new rows.
#include "common.h"
#include "launchers.h"
#include "epilogue.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

// What the first part of a product cut over K adds to its plane: the rows the product is
// added to, given as a sum of planes [n][M][N] (added in their order), or nothing.
struct BaseSum {
    const float* planes;
    int n;
    int64_t stride;
};

template <typename OutT, int MT, int NT, int MAXW>
__global__ void __launch_bounds__(64 * MAXW)
gemm_skinny_kernel(const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int M, int N, int K,
                   EpiParams epi, BaseSum base, int part_k, int64_t part_stride) {
    constexpr int UPT = (MT * NT == 1) ? 2 : 1;  // units of 64 k per trip
    constexpr int TILES = MT * NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int ksplit = blockDim.x / 64;
    float* red = reinterpret_cast<float*>(smem);

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16 * NT;
    const int m0 = blockIdx.y * 16 * MT;  // this workgroup's rows: [m0, m0 + 16 MT) of M
    // K may be cut into parts of part_k (a multiple of 64) over blockIdx.z, each part's sums
    // going to its own plane of the output; this workgroup's k are [k_begin, k_end)
    const int k_begin = blockIdx.z * part_k, k_end = min(K, k_begin + part_k);
    const int units = (k_end - k_begin + 63) / 64;
    if (gridDim.z > 1) epi.out = static_cast<float*>(epi.out) + blockIdx.z * part_stride;
    if (blockIdx.z > 0) epi.bias = nullptr;  // a cut product's bias goes to its first plane only
    const u32x4 zero = {0, 0, 0, 0};
    const bf16_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wrow[t] = w + static_cast<int64_t>(min(n0 + 16 * t + i, N - 1)) * K;

    // 8 consecutive k of a row; past the end it is the last piece, read and dropped: a load under
    // a branch would make the compiler wait for every load in flight, the next trip's too
    auto piece = [&](const bf16_t* row, int k) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + min(k, k_end - 8));
        return k < k_end ? v : zero;
    };
    // unit u covers k in k_begin + [64 u, 64 u + 64): two instructions of 32 k, this lane's 8 start at 8 g
    auto load_w = [&](int u0, Frag (&f)[UPT][NT][2]) {
#pragma unroll
        for (int p = 0; p < UPT; ++p) {
            const int k = k_begin + (u0 + p) * 64 + g * 8;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                f[p][t][0].u = piece(wrow[t], k);
                f[p][t][1].u = piece(wrow[t], k + 32);
            }
        }
    };
    // How K goes to the waves. As a rule a trip of the workgroup is UPT * ksplit consecutive
    // units, one wave after the other, and the next trip the next such stretch. Where rows lie
    // a multiple of 32 KB apart (K a multiple of 16,384), the sixteen rows of a workgroup, and
    // every workgroup's, begin in the same few memory channels, and workgroups in step crowd
    // those: there a wave walks a block of consecutive trips of its own, and a workgroup starts
    // blockIdx.x mod trips trips into its blocks and goes round past their end (16,384 ->
    // 4,096 in a decode step: 34.3 -> 28.3 us; at rows of 8 KB the same walk is no faster in
    // a step, though up to 12 % faster alone). The order of a sum depends on the output
    // feature, K and the split only, never on M.
    const bool blocks = K % 16384 == 0;
    const int trips = max(1, (units + UPT * ksplit - 1) / (UPT * ksplit));
    int trip = blocks ? static_cast<int>(blockIdx.x % trips) : 0;
    auto unit_of = [&](int t) { return blocks ? (wave * trips + t) * UPT : (t * ksplit + wave) * UPT; };
    Frag wc[UPT][NT][2];
    load_w(unit_of(trip), wc);
    // what the epilogue will read for this thread's first output (bias, residual) is asked for
    // now: after the sums it would be one more trip to memory on the critical path
    const int e_m = m0 + 16 * ((tid / 256) / NT) + (tid % 256) / 16, e_n = n0 + 16 * ((tid / 256) % NT) + tid % 16;
    const bool e_mine = tid < TILES * 256 && e_m < M && e_n < N;
    const float e_bias = (e_mine && epi.bias != nullptr) ? epi.bias[e_n] : 0.0f;
    const float e_res = (e_mine && epi.mode == kEpiResidual) ? epi.residual[static_cast<int64_t>(e_m) * epi.ldr + e_n] : 0.0f;
    // the first part's share of the rows the product is added to: up to four planes asked for
    // together (a plane past the last is the last one again, read and dropped)
    const bool based = base.planes != nullptr && blockIdx.z == 0;
    float e_base[4];
    {
        // no branch around the loads (a load under a branch is waited for where the branch ends,
        // and the weights asked for above with it): whoever has nothing to add reads a word of
        // the weights instead and drops it
        const float* src = based ? base.planes : reinterpret_cast<const float*>(w);
        const int64_t at = (based && e_mine) ? static_cast<int64_t>(e_m) * N + e_n : 0;
        const int64_t stride = based ? base.stride : 0;
        const int last = based ? base.n - 1 : 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) e_base[q] = src[min(q, last) * stride + at];
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the loads here: the scheduler would sink them to their use

    const bf16_t* arow[MT];
#pragma unroll
    for (int s = 0; s < MT; ++s) arow[s] = a + static_cast<int64_t>(min(m0 + 16 * s + i, M - 1)) * lda;
    // the tokens' fragments travel with the weights', a trip ahead: asked for after the next
    // trip's weights they would make every trip wait for those too (loads return in order)
    auto load_x = [&](int u0, Frag (&x)[UPT][MT][2]) {
#pragma unroll
        for (int p = 0; p < UPT; ++p) {
            const int k = k_begin + (u0 + p) * 64 + g * 8;
#pragma unroll
            for (int s = 0; s < MT; ++s) {
                x[p][s][0].u = piece(arow[s], k);
                x[p][s][1].u = piece(arow[s], k + 32);
            }
        }
    };
    Frag xc[UPT][MT][2];
    load_x(unit_of(trip), xc);

    floatx4 acc[MT][NT];
#pragma unroll
    for (int s = 0; s < MT; ++s)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[s][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    auto multiply = [&]() {
#pragma unroll
        for (int p = 0; p < UPT; ++p)
#pragma unroll
            for (int s = 0; s < MT; ++s)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][0].v, xc[p][s][0].v, acc[s][t], 0, 0, 0);
                    acc[s][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][1].v, xc[p][s][1].v, acc[s][t], 0, 0, 0);
                }
    };
    // every trip but the last asks for the next trip's operands before it multiplies; the last
    // one is peeled off, so no trip asks for (and then waits for) operands nobody uses
    // (dealt trip by trip, a wave whose unit of the last trip lies past the end of K stops a trip
    // early: it would ask for the rows' last bytes again, as every such wave would, and drop them)
    const int my_trips = blocks ? trips : max(1, (units - wave * UPT + UPT * ksplit - 1) / (UPT * ksplit));
    for (int left = my_trips - 1; left > 0; --left) {
        trip = trip + 1 == trips ? 0 : trip + 1;
        Frag wn[UPT][NT][2], xn[UPT][MT][2];
        load_w(unit_of(trip), wn);
        load_x(unit_of(trip), xn);
        multiply();
#pragma unroll
        for (int p = 0; p < UPT; ++p) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                wc[p][t][0] = wn[p][t][0];
                wc[p][t][1] = wn[p][t][1];
            }
#pragma unroll
            for (int s = 0; s < MT; ++s) {
                xc[p][s][0] = xn[p][s][0];
                xc[p][s][1] = xn[p][s][1];
            }
        }
    }
    multiply();  // a wave past the end of K holds zeros
    // acc[s][t][r] = partial C^T[n = 16 t + 4 g + r][m = 16 s + i]; kept [tile][m][n] per wave
#pragma unroll
    for (int s = 0; s < MT; ++s)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) red[(wave * TILES + s * NT + t) * 256 + i * 16 + 4 * g + r] = acc[s][t][r];
    __syncthreads();
    for (int e = tid; e < TILES * 256; e += blockDim.x) {
        const int tile = e / 256, s = tile / NT, t = tile % NT;
        const int m = m0 + 16 * s + (e % 256) / 16, n = n0 + 16 * t + e % 16;
        float v = 0.0f;
        for (int q = 0; q < ksplit; ++q) v += red[q * TILES * 256 + e];
        if (m >= M || n >= N) continue;
        if (based) {
            // this plane = (sums + bias) + (base planes added up in their order)
            const float* bp = base.planes + static_cast<int64_t>(m) * N + n;
            float b;
            if (e == tid) {
                b = e_base[0];
#pragma unroll
                for (int q = 1; q < 4; ++q)
                    if (q < base.n) b += e_base[q];
                for (int q = 4; q < base.n; ++q) b += bp[q * base.stride];
            } else {
                b = bp[0];
                for (int q = 1; q < base.n; ++q) b += bp[q * base.stride];
            }
            v = (v + (e == tid ? e_bias : epilogue_bias(epi, n))) + b;
            static_cast<float*>(epi.out)[static_cast<int64_t>(m) * epi.ldo + n] = v;
            continue;
        }
        if (e != tid) epilogue_store<OutT>(epi, m, n, v);
        else if (epi.mode == kEpiResidual) epi.residual[static_cast<int64_t>(m) * epi.ldr + n] = e_res + (v + e_bias);
        else epilogue_store_biased<OutT>(epi, m, n, v + e_bias);
    }
}

template <int MT, int NT, int MAXW>
int launch_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit, const EpiParams& epi,
                  const BaseSum& base, int kparts, int64_t part_stride, hipStream_t stream) {
    // K in kparts parts, each a whole number of units of 64 and none of them empty (the caller's check)
    const int part_k = ((K + 63) / 64 + kparts - 1) / kparts * 64;
    const dim3 grid((N + 16 * NT - 1) / (16 * NT), (M + 16 * MT - 1) / (16 * MT), kparts);
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (ksplit > MAXW) ksplit = MAXW;
    size_t smem = static_cast<size_t>(ksplit) * MT * NT * 256 * sizeof(float);
    const bool f32 = epi.mode == kEpiResidual || epi.out_dtype == kF32;
    if (f32) {
        auto kern = gemm_skinny_kernel<float, MT, NT, MAXW>;
        static bool ready = false;
        if (!ready) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            ready = true;
        }
        kern<<<grid, 64 * ksplit, smem, stream>>>(pa, lda, pw, M, N, K, epi, base, part_k, part_stride);
    } else {
        auto kern = gemm_skinny_kernel<bf16_t, MT, NT, MAXW>;
        static bool ready = false;
        if (!ready) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            ready = true;
        }
        kern<<<grid, 64 * ksplit, smem, stream>>>(pa, lda, pw, M, N, K, epi, base, part_k, part_stride);
    }
    return check_launch("gemm_skinny");
}

static int skinny_dispatch(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit, int wide, int mtile,
                           const EpiParams& epi, const BaseSum& base, hipStream_t stream, int kparts = 1,
                           int64_t part_stride = 0) {
    // tiles of 16 rows a workgroup: all of M in one workgroup reads the weights once; with few
    // output features that leaves most of the chip idle, and the rows are spread over workgroups
    // instead (the weights then come from L2 after their first reading)
    // (measured at 24 to 64 rows over GPT-2 small's, medium's and XL's shapes: the most rows a
    // workgroup that still leaves 144 workgroups or more is the fastest or close to it)
    int mt = 1;
    if (mtile > 0) {
        mt = mtile;
    } else {
        const int strips = (N + 15) / 16;
        for (int cand = M <= 16 ? 1 : (M <= 32 ? 2 : 4); cand > 1; cand /= 2)
            if (strips * ((M + 16 * cand - 1) / (16 * cand)) >= 144) {
                mt = cand;
                break;
            }
    }
    LIYAB_REQUIRE(mt == 1 || mt == 2 || mt == 4, "gemm_skinny: %d tiles of rows a workgroup is not 1, 2 or 4", mt);
    // wide tiles of N (64 features a workgroup) when N is so large that every workgroup
    // re-reading the tokens would cost more than the weights
    if (wide < 0) wide = (mt > 1 && static_cast<long>(N) * M > (1L << 20)) ? 1 : 0;
    const int nt = wide ? 4 : 1;
    if (ksplit == 0) {
        // waves until each has one trip's worth of K (everything is then asked for at once),
        // or they cover the chip several times over
        const int tiles = ((N + 16 * nt - 1) / (16 * nt)) * ((M + 16 * mt - 1) / (16 * mt)) * kparts;
        const int units = ((K + 63) / 64 + kparts - 1) / kparts, per_trip = mt * nt == 1 ? 2 : 1;
        ksplit = 1;
        // (with so many output features that one wave a workgroup covers the chip, two or four
        // still pay while a wave keeps more than 8 units: 18.3 against 20.0 us for 768 -> 50,257)
        while (ksplit < 16 && units > ksplit * per_trip && (tiles * ksplit < 2048 || units / ksplit > 8)) ksplit *= 2;
    }
    LIYAB_REQUIRE(ksplit == 1 || ksplit == 2 || ksplit == 4 || ksplit == 8 || ksplit == 16,
                  "gemm_skinny: ksplit %d is not 1, 2, 4, 8 or 16", ksplit);
    if (nt == 1) {
        if (mt == 1) return launch_skinny<1, 1, 16>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
        if (mt == 2) return launch_skinny<2, 1, 16>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
        return launch_skinny<4, 1, 16>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
    }
    if (mt == 1) return launch_skinny<1, 4, 4>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
    if (mt == 2) return launch_skinny<2, 4, 4>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
    return launch_skinny<4, 4, 4>(a, lda, w, M, N, K, ksplit, epi, base, kparts, part_stride, stream);
}

}  // namespace liyab

using namespace liyab;

// a [M <= 64, K] and w [N, K] are bfloat16. ksplit: waves per workgroup sharing K (0 = chosen
// from the shape; 1, 2, 4, 8 or 16). wide: 64 instead of 16 output features a workgroup
// (-1 = chosen from the shape). mtile: tiles of 16 rows a workgroup, 1, 2 or 4 (0 = chosen from the shape).
extern "C" int liyab_gemm_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit, int wide,
                                 int mtile, const EpiParams* epi_in, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && epi_in, "gemm: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d (at most 64) N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % 8 == 0 && lda % 8 == 0 && lda >= K, "gemm_skinny: K %d and lda %lld must be multiples of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_skinny: operands must be 16-byte aligned");
    EpiParams epi = *epi_in;
    if (int rc = check_epilogue(epi, M, N)) return rc;
    if (M == 0) return 0;
    return skinny_dispatch(a, lda, w, M, N, K, ksplit, wide, mtile, epi, BaseSum{nullptr, 0, 0}, stream);
}

// The product's sums over `kparts` parts of K, one plane [M, N] of 32-bit sums a part:
// parts[p * part_stride + m * N + n] = sum over the p-th part of K of a[m, k] w[n, k].
// For a product with few output features and a long K: cut over K it fills the chip, and
// whoever reads the result next adds the planes up in their order (the norm kernels do).
// With `base` (n_base planes [M, N], base_stride floats apart, not overlapping `parts`), the
// first plane also takes bias[n] and base[0][m, n] + base[1][m, n] + ...: the planes together
// are then base + a . w^T + bias, the rows of a residual stream after the product was added.
// Without `base`, `bias` must be null. Every part holds at least one unit of 64 k:
// (kparts - 1) * ceil(ceil(K / 64) / kparts) * 64 < K.
extern "C" int liyab_gemm_skinny_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts,
                                       int ksplit, float* parts, int64_t part_stride, const float* bias,
                                       const float* base, int n_base, int64_t base_stride, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && parts, "gemm: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny_parts: bad sizes M=%d (at most 64) N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % 8 == 0 && lda % 8 == 0 && lda >= K, "gemm_skinny_parts: K %d and lda %lld must be multiples of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_skinny_parts: operands must be 16-byte aligned");
    const int units = (K + 63) / 64;
    LIYAB_REQUIRE(kparts >= 1 && kparts <= 16 && (kparts - 1) * ((units + kparts - 1) / kparts) < units,
                  "gemm_skinny_parts: K = %d does not cut into %d parts of whole units of 64", K, kparts);
    LIYAB_REQUIRE(part_stride >= static_cast<int64_t>(M) * N, "gemm_skinny_parts: planes of %lld overlap", static_cast<long long>(part_stride));
    LIYAB_REQUIRE(base != nullptr || bias == nullptr, "gemm_skinny_parts: a bias needs the rows it is added to");
    if (base != nullptr) {
        LIYAB_REQUIRE(n_base >= 1 && n_base <= 16 && (n_base == 1 || base_stride >= static_cast<int64_t>(M) * N),
                      "gemm_skinny_parts: bad planes of rows to add to (%d, %lld apart)", n_base, static_cast<long long>(base_stride));
        const float* base_end = base + (n_base - 1) * base_stride + static_cast<int64_t>(M) * N;
        const float* parts_end = parts + (kparts - 1) * part_stride + static_cast<int64_t>(M) * N;
        LIYAB_REQUIRE(base_end <= parts || parts_end <= base, "gemm_skinny_parts: the rows to add to overlap the planes written");
    }
    if (M == 0) return 0;
    EpiParams epi{};
    epi.mode = kEpiNone;
    epi.out_dtype = kF32;
    epi.out = parts;
    epi.ldo = N;
    epi.bias = bias;
    // cut over K: 16 rows a workgroup (the parts cover the chip); whole: as the plain product chooses
    return skinny_dispatch(a, lda, w, M, N, K, ksplit, 0, kparts > 1 ? 1 : 0, epi, BaseSum{base, n_base, base_stride}, stream, kparts,
                           part_stride);
}
