// out[M,N] = LayerNorm(x)[M,K] . w[N,K]^T in bfloat16 for steps of at most 32 tokens,
// the norm computed by the product kernel itself: a decode step is a chain of
// small kernels, each of which costs its launch and a first trip to memory
// whatever its work, and the norm is two of the seven kernels of a layer.
//
// x, the 32-bit residual stream, may come as a sum of planes (a product cut
// over its inner dimension leaves one plane of sums a part; the first plane
// holds the stream it was added to): x[m] = planes[0][m] + planes[1][m] + ...,
// added in that order. A workgroup owns 16 output features and all M rows.
// Its eight waves first ask for their share of the weights (K is split over
// the waves, as in the plain streaming kernel), then each wave normalises
// rows m = wave, wave + 8, ...: the row's pieces of every plane are asked for
// together, 16 bytes a lane, no load under a branch; statistics are two
// passes over registers with the standalone kernel's reduction tree (the
// reference's layernorm, src/core/transformer.cpp:77-106), so both kernels
// give the same bits. The normalised rows go to LDS in bfloat16 and are the
// second operand of v_mfma_f32_16x16x32_bf16; the weights' trip to memory and
// the norm overlap. Every workgroup repeats the norm: it pays while the rows
// are few (M * K * planes * 4 bytes from L2 a workgroup).
#include "common.h"
#include "launchers.h"
#include "epilogue.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

namespace ln_fold {

union Frag {
    u32x4 u;
    bf16x8 v;
};

constexpr int LN_WAVES = 8;

struct NormParams {
    const float* planes;  // [n_planes][rows][K]
    int n_planes;
    int64_t plane_stride;
    const float* weight;  // [K] or null
    const float* bias;    // [K] or null
    float eps;
};

template <typename OutT, int MAXV, int MT, int NT>
__global__ void __launch_bounds__(64 * LN_WAVES)
gemm_skinny_ln_kernel(NormParams ln, const bf16_t* __restrict__ w, int M, int N, int K, EpiParams epi) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int ldx = K + 8;  // rows 16 bytes apart modulo the banks: a group of 16 lanes reads 16 rows without conflict
    constexpr int TILES = MT * NT;  // MT tiles of 16 rows (all M rows), NT tiles of 16 output features
    bf16_t* xs = reinterpret_cast<bf16_t*>(smem);  // [M][K + 8]
    float* red = reinterpret_cast<float*>(smem + ((static_cast<size_t>(M) * ldx * 2 + 15) / 16) * 16);  // [waves][TILES][256]

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16 * NT;  // NT tiles of 16 output features a workgroup
    const int units = (K + 63) / 64;
    const u32x4 zero = {0, 0, 0, 0};
    const bf16_t* wrow[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wrow[t] = w + static_cast<int64_t>(min(n0 + 16 * t + i, N - 1)) * K;

    // 8 consecutive k of a row; past the end it is the last piece, read and dropped
    auto piece = [&](const bf16_t* row, int k) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(row + min(k, K - 8));
        return k < K ? v : zero;
    };
    // a trip of a wave is two units of 64 k: unit u covers k in [64 u, 64 u + 64), two
    // instructions of 32 k, this lane's 8 start at 8 g
    auto load_w = [&](int u0, Frag (&f)[2][NT][2]) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int k = (u0 + p) * 64 + g * 8;
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                f[p][t][0].u = piece(wrow[t], k);
                f[p][t][1].u = piece(wrow[t], k + 32);
            }
        }
    };
    Frag wc[2][NT][2];
    // this thread's first output: tile tid / 256 = (row tile, feature tile)
    const int e_m = 16 * ((tid / 256) / NT) + (tid % 256) / 16, e_n = n0 + 16 * ((tid / 256) % NT) + tid % 16;
    const bool e_mine = tid < TILES * 256 && e_m < M && e_n < N;
    float e_bias = 0.0f;

    // -- the norm: a wave per row, the row in registers ---------------------------------
    const int nv = K / 4;
    const floatx4 fzero = {0.0f, 0.0f, 0.0f, 0.0f}, fone = {1.0f, 1.0f, 1.0f, 1.0f};
    // `between` runs once the row's first loads are asked for and before anything waits for them
    auto norm_row = [&](int m, bool keep, auto&& between) {
        const float* row0 = ln.planes + static_cast<int64_t>(m) * K;
        // the norm's weight and bias travel with the row: asked for after the weights of the
        // product, a wait for them would be a wait for those
        floatx4 v[MAXV], gw[MAXV], gb[MAXV];
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
            const int at = min(lane + kWave * j, nv - 1);  // past the row: its last piece again, unused
            v[j] = reinterpret_cast<const floatx4*>(row0)[at];
            gw[j] = ln.weight != nullptr ? reinterpret_cast<const floatx4*>(ln.weight)[at] : fone;
            gb[j] = ln.bias != nullptr ? reinterpret_cast<const floatx4*>(ln.bias)[at] : fzero;
        }
        // further planes, PB together (a plane past the last is the last one again, read and dropped)
        constexpr int PB = MAXV <= 4 ? 3 : 1;  // what the registers hold
        bool first = true;
        for (int q0 = 1; q0 < ln.n_planes || first; q0 += PB) {
            floatx4 plane[PB][MAXV];
#pragma unroll
            for (int u = 0; u < PB; ++u) {
                const float* row = row0 + min(q0 + u, ln.n_planes - 1) * ln.plane_stride;
#pragma unroll
                for (int j = 0; j < MAXV; ++j) plane[u][j] = reinterpret_cast<const floatx4*>(row)[min(lane + kWave * j, nv - 1)];
            }
            if (first) {
                between();
                __builtin_amdgcn_sched_barrier(0);  // keep the loads in this order: the scheduler would sink them to their use
                first = false;
            }
#pragma unroll
            for (int u = 0; u < PB; ++u)
#pragma unroll
                for (int j = 0; j < MAXV; ++j)
                    if (q0 + u < ln.n_planes) v[j] += plane[u][j];
        }
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (lane + kWave * j < nv) s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
        const float mean = wave_sum(s) / static_cast<float>(K);
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (lane + kWave * j < nv) {
                const floatx4 dev = v[j] - mean;
                ss += (dev[0] * dev[0] + dev[1] * dev[1]) + (dev[2] * dev[2] + dev[3] * dev[3]);
            }
        const float scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(K) + ln.eps);
#pragma unroll
        for (int j = 0; j < MAXV; ++j)
            if (keep && lane + kWave * j < nv) {
                const floatx4 y = (v[j] - mean) * scale * gw[j] + gb[j];
                uint2 packed;
                packed.x = static_cast<uint32_t>(float_to_bf16(y[0])) | (static_cast<uint32_t>(float_to_bf16(y[1])) << 16);
                packed.y = static_cast<uint32_t>(float_to_bf16(y[2])) | (static_cast<uint32_t>(float_to_bf16(y[3])) << 16);
                *reinterpret_cast<uint2*>(xs + m * ldx + 4 * (lane + kWave * j)) = packed;
            }
    };
    // The wave's first row (a wave past the last row works on the last row and keeps nothing, so
    // that every wave runs the same loads). Its loads go first and the wave's share of the weights
    // and its bias right after: counted in order, a wait for the row does not wait for the weights,
    // which come from further away and arrive while the norm is computed.
    auto ask_weights = [&]() {
        load_w(wave * 2, wc);
        e_bias = (e_mine && epi.bias != nullptr) ? epi.bias[e_n] : 0.0f;
    };
    // (a wave past the last row asks for its weights only: a compute unit takes 64 bytes a cycle from
    // its cache, and eight waves that each ask for a row in four planes and the norm's two vectors
    // are 147 KB, six times the workgroup's weights)
    if (wave < M) norm_row(wave, true, ask_weights);
    else ask_weights();
    for (int m = wave + LN_WAVES; m < M; m += LN_WAVES) norm_row(m, true, []() {});
    lds_barrier();  // the weights may still be on their way

    // -- the product ------------------------------------------------------------------
    const bf16_t* arow[MT];
#pragma unroll
    for (int r = 0; r < MT; ++r) arow[r] = xs + min(16 * r + i, M - 1) * ldx;
    floatx4 acc[MT][NT];
#pragma unroll
    for (int r = 0; r < MT; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    auto multiply = [&](int u0) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int k = (u0 + p) * 64 + g * 8;
#pragma unroll
            for (int r = 0; r < MT; ++r) {
                Frag x0, x1;
                x0.u = piece(arow[r], k);
                x1.u = piece(arow[r], k + 32);
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][0].v, x0.v, acc[r][t], 0, 0, 0);
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[p][t][1].v, x1.v, acc[r][t], 0, 0, 0);
                }
            }
        }
    };
    // every trip but the last asks for the next trip's weights before it multiplies; the last
    // one is peeled off, so no trip asks for (and then waits for) weights nobody uses
    int u0 = wave * 2;
    for (; u0 + 2 * LN_WAVES < units; u0 += 2 * LN_WAVES) {
        Frag wn[2][NT][2];
        load_w(u0 + 2 * LN_WAVES, wn);
        multiply(u0);
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                wc[p][t][0] = wn[p][t][0];
                wc[p][t][1] = wn[p][t][1];
            }
    }
    multiply(u0);  // a wave past the end of K holds zeros
    // acc[r][t][c] = partial C^T[n = 16 t + 4 g + c][m = 16 r + i]; kept [tile][m][n] per wave, added up in wave order
#pragma unroll
    for (int r = 0; r < MT; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int c = 0; c < 4; ++c) red[(wave * TILES + r * NT + t) * 256 + i * 16 + 4 * g + c] = acc[r][t][c];
    __syncthreads();
    for (int e = tid; e < TILES * 256; e += 64 * LN_WAVES) {
        const int tile = e / 256, m = 16 * (tile / NT) + (e % 256) / 16, n = n0 + 16 * (tile % NT) + e % 16;
        float v = 0.0f;
#pragma unroll
        for (int q = 0; q < LN_WAVES; ++q) v += red[q * TILES * 256 + e];
        if (m >= M || n >= N) continue;
        if (e == tid) epilogue_store_biased<OutT>(epi, m, n, v + e_bias);
        else epilogue_store<OutT>(epi, m, n, v);
    }
}

template <typename OutT, int MAXV, int MT, int NT>
int launch_kernel(const NormParams& ln, const void* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    const dim3 grid((N + 16 * NT - 1) / (16 * NT));
    const size_t smem = ((static_cast<size_t>(M) * (K + 8) * 2 + 15) / 16) * 16 + LN_WAVES * MT * NT * 256 * sizeof(float);
    LIYAB_REQUIRE(smem <= 160 * 1024, "gemm_skinny_ln: %d rows of %d need %zu bytes of LDS", M, K, smem);
    auto kern = gemm_skinny_ln_kernel<OutT, MAXV, MT, NT>;
    static bool ready = false;
    if (!ready) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        ready = true;
    }
    kern<<<grid, 64 * LN_WAVES, smem, stream>>>(ln, static_cast<const bf16_t*>(w), M, N, K, epi);
    return check_launch("gemm_skinny_ln");
}

// A workgroup keeps a row in registers and so fills a compute unit: with more strips of 16
// output features than compute units a workgroup takes two strips, or the workgroups would run
// in two rounds (one tile of rows only: with more rows the sums across waves fill the LDS).
template <typename OutT, int MAXV>
int launch_rows(const NormParams& ln, const void* w, int M, int N, int K, int wide, const EpiParams& epi, hipStream_t stream) {
    if (M <= 16) return wide ? launch_kernel<OutT, MAXV, 1, 2>(ln, w, M, N, K, epi, stream) : launch_kernel<OutT, MAXV, 1, 1>(ln, w, M, N, K, epi, stream);
    return launch_kernel<OutT, MAXV, 2, 1>(ln, w, M, N, K, epi, stream);
}
template <int MAXV>
int launch_ln(const NormParams& ln, const void* w, int M, int N, int K, int wide, const EpiParams& epi, hipStream_t stream) {
    if (epi.out_dtype == kF32) return launch_rows<float, MAXV>(ln, w, M, N, K, wide, epi, stream);
    return launch_rows<bf16_t, MAXV>(ln, w, M, N, K, wide, epi, stream);
}

}  // namespace ln_fold
}  // namespace liyab

using namespace liyab;
using namespace liyab::ln_fold;

// out = epilogue(LayerNorm(planes[0] + planes[1] + ...) . w^T + bias). planes: float32
// [n_planes][M][K], plane_stride floats apart (n_planes = 1: the rows themselves); w [N, K]
// bfloat16. M <= 32 (measured: from 32 rows on the norm's own kernel is faster; with 64 rows
// every workgroup normalising them all cost 950 against 810 us a step); K a multiple of 8, at
// most 2048. wide: 32 instead of 16 output features a workgroup, for M <= 16 (-1: when
// there are more strips of 16 than compute units). The residual epilogue
// is not taken (the product of a norm is never added to the stream as it is).
extern "C" int liyab_gemm_skinny_ln(const float* planes, int n_planes, int64_t plane_stride, const float* ln_weight,
                                    const float* ln_bias, float eps, const void* w, int M, int N, int K, int wide,
                                    const EpiParams* epi_in, hipStream_t stream) {
    LIYAB_REQUIRE(planes && w && epi_in, "gemm_skinny_ln: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 32 && N > 0 && K > 0, "gemm_skinny_ln: bad sizes M=%d (at most 32) N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % 8 == 0 && K <= 2048, "gemm_skinny_ln: K %d must be a multiple of 8, at most 2048", K);
    LIYAB_REQUIRE(n_planes >= 1 && n_planes <= 16, "gemm_skinny_ln: %d planes (1 to 16)", n_planes);
    LIYAB_REQUIRE(n_planes == 1 || plane_stride >= static_cast<int64_t>(M) * K, "gemm_skinny_ln: planes of %lld floats overlap",
                  static_cast<long long>(plane_stride));
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    LIYAB_REQUIRE(al16(planes) && al16(w) && al16(ln_weight) && al16(ln_bias) && plane_stride % 4 == 0,
                  "gemm_skinny_ln: operands must be 16-byte aligned");
    LIYAB_REQUIRE(eps >= 0.0f, "gemm_skinny_ln: negative eps");
    EpiParams epi = *epi_in;
    LIYAB_REQUIRE(epi.mode != kEpiResidual, "gemm_skinny_ln: the residual epilogue is not taken");
    if (int rc = check_epilogue(epi, M, N)) return rc;
    if (M == 0) return 0;
    if (wide < 0) {
        static int units = 0;  // compute units of the device (one device a process)
        if (units == 0) {
            int dev = 0;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || units <= 0)
                units = 256;
        }
        wide = (N + 15) / 16 > units ? 1 : 0;
    }
    LIYAB_REQUIRE(!wide || M <= 16, "gemm_skinny_ln: strips of 32 output features go with at most 16 rows (%d)", M);
    const NormParams ln{planes, n_planes, plane_stride, ln_weight, ln_bias, eps};
    if (K <= 256) return launch_ln<1>(ln, w, M, N, K, wide, epi, stream);
    if (K <= 512) return launch_ln<2>(ln, w, M, N, K, wide, epi, stream);
    if (K <= 768) return launch_ln<3>(ln, w, M, N, K, wide, epi, stream);
    if (K <= 1024) return launch_ln<4>(ln, w, M, N, K, wide, epi, stream);
    return launch_ln<8>(ln, w, M, N, K, wide, epi, stream);
}
