// out[M,N] = a[M,K] . w[N,K]^T in bfloat16 for steps of few tokens (M <= 16):
// decoding, where the product is a stream of the weights.
//
// A workgroup owns 16 output features (16 rows of `w`) and all M tokens; its
// waves split K and add their partial sums through LDS in wave order. With
// v_mfma_f32_16x16x32_bf16 the weights are the first operand (16 rows) and
// the tokens the second (up to 16), so the accumulator is the transposed
// output tile. A lane holds 8 consecutive k of its row per instruction; here
// each lane reads a run of 16 consecutive k (32 bytes) and feeds two
// instructions, and both operands use the same assignment of k to (lane
// group, instruction), which a dot product does not mind. Weights are read
// once, straight from global memory into registers, 16 bytes a lane; the
// tokens' rows come from L2. K must be a multiple of 8. The order of the sum
// depends on K and the split only, never on M.
#include "common.h"
#include "epilogue.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float floatx4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

template <typename OutT, int KSPLIT>
__global__ void __launch_bounds__(64 * KSPLIT)
gemm_skinny_kernel(const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int M, int N, int K,
                   EpiParams epi) {
    __shared__ float red[KSPLIT][256];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int i = lane % 16, g = lane / 16;
    const int n0 = blockIdx.x * 16;
    const bf16_t* wrow = w + static_cast<int64_t>(min(n0 + i, N - 1)) * K;
    const bf16_t* arow = a + static_cast<int64_t>(min(i, M - 1)) * lda;
    floatx4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const int units = (K + 63) / 64;
    const u32x4 zero = {0, 0, 0, 0};
    int u = wave;
    // two units per trip: eight 16-byte loads in flight per lane
    for (; u + KSPLIT < units; u += 2 * KSPLIT) {
        const int k0 = u * 64 + g * 16, k1 = (u + KSPLIT) * 64 + g * 16;
        Frag w0, w1, w2, w3, x0, x1, x2, x3;
        w0.u = *reinterpret_cast<const u32x4*>(wrow + k0);
        w1.u = *reinterpret_cast<const u32x4*>(wrow + k0 + 8);
        w2.u = k1 < K ? *reinterpret_cast<const u32x4*>(wrow + k1) : zero;
        w3.u = k1 + 8 < K ? *reinterpret_cast<const u32x4*>(wrow + k1 + 8) : zero;
        x0.u = *reinterpret_cast<const u32x4*>(arow + k0);
        x1.u = *reinterpret_cast<const u32x4*>(arow + k0 + 8);
        x2.u = k1 < K ? *reinterpret_cast<const u32x4*>(arow + k1) : zero;
        x3.u = k1 + 8 < K ? *reinterpret_cast<const u32x4*>(arow + k1 + 8) : zero;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0.v, x0.v, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1.v, x1.v, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w2.v, x2.v, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w3.v, x3.v, acc, 0, 0, 0);
    }
    for (; u < units; u += KSPLIT) {
        const int k0 = u * 64 + g * 16;
        Frag w0, w1, x0, x1;
        w0.u = k0 < K ? *reinterpret_cast<const u32x4*>(wrow + k0) : zero;
        w1.u = k0 + 8 < K ? *reinterpret_cast<const u32x4*>(wrow + k0 + 8) : zero;
        x0.u = k0 < K ? *reinterpret_cast<const u32x4*>(arow + k0) : zero;
        x1.u = k0 + 8 < K ? *reinterpret_cast<const u32x4*>(arow + k0 + 8) : zero;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0.v, x0.v, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1.v, x1.v, acc, 0, 0, 0);
    }
    // acc[r] = partial C^T[n = 4 g + r][m = i]
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][i * 16 + 4 * g + r] = acc[r];  // [m][n]
    __syncthreads();
    for (int t = tid; t < 256; t += 64 * KSPLIT) {
        const int m = t / 16, n = n0 + t % 16;
        float v = 0.0f;
#pragma unroll
        for (int s = 0; s < KSPLIT; ++s) v += red[s][t];
        if (m < M && n < N) epilogue_store<OutT>(epi, m, n, v);
    }
}

template <int KSPLIT>
int launch_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    const int grid = (N + 15) / 16;
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (epi.mode == kEpiResidual || epi.out_dtype == kF32) {
        gemm_skinny_kernel<float, KSPLIT><<<grid, 64 * KSPLIT, 0, stream>>>(pa, lda, pw, M, N, K, epi);
    } else {
        gemm_skinny_kernel<bf16_t, KSPLIT><<<grid, 64 * KSPLIT, 0, stream>>>(pa, lda, pw, M, N, K, epi);
    }
    return check_launch("gemm_skinny");
}

}  // namespace liyab

using namespace liyab;

// a [M <= 16, K] and w [N, K] are bfloat16. ksplit: waves per workgroup sharing K (0 = chosen
// from the shape; 1, 2, 4, 8 or 16).
extern "C" int liyab_gemm_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit,
                                 const EpiParams* epi_in, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && epi_in, "gemm: null operand");
    LIYAB_REQUIRE(M >= 0 && M <= 16 && N > 0 && K > 0, "gemm_skinny: bad sizes M=%d (at most 16) N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % 8 == 0 && lda % 8 == 0 && lda >= K, "gemm_skinny: K %d and lda %lld must be multiples of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_skinny: operands must be 16-byte aligned");
    EpiParams epi = *epi_in;
    if (int rc = check_epilogue(epi, M, N)) return rc;
    if (M == 0) return 0;
    if (ksplit == 0) {
        // enough waves to cover the chip several times over, each with at least 128 k
        const int tiles = (N + 15) / 16, units = (K + 63) / 64;
        ksplit = 1;
        while (ksplit < 16 && tiles * ksplit < 2048 && units / (ksplit * 2) >= 2) ksplit *= 2;
    }
    switch (ksplit) {
        case 1: return launch_skinny<1>(a, lda, w, M, N, K, epi, stream);
        case 2: return launch_skinny<2>(a, lda, w, M, N, K, epi, stream);
        case 4: return launch_skinny<4>(a, lda, w, M, N, K, epi, stream);
        case 8: return launch_skinny<8>(a, lda, w, M, N, K, epi, stream);
        case 16: return launch_skinny<16>(a, lda, w, M, N, K, epi, stream);
        default: return fail(1, "gemm_skinny: ksplit %d is not 1, 2, 4, 8 or 16", ksplit);
    }
}
