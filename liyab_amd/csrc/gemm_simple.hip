// out[M,N] = a[M,K] . w[N,K]^T (+ bias) with an epilogue: the plain tiled
// product. It is the product of the true 32-bit path (32-bit operands, FMA
// accumulation, no matrix-core reduced precision) and the fallback for
// bfloat16 shapes the MFMA kernels refuse.
//
// Both operands are contiguous along K (a row of `w` is one output feature,
// as the reference lays matrices out: include/liyab/types.h:165-184,
// y = x . W^T in include/liyab/backend.h:35). Each output element is one
// sequential sum over k = 0..K-1 in a fixed order that does not depend on M,
// so a row's result is the same whatever else is in the batch
// (include/liyab/backend.h:40-42).
#include "activations.h"
#include "common.h"

namespace liyab {

constexpr int BM = 64, BN = 64, BK = 16;

template <typename T, typename OutT, int EPI, bool EXACT>
__global__ void __launch_bounds__(256)
gemm_simple_kernel(OutT* __restrict__ out, int64_t ldo, const T* __restrict__ a, int64_t lda, const T* __restrict__ w,
                   const float* __restrict__ bias, float* __restrict__ residual, int64_t ldr, int M, int N, int K) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int ty = tid / 16, tx = tid % 16;
    const int lrow = tid / 4, lk = (tid % 4) * 4;  // this thread loads 4 k of one row
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
        {
            const int m = m0 + lrow;
            const T* p = a + static_cast<int64_t>(m) * lda + k0 + lk;
#pragma unroll
            for (int i = 0; i < 4; ++i) As[lk + i][lrow] = (m < M && k0 + lk + i < K) ? to_float<T>(p[i]) : 0.0f;
            const int n = n0 + lrow;
            const T* q = w + static_cast<int64_t>(n) * K + k0 + lk;
#pragma unroll
            for (int i = 0; i < 4; ++i) Ws[lk + i][lrow] = (n < N && k0 + lk + i < K) ? to_float<T>(q[i]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float v = acc[i][j];
            if (bias != nullptr) v += bias[n];
            if constexpr (EPI == kEpiGeluTanh) v = gelu_tanh(v);
            if constexpr (EPI == kEpiGeluErf) v = EXACT ? gelu_erf_exact(v) : gelu_erf_fast(v);
            if constexpr (EPI == kEpiResidual) {
                residual[static_cast<int64_t>(m) * ldr + n] += v;
            } else {
                out[static_cast<int64_t>(m) * ldo + n] = from_float<OutT>(v);
            }
        }
    }
}

// The same product for steps of few rows (decoding): a thread per output element walks K in
// the same order with the same fused multiply-adds as the tiled kernel, so a row's result has
// the same bits whichever of the two computed it. A wave takes 64 output features of one row;
// rows of `w` are streamed 16 bytes a lane, the row of `a` through scalar loads.
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

template <int EPI, bool EXACT>
__global__ void __launch_bounds__(64)
gemm_rowwise_f32_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ a, int64_t lda,
                        const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ residual,
                        int64_t ldr, int N, int K, int vec) {
    const int n = blockIdx.x * 64 + threadIdx.x, m = blockIdx.y;
    const float* wr = w + static_cast<int64_t>(min(n, N - 1)) * K;
    const float* ar = a + static_cast<int64_t>(m) * lda;
    float acc = 0.0f;
    int k = 0;
    if (vec) {
#pragma unroll 8
        for (; k + 4 <= K; k += 4) {
            const f32x4_t wv = *reinterpret_cast<const f32x4_t*>(wr + k);
            const f32x4_t av = *reinterpret_cast<const f32x4_t*>(ar + k);
            acc = fmaf(av[0], wv[0], acc);
            acc = fmaf(av[1], wv[1], acc);
            acc = fmaf(av[2], wv[2], acc);
            acc = fmaf(av[3], wv[3], acc);
        }
    }
    for (; k < K; ++k) acc = fmaf(ar[k], wr[k], acc);
    if (n >= N) return;
    float v = acc;
    if (bias != nullptr) v += bias[n];
    if constexpr (EPI == kEpiGeluTanh) v = gelu_tanh(v);
    if constexpr (EPI == kEpiGeluErf) v = EXACT ? gelu_erf_exact(v) : gelu_erf_fast(v);
    if constexpr (EPI == kEpiResidual) {
        residual[static_cast<int64_t>(m) * ldr + n] += v;
    } else {
        out[static_cast<int64_t>(m) * ldo + n] = v;
    }
}

constexpr int kRowwiseRows = 16;  // steps of at most this many rows take the row-wise kernel

int launch_rowwise_f32(float* out, int64_t ldo, const float* a, int64_t lda, const float* w, const float* bias,
                       float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream) {
    const dim3 grid((N + 63) / 64, M);
    const int vec = (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && lda % 4 == 0 && K % 4 == 0;
#define LIYAB_GO(E) gemm_rowwise_f32_kernel<E, true><<<grid, 64, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, N, K, vec)
    switch (epi) {
        case kEpiNone: LIYAB_GO(kEpiNone); break;
        case kEpiGeluTanh: LIYAB_GO(kEpiGeluTanh); break;
        case kEpiGeluErf: LIYAB_GO(kEpiGeluErf); break;
        case kEpiResidual: LIYAB_GO(kEpiResidual); break;
        default: return fail(1, "gemm: unknown epilogue %d", epi);
    }
#undef LIYAB_GO
    return check_launch("gemm_rowwise");
}

template <typename T, typename OutT, bool EXACT>
int launch_simple(void* out, int64_t ldo, const void* a, int64_t lda, const void* w, const float* bias,
                  float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream) {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    auto* o = static_cast<OutT*>(out);
    auto* pa = static_cast<const T*>(a);
    auto* pw = static_cast<const T*>(w);
#define LIYAB_GO(E) \
    gemm_simple_kernel<T, OutT, E, EXACT><<<grid, 256, 0, stream>>>(o, ldo, pa, lda, pw, bias, residual, ldr, M, N, K)
    switch (epi) {
        case kEpiNone: LIYAB_GO(kEpiNone); break;
        case kEpiGeluTanh: LIYAB_GO(kEpiGeluTanh); break;
        case kEpiGeluErf: LIYAB_GO(kEpiGeluErf); break;
        case kEpiResidual: LIYAB_GO(kEpiResidual); break;
        default: return fail(1, "gemm: unknown epilogue %d", epi);
    }
#undef LIYAB_GO
    return check_launch("gemm_simple");
}

}  // namespace liyab

using namespace liyab;

// dtype: element type of `a` and `w`; out_dtype: of `out` (ignored for the
// residual epilogue, which adds into `residual`, 32-bit, row stride ldr).
extern "C" int liyab_gemm_simple(void* out, int out_dtype, int64_t ldo, const void* a, int64_t lda, const void* w,
                                 int dtype, const float* bias, float* residual, int64_t ldr, int M, int N, int K,
                                 int epi, hipStream_t stream) {
    LIYAB_REQUIRE(a && w, "gemm: null operand");
    LIYAB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(lda >= K, "gemm: lda %lld < K %d", static_cast<long long>(lda), K);
    if (epi == kEpiResidual) {
        LIYAB_REQUIRE(residual != nullptr && ldr >= N, "gemm: the residual epilogue needs a residual of row stride >= N");
    } else {
        LIYAB_REQUIRE(out != nullptr && ldo >= N, "gemm: needs an output of row stride >= N");
    }
    if (M == 0) return 0;
    if (dtype == kF32) {
        LIYAB_REQUIRE(epi == kEpiResidual || out_dtype == kF32, "gemm: 32-bit operands give a 32-bit output");
        if (M <= kRowwiseRows)
            return launch_rowwise_f32(static_cast<float*>(out), ldo, static_cast<const float*>(a), lda, static_cast<const float*>(w),
                                      bias, residual, ldr, M, N, K, epi, stream);
        return launch_simple<float, float, true>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, epi, stream);
    }
    if (dtype == kBF16) {
        if (out_dtype == kF32) return launch_simple<bf16_t, float, false>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, epi, stream);
        if (out_dtype == kBF16) return launch_simple<bf16_t, bf16_t, false>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, epi, stream);
        return fail(1, "gemm: unknown output dtype %d", out_dtype);
    }
    return fail(1, "gemm: unknown dtype %d", dtype);
}
