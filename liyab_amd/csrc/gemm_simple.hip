// out[M,N] = a[M,K] . w[N,K]^T (+ bias) with an epilogue: the plain tiled
// product. It is the product of the true 32-bit path (32-bit operands, FMA
// accumulation, no matrix-core reduced precision) and the fallback for
// bfloat16 shapes the MFMA kernels refuse.
//
// Both operands are contiguous along K (a row of `w` is one output feature,
// as the reference lays matrices out: include/liyab/types.h:165-184,
// y = x . W^T in include/liyab/backend.h:35). Each output element is summed
// in one fixed order that does not depend on M, so a row's result is the same
// whatever else is in the batch (include/liyab/backend.h:40-42): K in chunks
// of 64; within a chunk one chain of fused multiply-adds over ascending k that
// starts from zero; the chunks' sums added in ascending order. (Chunks, so that
// a step of few rows, which has few output elements, can still spread one
// element's sum over several waves: gemm_rowwise_f32_kernel below.)
#include <type_traits>

#include "activations.h"
#include "common.h"
#include "launchers.h"

namespace liyab {

constexpr int BM = 64, BN = 64, BK = 16;
constexpr int kChunk = 64;  // k of one chain of multiply-adds
static_assert(kChunk % BK == 0, "a chunk is whole tiles");

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
    float acc[4][4] = {}, tot[4][4] = {};
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
        if ((k0 + BK) % kChunk == 0 || k0 + BK >= K) {  // the chunk's chain ends: its sum joins the others'
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    tot[i][j] += acc[i][j];
                    acc[i][j] = 0.0f;
                }
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
            float v = tot[i][j];
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

// The tiled kernel for large 32-bit products: tiles of 128 x 128, a thread 8 x 8 output elements (rows
// ty * 4 + {0..3} and 64 + the same, columns likewise), so that a step of k costs four 16-byte reads from
// LDS for 64 multiply-adds where the 64 x 64 tiles above read two for 16: there the reads set the pace
// (35 TFLOP/s). The chains and the order of sums are the ones above, bit for bit.
constexpr int BM2 = 128, BN2 = 128;

template <int EPI, bool EXACT>
__global__ void __launch_bounds__(256)
gemm_simple128_f32_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ a, int64_t lda, const float* __restrict__ w,
                          const float* __restrict__ bias, float* __restrict__ residual, int64_t ldr, int M, int N, int K) {
    __shared__ float As[BK][BM2 + 4];
    __shared__ float Ws[BK][BN2 + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * BM2, n0 = blockIdx.x * BN2;
    const int ty = tid / 16, tx = tid % 16;
    const int lrow = tid / 4, lk = (tid % 4) * 4;  // this thread loads 4 k of rows lrow and lrow + 64
    float acc[8][8] = {}, tot[8][8] = {};
    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int m = m0 + lrow + 64 * h, n = n0 + lrow + 64 * h;
            const float* p = a + static_cast<int64_t>(m) * lda + k0 + lk;
            const float* q = w + static_cast<int64_t>(n) * K + k0 + lk;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool in = k0 + lk + i < K;
                As[lk + i][lrow + 64 * h] = (m < M && in) ? p[i] : 0.0f;
                Ws[lk + i][lrow + 64 * h] = (n < N && in) ? q[i] : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float av[8], wv[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                av[i] = As[k][ty * 4 + i];
                av[4 + i] = As[k][64 + ty * 4 + i];
                wv[i] = Ws[k][tx * 4 + i];
                wv[4 + i] = Ws[k][64 + tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        if ((k0 + BK) % kChunk == 0 || k0 + BK >= K) {  // the chunk's chain ends: its sum joins the others'
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    tot[i][j] += acc[i][j];
                    acc[i][j] = 0.0f;
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int m = m0 + (i / 4) * 64 + ty * 4 + i % 4;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int n = n0 + (j / 4) * 64 + tx * 4 + j % 4;
            if (n >= N) continue;
            float v = tot[i][j];
            if (bias != nullptr) v += bias[n];
            if constexpr (EPI == kEpiGeluTanh) v = gelu_tanh(v);
            if constexpr (EPI == kEpiGeluErf) v = EXACT ? gelu_erf_exact(v) : gelu_erf_fast(v);
            if constexpr (EPI == kEpiResidual) {
                residual[static_cast<int64_t>(m) * ldr + n] += v;
            } else {
                out[static_cast<int64_t>(m) * ldo + n] = v;
            }
        }
    }
}

// The same product for steps of few rows (decoding), in the same order of sums, so a row's
// result has the same bits whichever of the two kernels computed it. A workgroup of four or
// eight waves takes NB output features and 16 rows (blockIdx.y: which 16); the chunks of K go round the waves. A wave
// brings its chunk of the NB rows of `w` and of the rows of `a` through registers into LDS of
// its own (256 bytes a row and load, the next chunk in flight meanwhile); lane (feature, row
// group) then runs the chunk's chain for its rows; after each round of chunks one thread
// an output element adds the round's sums in chunk order. Few features a workgroup where N is
// small: the weights then stream through enough compute units.
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int kRowwiseRows = 16;     // rows a workgroup
constexpr int kRowwiseMaxRows = 64;  // steps of at most this many rows take the row-wise kernel
constexpr int kTiled128MinTiles = 512;  // tiles of 128 x 128 from this many on: two a compute unit (288 of them, 2,048 x 2,304 x 768: 305 us against 222 in tiles of 64 x 64; 576, 4,096 rows: 349 against 440)
constexpr int kTiledMinTiles = 512;  // and so do larger ones that would give the tiled kernel fewer tiles than this

template <int NB, int WAVES, int EPI, bool EXACT>
__global__ void __launch_bounds__(64 * WAVES)
gemm_rowwise_f32_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ a, int64_t lda,
                        const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ residual,
                        int64_t ldr, int M_all, int N, int K) {
    const int row0 = blockIdx.y * kRowwiseRows, M = min(kRowwiseRows, M_all - row0);
    a += static_cast<int64_t>(row0) * lda;
    constexpr int LD = kChunk + 4;  // (rows 16 bytes apart in the banks: a lane's 16-byte reads do not collide)
    constexpr int MG = 64 / NB;                // row groups of lanes
    constexpr int RPL = kRowwiseRows / MG;     // rows a lane
    constexpr int W_LOADS = NB / 4, A_LOADS = kRowwiseRows / 4;  // a load covers 4 rows: 16 lanes a row, 16 bytes a lane
    static_assert(NB % 4 == 0 && 64 % NB == 0 && kRowwiseRows % MG == 0, "lanes are features x row groups");
    __shared__ float Wt[WAVES][NB][LD];
    __shared__ float At[WAVES][kRowwiseRows][LD];
    __shared__ float P[WAVES][kRowwiseRows][NB];
    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int n0 = blockIdx.x * NB;
    const int chunks = (K + kChunk - 1) / kChunk;
    const int lrow = lane / 16, lk = (lane % 16) * 4;  // as a loader
    const int fn = lane % NB, mg = lane / NB;          // as a summer
    f32x4_t wreg[W_LOADS], areg[A_LOADS];
    auto fetch = [&](int c) {  // chunk c into registers; past K zeros (they add nothing to a chain)
        const int k = c * kChunk + lk;
        const bool in = k < K;  // K is a multiple of 4 (the launcher's check): a lane's 4 are in or out together
        const int kc = in ? k : 0;
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int n = min(n0 + 4 * i + lrow, N - 1);
            const f32x4_t v = *reinterpret_cast<const f32x4_t*>(w + static_cast<int64_t>(n) * K + kc);
            wreg[i] = in ? v : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        }
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            if (4 * i < M) {  // (the same for every lane)
                const int m = min(4 * i + lrow, M - 1);
                const f32x4_t v = *reinterpret_cast<const f32x4_t*>(a + static_cast<int64_t>(m) * lda + kc);
                areg[i] = in ? v : f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    };
    float tot = 0.0f;  // of output element (tid / NB, tid % NB), for tid < 16 * NB
    if (wave < chunks) fetch(wave);
    for (int c0 = 0; c0 < chunks; c0 += WAVES) {
        const int c = c0 + wave;
        if (c < chunks) {
#pragma unroll
            for (int i = 0; i < W_LOADS; ++i) *reinterpret_cast<f32x4_t*>(&Wt[wave][4 * i + lrow][lk]) = wreg[i];
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i)
                if (4 * i < M) *reinterpret_cast<f32x4_t*>(&At[wave][4 * i + lrow][lk]) = areg[i];
            if (c + WAVES < chunks) fetch(c + WAVES);
            float part[RPL];
#pragma unroll
            for (int r = 0; r < RPL; ++r) part[r] = 0.0f;
#pragma unroll 4
            for (int kk = 0; kk < kChunk; kk += 4) {
                const f32x4_t wv = *reinterpret_cast<const f32x4_t*>(&Wt[wave][fn][kk]);
#pragma unroll
                for (int r = 0; r < RPL; ++r) {
                    const f32x4_t av = *reinterpret_cast<const f32x4_t*>(&At[wave][mg + r * MG][kk]);
                    part[r] = fmaf(av[0], wv[0], part[r]);
                    part[r] = fmaf(av[1], wv[1], part[r]);
                    part[r] = fmaf(av[2], wv[2], part[r]);
                    part[r] = fmaf(av[3], wv[3], part[r]);
                }
            }
#pragma unroll
            for (int r = 0; r < RPL; ++r) P[wave][mg + r * MG][fn] = part[r];
        }
        __syncthreads();
        if (tid < kRowwiseRows * NB) {
            const int live = min(WAVES, chunks - c0);
            for (int wv = 0; wv < live; ++wv) tot += P[wv][tid / NB][tid % NB];
        }
        __syncthreads();
    }
    const int n = n0 + tid % NB;
    if (tid >= kRowwiseRows * NB || tid / NB >= M || n >= N) return;
    const int m = row0 + tid / NB;
    float v = tot;
    if (bias != nullptr) v += bias[n];
    if constexpr (EPI == kEpiGeluTanh) v = gelu_tanh(v);
    if constexpr (EPI == kEpiGeluErf) v = EXACT ? gelu_erf_exact(v) : gelu_erf_fast(v);
    if constexpr (EPI == kEpiResidual) {
        residual[static_cast<int64_t>(m) * ldr + n] += v;
    } else {
        out[static_cast<int64_t>(m) * ldo + n] = v;
    }
}

// The same once more, one thread an output element, for operands that are not aligned to 16
// bytes or a K that is no multiple of 4.
template <int EPI, bool EXACT>
__global__ void __launch_bounds__(64)
gemm_rowwise_f32_plain_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ a, int64_t lda,
                              const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ residual,
                              int64_t ldr, int N, int K) {
    const int n = blockIdx.x * 64 + threadIdx.x, m = blockIdx.y;
    const float* wr = w + static_cast<int64_t>(min(n, N - 1)) * K;
    const float* ar = a + static_cast<int64_t>(m) * lda;
    float tot = 0.0f;
    for (int k0 = 0; k0 < K; k0 += kChunk) {
        float acc = 0.0f;
        const int k1 = min(k0 + kChunk, K);
        for (int k = k0; k < k1; ++k) acc = fmaf(ar[k], wr[k], acc);
        tot += acc;
    }
    if (n >= N) return;
    float v = tot;
    if (bias != nullptr) v += bias[n];
    if constexpr (EPI == kEpiGeluTanh) v = gelu_tanh(v);
    if constexpr (EPI == kEpiGeluErf) v = EXACT ? gelu_erf_exact(v) : gelu_erf_fast(v);
    if constexpr (EPI == kEpiResidual) {
        residual[static_cast<int64_t>(m) * ldr + n] += v;
    } else {
        out[static_cast<int64_t>(m) * ldo + n] = v;
    }
}

template <int EPI>
int launch_rowwise_f32_epi(float* out, int64_t ldo, const float* a, int64_t lda, const float* w, const float* bias,
                           float* residual, int64_t ldr, int M, int N, int K, hipStream_t stream) {
    const bool vec = (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && lda % 4 == 0 && K % 4 == 0;
    if (!vec) {
        gemm_rowwise_f32_plain_kernel<EPI, true><<<dim3((N + 63) / 64, M), 64, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, N, K);
        return check_launch("gemm_rowwise_plain");
    }
    // about two hundred workgroups or more: 4 features each up to 1,024 of them, 8 up to 2,560, 16 beyond
    const int row_blocks = (M + kRowwiseRows - 1) / kRowwiseRows;
    // (few features and a long K: eight waves share the chunks, twice as many loads in flight)
    if (N <= 1024 && K >= 2048) gemm_rowwise_f32_kernel<4, 8, EPI, true><<<dim3((N + 3) / 4, row_blocks), 512, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K);
    else if (N <= 1024) gemm_rowwise_f32_kernel<4, 4, EPI, true><<<dim3((N + 3) / 4, row_blocks), 256, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K);
    else if (N <= 2560) gemm_rowwise_f32_kernel<8, 4, EPI, true><<<dim3((N + 7) / 8, row_blocks), 256, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K);
    else gemm_rowwise_f32_kernel<16, 4, EPI, true><<<dim3((N + 15) / 16, row_blocks), 256, 0, stream>>>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K);
    return check_launch("gemm_rowwise");
}

int launch_rowwise_f32(float* out, int64_t ldo, const float* a, int64_t lda, const float* w, const float* bias,
                       float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream) {
    switch (epi) {
        case kEpiNone: return launch_rowwise_f32_epi<kEpiNone>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, stream);
        case kEpiGeluTanh: return launch_rowwise_f32_epi<kEpiGeluTanh>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, stream);
        case kEpiGeluErf: return launch_rowwise_f32_epi<kEpiGeluErf>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, stream);
        case kEpiResidual: return launch_rowwise_f32_epi<kEpiResidual>(out, ldo, a, lda, w, bias, residual, ldr, M, N, K, stream);
        default: return fail(1, "gemm: unknown epilogue %d", epi);
    }
}

template <typename T, typename OutT, bool EXACT>
int launch_simple(void* out, int64_t ldo, const void* a, int64_t lda, const void* w, const float* bias,
                  float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream) {
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    auto* o = static_cast<OutT*>(out);
    auto* pa = static_cast<const T*>(a);
    auto* pw = static_cast<const T*>(w);
    if constexpr (std::is_same<T, float>::value && std::is_same<OutT, float>::value) {
        // large 32-bit products in tiles of 128 x 128 once those are two a compute unit (45-57 TFLOP/s against 31-37)
        const dim3 grid2((N + BN2 - 1) / BN2, (M + BM2 - 1) / BM2);
        if (static_cast<int64_t>(grid2.x) * grid2.y >= kTiled128MinTiles) {
#define LIYAB_GO2(E) gemm_simple128_f32_kernel<E, EXACT><<<grid2, 256, 0, stream>>>(o, ldo, pa, lda, pw, bias, residual, ldr, M, N, K)
            switch (epi) {
                case kEpiNone: LIYAB_GO2(kEpiNone); break;
                case kEpiGeluTanh: LIYAB_GO2(kEpiGeluTanh); break;
                case kEpiGeluErf: LIYAB_GO2(kEpiGeluErf); break;
                case kEpiResidual: LIYAB_GO2(kEpiResidual); break;
                default: return fail(1, "gemm: unknown epilogue %d", epi);
            }
#undef LIYAB_GO2
            return check_launch("gemm_simple128");
        }
    }
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
        // more rows than that take the tiled kernel once its tiles of 64 x 64 are two workgroups for every
        // compute unit (measured: from there it passes the row-wise kernel's steady 21 TFLOP/s); with fewer tiles
        // the row-wise kernel's many small workgroups are faster, if its
        // loads of 16 bytes fit the operands (else it would run one thread an element)
        const bool vec = (reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0 && lda % 4 == 0 && K % 4 == 0;
        const int64_t tiles = static_cast<int64_t>((N + BN - 1) / BN) * ((M + BM - 1) / BM);
        if (M <= kRowwiseMaxRows || (vec && tiles < kTiledMinTiles))
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
