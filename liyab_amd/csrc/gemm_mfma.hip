// out[M,N] = a[M,K] . w[N,K]^T in bfloat16 on the matrix cores, for steps of
// many tokens (prompt portions).
//
// Both operands are contiguous along K, which is the layout MFMA wants: for
// v_mfma_f32_32x32x16_bf16 a lane holds 8 consecutive k of one row (of `a`)
// or one output feature (of `w`), 16 bytes, so tiles go global -> LDS ->
// registers in 16-byte pieces with no transposition. A workgroup of 4 waves
// (2 x 2) computes a BM x BN tile; each wave owns (BM/2) x (BN/2) as 32 x 32
// blocks with 32-bit accumulators. Tiles of K (BK = 64) are double-buffered
// in LDS, rows padded by 16 bytes so that the 16-byte reads of 16 lanes fall
// in distinct banks. Partial tiles are zero-filled on load and masked on
// store; K must be a multiple of 8 (16-byte pieces). Each output element is
// a fixed-order sum over k, independent of M.
#include "common.h"
#include "launchers.h"
#include "epilogue.h"

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int GBK = 64;          // k per LDS tile
constexpr int GLD = GBK + 8;     // padded row, in elements

template <int BM, int BN, typename OutT>
__global__ void __launch_bounds__(256)
gemm_mfma_kernel(const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int M, int N, int K,
                 EpiParams epi) {
    constexpr int TM = BM / 64, TN = BN / 64;  // 32x32 blocks per wave in each direction
    constexpr int A_CHUNKS = BM * GBK / 8 / 256, W_CHUNKS = BN * GBK / 8 / 256;
    extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
    constexpr int STAGE = (BM + BN) * GLD;  // a stage holds the tile of `a`, then the tile of `w`

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wm = wave / 2, wn = wave % 2;
    // Workgroups go to the 8 XCDs round-robin, each XCD with an L2 of its own. Tile t of the
    // row-major tile order goes to the XCD that holds the tiles around it, so that an XCD's
    // tiles share a few row blocks of `a` and its L2 holds them beside all of `w`.
    const int tiles_n = (N + BN - 1) / BN, n_tiles = tiles_n * ((M + BM - 1) / BM);
    const int xcd = blockIdx.x % 8, base = n_tiles / 8, rem = n_tiles % 8;
    const int tile_id = xcd * base + min(xcd, rem) + blockIdx.x / 8;
    const int m0 = (tile_id / tiles_n) * BM, n0 = (tile_id % tiles_n) * BN;
    const int li = lane % 32, lk = (lane / 32) * 8;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 ra[A_CHUNKS], rw[W_CHUNKS];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i, row = c / (GBK / 8), kc = (c % (GBK / 8)) * 8;
            const int m = m0 + row, k = k0 + kc;
            ra[i] = (m < M && k < K) ? *reinterpret_cast<const u32x4*>(a + static_cast<int64_t>(m) * lda + k) : u32x4{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i, row = c / (GBK / 8), kc = (c % (GBK / 8)) * 8;
            const int n = n0 + row, k = k0 + kc;
            rw[i] = (n < N && k < K) ? *reinterpret_cast<const u32x4*>(w + static_cast<int64_t>(n) * K + k) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i) {
            const int c = tid + 256 * i, row = c / (GBK / 8), kc = (c % (GBK / 8)) * 8;
            *reinterpret_cast<u32x4*>(lds + buf * STAGE + row * GLD + kc) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < W_CHUNKS; ++i) {
            const int c = tid + 256 * i, row = c / (GBK / 8), kc = (c % (GBK / 8)) * 8;
            *reinterpret_cast<u32x4*>(lds + buf * STAGE + (BM + row) * GLD + kc) = rw[i];
        }
    };

    const int nk = (K + GBK - 1) / GBK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * GBK);
        const bf16_t* Ab = lds + buf * STAGE + (wm * (BM / 2) + li) * GLD + lk;
        const bf16_t* Wb = lds + buf * STAGE + (BM + wn * (BN / 2) + li) * GLD + lk;
#pragma unroll
        for (int ks = 0; ks < GBK; ks += 16) {
            bf16x8 fa[TM], fw[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const bf16x8*>(Ab + i * 32 * GLD + ks);
#pragma unroll
            for (int j = 0; j < TN; ++j) fw[j] = *reinterpret_cast<const bf16x8*>(Wb + j * 32 * GLD + ks);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            store_lds(buf ^ 1);  // the other buffer was last read before the previous barrier
            __syncthreads();
        }
    }
    // C block layout: lane holds column li; rows 8 * (r / 4) + 4 * (lane / 32) + r % 4
    // tiles wholly inside the output skip the per-element bounds checks (a guarded store is a
    // branch of its own: on an interior tile they cost as much as the whole product)
    const bool inside = m0 + BM <= M && n0 + BN <= N;
    if (epi.mode == kEpiQkvPaged) {
        // keys and values go to their pages: the rows' page places first, then the stores
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int mb = m0 + wm * (BM / 2) + i * 32 + 4 * (lane / 32);
            int64_t row_base[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) row_base[r] = qkv_row_base(epi, min(mb + 8 * (r / 4) + r % 4, M - 1));
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = n0 + wn * (BN / 2) + j * 32 + li;
                if (n >= N) continue;
                const float bias_n = epilogue_bias(epi, n);
                const int64_t col = qkv_col_offset(epi, n);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = mb + 8 * (r / 4) + r % 4;
                    if (inside || m < M) qkv_store<OutT>(epi, m, n, row_base[r], col, acc[i][j][r] + bias_n);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn * (BN / 2) + j * 32 + li;
            const int mb = m0 + wm * (BM / 2) + i * 32 + 4 * (lane / 32);
            const float bias_n = n < N ? epilogue_bias(epi, n) : 0.0f;
            if (inside) {
#pragma unroll
                for (int r = 0; r < 16; ++r) epilogue_store_biased<OutT, -1>(epi, mb + 8 * (r / 4) + r % 4, n, acc[i][j][r] + bias_n);
            } else if (n < N) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = mb + 8 * (r / 4) + r % 4;
                    if (m < M) epilogue_store_biased<OutT, -1>(epi, m, n, acc[i][j][r] + bias_n);
                }
            }
        }
}

template <int BM, int BN>
int launch_mfma(const void* a, int64_t lda, const void* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    dim3 grid(((N + BN - 1) / BN) * ((M + BM - 1) / BM));
    const size_t smem = 2 * static_cast<size_t>(BM + BN) * GLD * sizeof(bf16_t);
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (epi.mode == kEpiResidual || epi.out_dtype == kF32) {
        auto kern = gemm_mfma_kernel<BM, BN, float>;
        static bool ready = false;  // once per instantiation, outside any stream capture's first use
        if (!ready) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
            ready = true;
        }
        kern<<<grid, 256, smem, stream>>>(pa, lda, pw, M, N, K, epi);
    } else {
        auto kern = gemm_mfma_kernel<BM, BN, bf16_t>;
        static bool ready = false;
        if (!ready) {
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
            ready = true;
        }
        kern<<<grid, 256, smem, stream>>>(pa, lda, pw, M, N, K, epi);
    }
    return check_launch("gemm_mfma");
}

}  // namespace liyab

using namespace liyab;

// a [M, K] (row stride lda) and w [N, K] are bfloat16; the epilogue says where results go.
// tile: 0 = chosen from the shape, 1 = 128x128, 2 = 64x64, 3 = 128x64.
extern "C" int liyab_gemm_mfma(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile,
                               const EpiParams* epi_in, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && epi_in, "gemm: null operand");
    LIYAB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % 8 == 0 && lda % 8 == 0 && lda >= K, "gemm_mfma: K %d and lda %lld must be multiples of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_mfma: operands must be 16-byte aligned");
    EpiParams epi = *epi_in;
    if (int rc = check_epilogue(epi, M, N)) return rc;
    if (M == 0) return 0;
    if (tile == 0) {
        // measured at 2048 x {768, 2304, 3072} x {768, 3072}: 64 x 64 tiles (4 workgroups a CU,
        // many tiles) beat 128 x 128 (2 a CU, a ragged second round) until there are thousands of tiles
        const long big = static_cast<long>((M + 127) / 128) * ((N + 127) / 128);
        tile = big >= 2048 ? 1 : 2;
    }
    switch (tile) {
        case 1: return launch_mfma<128, 128>(a, lda, w, M, N, K, epi, stream);
        case 2: return launch_mfma<64, 64>(a, lda, w, M, N, K, epi, stream);
        case 3: return launch_mfma<128, 64>(a, lda, w, M, N, K, epi, stream);
        default: return fail(1, "gemm_mfma: unknown tile %d", tile);
    }
}
