// out[M,N] = a[M,K] . w[N,K]^T in bfloat16 on the matrix cores, with tiles
// brought from global memory straight into LDS (global_load_lds, 16 bytes a
// lane) in a ring of three stages, so that two tiles of K are in flight
// while one is multiplied. For steps of many tokens; K must be a multiple of
// 64 (other shapes go to the register-staged kernel in gemm_mfma.hip).
//
// A wave's direct load fills 1 KiB of LDS contiguously, lane after lane: 8
// rows of 64 k. Rows are therefore unpadded (128 bytes), and bank conflicts
// of the 16-byte fragment reads are avoided by a swizzle: within a row, the
// 16-byte piece c sits at position c ^ swizzle(row), applied on the
// global side when loading and again when reading. Rows past M or N are
// clamped to the last valid row; their results are never stored. MFMA
// operand layout and the fixed-order sum over k are those of gemm_mfma.hip.
//
// The product may be cut over K into parts (blockIdx.y), one plane of 32-bit
// sums a part, the first plane also taking the bias and the rows the product
// is added to (themselves a sum of planes): the planes together are then the
// residual stream after the product, as the streaming kernel of few rows
// leaves it (gemm_skinny.hip). A product with few output tiles and a long K
// covers the chip that way.
#include "common.h"
#include "launchers.h"
#include "epilogue.h"

#include <type_traits>

namespace liyab {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float floatx16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((address_space(3))) void* lds_void_ptr;

// Four consecutive outputs in one store (16 bytes of float32, 8 of bfloat16).
template <typename OutT>
__device__ __forceinline__ void store4(OutT* dst, const f32x4& v);
template <>
__device__ __forceinline__ void store4<float>(float* dst, const f32x4& v) { *reinterpret_cast<f32x4*>(dst) = v; }
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* dst, const f32x4& v) {
    uint2 packed;
    packed.x = static_cast<uint32_t>(float_to_bf16(v[0])) | (static_cast<uint32_t>(float_to_bf16(v[1])) << 16);
    packed.y = static_cast<uint32_t>(float_to_bf16(v[2])) | (static_cast<uint32_t>(float_to_bf16(v[3])) << 16);
    *reinterpret_cast<uint2*>(dst) = packed;
}

constexpr int DBK = 64;      // k per stage
constexpr int kEpiParts = 5;  // this file's own epilogue: a plane of sums a part of K

// A product cut over K: tiles of K a part, floats between the planes, and what the first plane adds.
struct PartsParams {
    int kt_per_part;
    int64_t part_stride;
    const float* base;  // rows the product is added to, a sum of n_base planes [M, N]; or null
    int n_base;
    int64_t base_stride;
};

// Where a row's 16-byte pieces sit within the row. LDS has 64 banks of 4 bytes: a 16-byte read
// serves 16 lanes a cycle, which read 16 consecutive rows at one piece index. Rows are 128 bytes,
// so even and odd rows start in different halves of the banks; within a half, 8 rows must land on
// 8 different pieces: the piece index is XORed with (row / 2) % 8.
__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }

// Dynamic LDS of a workgroup: the operand stages, or, where bfloat16 outputs leave through LDS as whole
// rows, the waves' padded output tiles if those take more (tiles of 256 x 256: 144 KB against 128).
template <int BM, int BN, int DSTAGES, int WM, int WN, int WK>
constexpr size_t dl_lds_bytes(size_t out_bytes) {
    const size_t stages = static_cast<size_t>(DSTAGES) * WK * (BM + BN) * 64 * 2;
    const size_t staging = out_bytes == 2 ? static_cast<size_t>(WM * WN * WK) * (BM / WM) * (BN / WN + 8) * 2 : 0;
    return stages > staging ? stages : staging;
}

template <int BM, int BN, int DSTAGES, typename OutT, int EPI, int WM = 2, int WN = 2, int WK = 1, int SETS = 1>
__global__ void __launch_bounds__(64 * WM * WN * WK)
gemm_mfma_dl_kernel(const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int M, int N, int K,
                    EpiParams epi, int vec_ok, int page_shift, PartsParams parts) {
    // WK groups of WM x WN waves, each wave with (BM / WM) x (BN / WN) of the tile in blocks of 32 x 32.
    // A stage holds WK consecutive units of 64 k, one a group: the groups walk K side by side (a
    // tile of few rows has few products a unit, and its walk is a chain of waits: load, barrier,
    // fragments, products; WK of them run at once), and their sums are added at the end in the
    // groups' order. SETS (with WK = 1): the one group keeps SETS sums, unit u of 64 k going to sum
    // u % SETS, added at the end in the sums' order: what WK = SETS groups would have left, bit
    // for bit, so that a row has one result in tiles of every shape (the batch-invariant mode).
    static_assert(SETS == 1 || (WK == 1 && SETS == 4), "sums by unit are for one group of waves, four of them");
    constexpr int GROUP = WM * WN, WAVES = GROUP * WK, TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int UNIT = (BM + BN) * DBK;       // elements of one unit of 64 k: the tile of a, then the tile of w
    constexpr int STAGE = WK * UNIT;            // elements per stage
    constexpr int A_LOADS = BM / 8 / GROUP, W_LOADS = BN / 8 / GROUP;  // wave-loads (8 rows each) per wave and stage
    static_assert(TM >= 1 && TN >= 1 && A_LOADS >= 1 && W_LOADS >= 1, "tile too small for its waves");
    extern __shared__ __attribute__((aligned(1024))) bf16_t lds[];

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
    const int wk = wave / GROUP, wg = wave % GROUP;
    const int wm = wg / WN, wn = wg % WN;
    // Workgroups go to the 8 XCDs round-robin, each XCD with an L2 of its own. Tile t of the
    // row-major tile order goes to the XCD that holds the tiles around it, so that an XCD's
    // tiles share a few row blocks of `a` and its L2 holds them beside all of `w`.
    // An XCD takes a stretch of the row-major tile order: a band of rows. While `w` is small that is
    // the best order: the XCD reads `w` once, and its rows of `a` are what its own workgroups of the
    // product before wrote (a prefill step's products all run over the same bands of tokens, so an
    // XCD's activations stay in its L2). With a large `w` the workgroups that run side by side on an
    // XCD, one row of tiles and all of `w`'s columns, share nothing of `w`, and every row of tiles
    // reads all of it again from memory (4,096 x 4,096 x 16,384 in 128 x 128 tiles: 3.9 GB of L2
    // misses for 0.27 GB of operands, at the memory's own speed): there the XCD's stretch goes in
    // groups of GM rows of tiles, down the rows first, so that its workgroups form a block of GM
    // rows by a few columns (half the misses; 721 -> 611 us). The bound between the two, 12 MB of
    // `w`: GPT-2 small's prefill of 2,048 tokens is 6 % slower in groups (its second feed-forward
    // product 24.2 -> 28.9 us), XL's of 8,192 tokens 6 % faster, width 4,096's 6 %.
    const int tiles_n = (N + BN - 1) / BN, tiles_m = (M + BM - 1) / BM, n_tiles = tiles_n * tiles_m;
    const int xcd = blockIdx.x % 8, base = n_tiles / 8, rem = n_tiles % 8;
    const int tile_id = xcd * base + min(xcd, rem) + blockIdx.x / 8;
    constexpr int GM = BM >= 128 ? 4 : 8;
    const bool groups = static_cast<int64_t>(N) * K > (6 << 20);
    const int per_group = groups ? GM * tiles_n : tiles_n;  // (plain rows: groups of one row of tiles)
    const int group = tile_id / per_group, first_m = group * (groups ? GM : 1), in_group = tile_id - group * per_group;
    const int gm = groups ? min(GM, tiles_m - first_m) : 1;
    int m0 = (first_m + in_group % gm) * BM;
    const int n0 = (in_group / gm) * BN;
    const int li = lane % 32, g = lane / 32;

    // this lane's part in a wave-load: row lane / 8 of the 8, LDS piece position lane % 8
    const int lrow = lane / 8, lpos = lane % 8;
    // a group's waves load their group's unit of the stage; a unit past the end of K is the last
    // one again (loaded and not multiplied: every wave asks for as many loads a stage as the
    // waits below count on)
    int units = K / DBK;  // units of 64 k this workgroup walks
    auto issue = [&](int kt, int stage) {
        const int k0 = min(kt * WK + wk, units - 1) * DBK;
        bf16_t* sa = lds + stage * STAGE + wk * UNIT;
        bf16_t* sw = sa + BM * DBK;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int r0 = (wg * A_LOADS + i) * 8, row = r0 + lrow;
            const int c = lpos ^ swizzle(row);
            const bf16_t* src = a + static_cast<int64_t>(min(m0 + row, M - 1)) * lda + k0 + c * 8;
            __builtin_amdgcn_global_load_lds(src, (lds_void_ptr)(sa + r0 * DBK), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < W_LOADS; ++i) {
            const int r0 = (wg * W_LOADS + i) * 8, row = r0 + lrow;
            const int c = lpos ^ swizzle(row);
            const bf16_t* src = w + static_cast<int64_t>(min(n0 + row, N - 1)) * K + k0 + c * 8;
            __builtin_amdgcn_global_load_lds(src, (lds_void_ptr)(sw + r0 * DBK), 16, 0, 0);
        }
    };

    floatx16 sums[SETS][TM][TN];
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) sums[s][i][j][r] = 0.0f;

    if constexpr (EPI == kEpiParts) {
        // this workgroup's part of K: units [kt0, kt0 + units)
        const int kt0 = blockIdx.y * parts.kt_per_part;
        units = min(units - kt0, parts.kt_per_part);
        a += static_cast<int64_t>(kt0) * DBK;
        w += static_cast<int64_t>(kt0) * DBK;
        if (blockIdx.y > 0) epi.bias = nullptr;  // the bias goes to the first plane only
    }
    const int nk = (units + WK - 1) / WK;  // stages walked
    constexpr int AHEAD = DSTAGES - 1;  // tiles of K in flight or in use beside the one being multiplied
#pragma unroll
    for (int p = 0; p < AHEAD; ++p)
        if (p < nk) issue(p, p);
    auto step = [&](int kt, auto set) {
        floatx16 (&acc)[TM][TN] = sums[decltype(set)::value];
        // tile kt must have landed: the loads of the tiles after it may still be in flight (a
        // wave's loads complete in order, A_LOADS + W_LOADS a tile)
        const int later = min(nk - 1 - kt, AHEAD - 1);
        constexpr int PER_TILE = A_LOADS + W_LOADS;
        static_assert((AHEAD - 1) * PER_TILE <= 63, "the counter of loads in flight has six bits");
        if (later >= 7) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD > 7 ? 7 * PER_TILE : 0) : "memory");
        else if (later == 6) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD > 6 ? 6 * PER_TILE : 0) : "memory");
        else if (later == 5) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD > 5 ? 5 * PER_TILE : 0) : "memory");
        else if (later == 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD > 4 ? 4 * PER_TILE : 0) : "memory");
        else if (later == 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD > 3 ? 3 * PER_TILE : 0) : "memory");
        else if (later == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (A_LOADS + W_LOADS)) : "memory");
        else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(A_LOADS + W_LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        // everyone's loads of tile kt are in LDS; everyone is done reading tile kt - 1. A bare
        // barrier: __syncthreads() would also wait for the loads still meant to be in flight.
        __builtin_amdgcn_s_barrier();
        if (kt + AHEAD < nk) issue(kt + AHEAD, (kt + AHEAD) % DSTAGES);  // into the stage tile kt - 1 used
        const bf16_t* sa = lds + (kt % DSTAGES) * STAGE + wk * UNIT;
        const bf16_t* sw = sa + BM * DBK;
        if (WK > 1 && kt * WK + wk >= units) return;  // this group's unit is past the end of K (the last stage only)
        // fragments of slab ks + 1 are read from LDS while slab ks multiplies
        bf16x8 fa[2][TM], fw[2][TN];
        auto read_frags = [&](int ks, int buf) {
            const int c = ks * 2 + g;  // the 16-byte piece of the row this lane needs
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int row = wm * (BM / WM) + i * 32 + li;
                fa[buf][i] = *reinterpret_cast<const bf16x8*>(sa + row * DBK + ((c ^ swizzle(row)) * 8));
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int row = wn * (BN / WN) + j * 32 + li;
                fw[buf][j] = *reinterpret_cast<const bf16x8*>(sw + row * DBK + ((c ^ swizzle(row)) * 8));
            }
        };
        read_frags(0, 0);
#pragma unroll
        for (int ks = 0; ks < DBK / 16; ++ks) {
            if (ks + 1 < DBK / 16) read_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw[ks & 1][j], fa[ks & 1][i], acc[i][j], 0, 0, 0);
        }
    };
    if constexpr (SETS == 1) {
        for (int kt = 0; kt < nk; ++kt) step(kt, std::integral_constant<int, 0>{});
    } else {
        for (int kt = 0; kt < nk; kt += 4) {
            step(kt, std::integral_constant<int, 0>{});
            if (kt + 1 < nk) step(kt + 1, std::integral_constant<int, 1>{});
            if (kt + 2 < nk) step(kt + 2, std::integral_constant<int, 2>{});
            if (kt + 3 < nk) step(kt + 3, std::integral_constant<int, 3>{});
        }
#pragma unroll
        for (int q = 1; q < SETS; ++q)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sums[0][i][j][r] += sums[q][i][j][r];
    }
    floatx16 (&acc)[TM][TN] = sums[0];
    if constexpr (WK > 1) {
        // the groups' sums, added in the groups' order by the first group, which alone stores:
        // the others go through the epilogue as a tile below the last row
        constexpr int PER_WAVE = TM * TN * 16 * 64;
        static_assert((WK - 1) * GROUP * PER_WAVE * 4 <= DSTAGES * STAGE * 2, "the groups' sums must fit the operand stages");
        float* red = reinterpret_cast<float*>(lds);
        __syncthreads();  // everyone is done reading the last operand stage
        if (wk > 0) {
            float* mine = red + ((wk - 1) * GROUP + wg) * PER_WAVE + lane;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) mine[((i * TN + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (wk == 0) {
#pragma unroll
            for (int q = 1; q < WK; ++q) {
                const float* theirs = red + ((q - 1) * GROUP + wg) * PER_WAVE + lane;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int r = 0; r < 16; ++r) acc[i][j][r] += theirs[((i * TN + j) * 16 + r) * 64];
            }
        } else {
            m0 = M;
        }
    }
    // The products were taken transposed (w's fragment as the first operand), so a lane holds one
    // row of each 32 x 32 block, m = li, and of its columns the four groups 8q + 4g + {0..3}: what
    // depends on the row (a token's place in the pages) is computed once, and every store is four
    // consecutive columns wide. Tiles wholly inside the output take that path without bounds
    // checks (a guarded store is a branch of its own: on an interior tile they cost as much as
    // the whole product); tiles at the bottom edge take the same paths with their rows checked;
    // tiles at the right edge, and operands that are not aligned for it, go element by element.
    const bool inside = m0 + BM <= M && n0 + BN <= N, columns_inside = n0 + BN <= N;
    if constexpr (sizeof(OutT) == 2 && EPI >= 0 && EPI != kEpiResidual) {
        // bfloat16 outputs of interior tiles go through LDS once more, so that they leave as whole
        // rows: a wave lays its (BM / WM) x (BN / WN) results out row by row (bias and activation
        // applied), then every lane stores 16 bytes and eight lanes a row of 64 columns: full
        // cache lines, where the accumulators' own layout would write 16 bytes of 32 different
        // rows with every instruction (measured: 5.7 of 19.7 us on a 2,048 x 2,304 product).
        constexpr int RM = BM / WM, CN = BN / WN, LDO = CN + 8;  // padded rows, 16-byte aligned
        static_assert(WAVES * RM * LDO * 2 <= dl_lds_bytes<BM, BN, DSTAGES, WM, WN, WK>(2), "the output staging must fit the dynamic LDS the launcher asks for");
        if (columns_inside && vec_ok > 1) {
            lds_barrier();  // everyone is done reading the last operand stage
            bf16_t* tile = lds + wave * RM * LDO;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const int nb = n0 + wn * CN + j * 32 + 4 * g;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x4 b4 = epi.bias != nullptr ? *reinterpret_cast<const f32x4*>(epi.bias + nb + 8 * q) : f32x4{0.f, 0.f, 0.f, 0.f};
                        f32x4 v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[e] = acc[i][j][4 * q + e] + b4[e];
                            if constexpr (EPI == kEpiGeluTanh) v[e] = gelu_tanh_fast(v[e]);
                            if constexpr (EPI == kEpiGeluErf) v[e] = epi.exact ? gelu_erf_exact(v[e]) : gelu_erf_fast(v[e]);
                        }
                        store4<bf16_t>(tile + (i * 32 + li) * LDO + j * 32 + 8 * q + 4 * g, v);
                    }
                }
            lds_barrier();
            constexpr int CHUNKS = CN / 8, ROUNDS = RM * CHUNKS / 64;  // 16-byte pieces a row; store instructions a lane
            static_assert(RM * CHUNKS % 64 == 0, "a wave's results must be whole rounds of 64 pieces");
            const int mw = m0 + wm * RM, nw = n0 + wn * CN;
            int64_t row_base[ROUNDS];
            if constexpr (EPI == kEpiQkvPaged) {
                // the rows' places in the pages first: a load between two stores would wait for the first
#pragma unroll
                for (int t = 0; t < ROUNDS; ++t) {
                    const int slot = epi.slots[min(mw + (t * 64 + lane) / CHUNKS, M - 1)];
                    const int page = page_shift >= 0 ? slot >> page_shift : slot / epi.page_size;
                    const int off = slot - page * epi.page_size;
                    row_base[t] = static_cast<uint32_t>(slot) >= epi.num_slots ? -1 : static_cast<int64_t>(page) * epi.n_kv_head * epi.page_size * epi.hd + static_cast<int64_t>(off) * epi.hd;
                }
            }
#pragma unroll
            for (int t = 0; t < ROUNDS; ++t) {
                const int c = t * 64 + lane, row = c / CHUNKS, n = nw + (c % CHUNKS) * 8;
                if (!inside && mw + row >= M) continue;
                const u32x4 piece = *reinterpret_cast<const u32x4*>(tile + row * LDO + (c % CHUNKS) * 8);
                bf16_t* dst;
                if constexpr (EPI == kEpiQkvPaged) {
                    if (n < epi.q_dim) {
                        dst = static_cast<bf16_t*>(epi.out) + static_cast<int64_t>(mw + row) * epi.ldo + n;
                    } else {
                        if (row_base[t] < 0) continue;
                        const bool is_v = n >= epi.q_dim + epi.kv_dim;
                        const int cc = n - epi.q_dim - (is_v ? epi.kv_dim : 0);
                        const int head = cc / epi.hd, dim = cc - head * epi.hd;
                        dst = static_cast<bf16_t*>(is_v ? epi.vc : epi.kc) + row_base[t] + static_cast<int64_t>(head) * epi.page_size * epi.hd + dim;
                    }
                } else {
                    dst = static_cast<bf16_t*>(epi.out) + static_cast<int64_t>(mw + row) * epi.ldo + n;
                }
                *reinterpret_cast<u32x4*>(dst) = piece;
            }
            return;
        }
    }
    if (EPI >= 0 && columns_inside && vec_ok) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = m0 + wm * (BM / WM) + i * 32 + li;
            if (!inside && m >= M) continue;
            int64_t row_base = -1;
            if constexpr (EPI == kEpiQkvPaged) {
                const int slot = epi.slots[m];
                const int page = page_shift >= 0 ? slot >> page_shift : slot / epi.page_size;
                const int off = slot - page * epi.page_size;
                row_base = static_cast<uint32_t>(slot) >= epi.num_slots ? -1 : static_cast<int64_t>(page) * epi.n_kv_head * epi.page_size * epi.hd + static_cast<int64_t>(off) * epi.hd;
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int nb = n0 + wn * (BN / WN) + j * 32 + 4 * g;
                // loads first, stores after: a load between two stores waits for the first of them
                f32x4 b4[4], r4[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    b4[q] = epi.bias != nullptr ? *reinterpret_cast<const f32x4*>(epi.bias + nb + 8 * q) : f32x4{0.f, 0.f, 0.f, 0.f};
                    if constexpr (EPI == kEpiResidual)
                        r4[q] = *reinterpret_cast<const f32x4*>(epi.residual + static_cast<int64_t>(m) * epi.ldr + nb + 8 * q);
                    if constexpr (EPI == kEpiParts) {
                        // the first part adds the rows the product is added to, their planes in order
                        r4[q] = f32x4{0.f, 0.f, 0.f, 0.f};
                        if (blockIdx.y == 0 && parts.base != nullptr) {
                            const float* bp = parts.base + static_cast<int64_t>(m) * N + nb + 8 * q;
                            r4[q] = *reinterpret_cast<const f32x4*>(bp);
                            for (int p = 1; p < parts.n_base; ++p) r4[q] += *reinterpret_cast<const f32x4*>(bp + p * parts.base_stride);
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = nb + 8 * q;
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e] + b4[q][e];
                    if constexpr (EPI == kEpiResidual) {
                        *reinterpret_cast<f32x4*>(epi.residual + static_cast<int64_t>(m) * epi.ldr + n) = v + r4[q];
                    } else if constexpr (EPI == kEpiParts) {
                        float* plane = static_cast<float*>(epi.out) + blockIdx.y * parts.part_stride;
                        *reinterpret_cast<f32x4*>(plane + static_cast<int64_t>(m) * N + n) = v + r4[q];
                    } else if constexpr (EPI == kEpiQkvPaged) {
                        if (n < epi.q_dim) {
                            store4<OutT>(static_cast<OutT*>(epi.out) + static_cast<int64_t>(m) * epi.ldo + n, v);
                        } else if (row_base >= 0) {
                            const bool is_v = n >= epi.q_dim + epi.kv_dim;
                            const int c = n - epi.q_dim - (is_v ? epi.kv_dim : 0);
                            const int head = c / epi.hd, dim = c - head * epi.hd;
                            store4<OutT>(static_cast<OutT*>(is_v ? epi.vc : epi.kc) + row_base + static_cast<int64_t>(head) * epi.page_size * epi.hd + dim, v);
                        }
                    } else {
                        if constexpr (EPI == kEpiGeluTanh) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = gelu_tanh_fast(v[e]);
                        } else if constexpr (EPI == kEpiGeluErf) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = epi.exact ? gelu_erf_exact(v[e]) : gelu_erf_fast(v[e]);
                        }
                        store4<OutT>(static_cast<OutT*>(epi.out) + static_cast<int64_t>(m) * epi.ldo + n, v);
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * (BM / WM) + i * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int n = n0 + wn * (BN / WN) + j * 32 + 8 * (r / 4) + 4 * g + r % 4;
                if constexpr (EPI == kEpiParts) {
                    if (n < N) {
                        float v = acc[i][j][r] + epilogue_bias(epi, n);
                        if (blockIdx.y == 0 && parts.base != nullptr) {
                            const float* bp = parts.base + static_cast<int64_t>(m) * N + n;
                            float b = bp[0];
                            for (int p = 1; p < parts.n_base; ++p) b += bp[p * parts.base_stride];
                            v += b;
                        }
                        (static_cast<float*>(epi.out) + blockIdx.y * parts.part_stride)[static_cast<int64_t>(m) * N + n] = v;
                    }
                } else {
                    if (n < N) epilogue_store<OutT, EPI>(epi, m, n, acc[i][j][r]);
                }
            }
    }
}

template <int BM, int BN, int DSTAGES, typename OutT, int EPI, int WM = 2, int WN = 2, int WK = 1, int SETS = 1>
int launch_dl_as(const bf16_t* a, int64_t lda, const bf16_t* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    const int grid = ((N + BN - 1) / BN) * ((M + BM - 1) / BM);
    constexpr size_t smem = dl_lds_bytes<BM, BN, DSTAGES, WM, WN, WK>(sizeof(OutT));
    static_assert(smem <= 160 * 1024, "a workgroup's LDS");
    auto kern = gemm_mfma_dl_kernel<BM, BN, DSTAGES, OutT, EPI, WM, WN, WK, SETS>;
    static bool ready = false;  // once per instantiation, outside any stream capture's first use
    if (!ready) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        ready = true;
    }
    // four-wide stores need aligned rows; the cache's slots fit 32 bits (checked by the launcher)
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    bool vec = N % 4 == 0 && (epi.bias == nullptr || al16(epi.bias));
    int page_shift = -1;
    if (EPI == kEpiResidual) {
        vec = vec && al16(epi.residual) && epi.ldr % 4 == 0;
    } else if (EPI == kEpiQkvPaged) {
        vec = vec && al16(epi.out) && al16(epi.kc) && al16(epi.vc) && epi.ldo % 4 == 0 && epi.hd % 4 == 0 && epi.q_dim % 4 == 0;
        for (int b = 0; b < 31; ++b)
            if ((1 << b) == epi.page_size) page_shift = b;
    } else {
        vec = vec && al16(epi.out) && epi.ldo % 4 == 0;
    }
    // 16-byte pieces of bfloat16 rows: row strides and the boundaries between queries, keys and
    // values in multiples of 8 elements
    bool vec16 = vec && sizeof(OutT) == 2 && N % 8 == 0;
    if (EPI == kEpiQkvPaged) vec16 = vec16 && epi.ldo % 8 == 0 && epi.hd % 8 == 0 && epi.q_dim % 8 == 0;
    else if (EPI != kEpiResidual) vec16 = vec16 && epi.ldo % 8 == 0;
    kern<<<grid, 64 * WM * WN * WK, smem, stream>>>(a, lda, w, M, N, K, epi, vec16 ? 2 : (vec ? 1 : 0), page_shift, PartsParams{});
    return check_launch("gemm_mfma_dl");
}

// The product cut over K into `kparts` parts (see the head of this file); epi carries the planes
// (out, float32, rows of N) and the first plane's bias.
template <int BM, int BN, int DSTAGES, int WM = 2, int WN = 2, int WK = 1>
int launch_dl_parts(const bf16_t* a, int64_t lda, const bf16_t* w, int M, int N, int K, int kparts, const EpiParams& epi,
                    const PartsParams& parts, hipStream_t stream) {
    const dim3 grid(((N + BN - 1) / BN) * ((M + BM - 1) / BM), kparts);
    const size_t smem = static_cast<size_t>(DSTAGES) * WK * (BM + BN) * DBK * sizeof(bf16_t);
    auto kern = gemm_mfma_dl_kernel<BM, BN, DSTAGES, float, kEpiParts, WM, WN, WK>;
    static bool ready = false;
    if (!ready) {
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem));
        ready = true;
    }
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec = N % 4 == 0 && al16(epi.bias) && al16(epi.out) && al16(parts.base) && parts.part_stride % 4 == 0 && parts.base_stride % 4 == 0;
    kern<<<grid, 64 * WM * WN * WK, smem, stream>>>(a, lda, w, M, N, K, epi, vec ? 1 : 0, -1, parts);
    return check_launch("gemm_mfma_dl_parts");
}

template <int BM, int BN, int DSTAGES, int WM = 2, int WN = 2, int WK = 1, int SETS = 1>
int launch_dl(const void* a, int64_t lda, const void* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (epi.mode == kEpiResidual) return launch_dl_as<BM, BN, DSTAGES, float, kEpiResidual, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
    if (epi.out_dtype == kF32) {
        if (epi.mode == kEpiNone) return launch_dl_as<BM, BN, DSTAGES, float, kEpiNone, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
        return launch_dl_as<BM, BN, DSTAGES, float, -1, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
    }
    switch (epi.mode) {
        case kEpiNone: return launch_dl_as<BM, BN, DSTAGES, bf16_t, kEpiNone, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
        case kEpiGeluTanh: return launch_dl_as<BM, BN, DSTAGES, bf16_t, kEpiGeluTanh, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
        case kEpiGeluErf: return launch_dl_as<BM, BN, DSTAGES, bf16_t, kEpiGeluErf, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
        case kEpiQkvPaged: return launch_dl_as<BM, BN, DSTAGES, bf16_t, kEpiQkvPaged, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
        default: return launch_dl_as<BM, BN, DSTAGES, bf16_t, -1, WM, WN, WK, SETS>(pa, lda, pw, M, N, K, epi, stream);
    }
}

}  // namespace liyab

using namespace liyab;

// tile: 2 = 64x64 tiles, three stages deep, on four waves; 6 = the same with four stages; 8 = 128x128, two
// stages, on eight waves; 17 = 32x32 on four waves that walk K side by side (a workgroup then brings in a
// third less of the operands, and twice as many workgroups pull: 64 rows with cold weights, 768 -> 2,304 in
// 5.05 us against 5.53, 1,024 -> 3,072 in 5.97 against 6.85; for as long as every tile has a compute unit
// of its own: 1,600 -> 4,800 in 13.9 against 9.7); 16 = 64x32 on four groups of two waves that walk K side by side, three stages of
// four units (for one tile of rows: 8.2 us for 64 x 4,800 x 1,600 where two waves walking K alone, four
// stages deep, took 10.3; deeper rings for those took longer, 11.1 with eight stages: the walk waits on
// its own chain of load, barrier, fragments and products, not on the loads in flight); 0 = chosen from
// the shape. (Measured and dropped: 128x128 on four waves, 128x64, 128x192, and deeper rings under
// 128x128, whose LDS leaves one workgroup a compute unit, so that 288 tiles take two rounds.)
// The epilogues that tiles of 256 x 256 are compiled with: into the residual stream, plain 32-bit
// outputs, and bfloat16 outputs plain, through the tanh GELU or into the cache's pages.
static bool dl_takes_256(const EpiParams& epi) {
    if (epi.mode == kEpiResidual) return true;
    if (epi.out_dtype == kF32) return epi.mode == kEpiNone;
    return epi.mode == kEpiNone || epi.mode == kEpiGeluTanh || epi.mode == kEpiQkvPaged;
}

static int launch_dl_256(const void* a, int64_t lda, const void* w, int M, int N, int K, const EpiParams& epi, hipStream_t stream) {
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (epi.mode == kEpiResidual) return launch_dl_as<256, 256, 2, float, kEpiResidual, 2, 4>(pa, lda, pw, M, N, K, epi, stream);
    if (epi.out_dtype == kF32) return launch_dl_as<256, 256, 2, float, kEpiNone, 2, 4>(pa, lda, pw, M, N, K, epi, stream);
    if (epi.mode == kEpiGeluTanh) return launch_dl_as<256, 256, 2, bf16_t, kEpiGeluTanh, 2, 4>(pa, lda, pw, M, N, K, epi, stream);
    if (epi.mode == kEpiQkvPaged) return launch_dl_as<256, 256, 2, bf16_t, kEpiQkvPaged, 2, 4>(pa, lda, pw, M, N, K, epi, stream);
    return launch_dl_as<256, 256, 2, bf16_t, kEpiNone, 2, 4>(pa, lda, pw, M, N, K, epi, stream);
}

extern "C" int liyab_gemm_mfma_dl(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile,
                                  const EpiParams* epi_in, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && epi_in, "gemm: null operand");
    LIYAB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma_dl: bad sizes M=%d N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % DBK == 0 && lda % 8 == 0 && lda >= K, "gemm_mfma_dl: K %d must be a multiple of 64 and lda %lld of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_mfma_dl: operands must be 16-byte aligned");
    EpiParams epi = *epi_in;
    if (int rc = check_epilogue(epi, M, N)) return rc;
    // measured on {256..8192} x {768 .. 16,384} x {768 .. 16,384}: 64 x 64 tiles, three workgroups a
    // CU, win or tie for small outputs; a long K likes one more stage in flight; a large output
    // (2,048 x 2,304 and up) likes 128 x 128 tiles, two stages deep, on eight waves (16.9 us against
    // 17.3 for 2,048 x 2,304 x 768, 18.0 against 22.6 for 2,048 x 3,072 x 768)
    // A large output takes the 128 x 128 tiles whatever K (2,048 x 16,384 x 4,096: 0.85 PFLOP/s against 0.46 in
    // tiles of 64 x 64), a somewhat smaller one with a long K too (2,048 x 1,600 x 6,400: 79 against 88 us); the
    // fourth stage pays while the tiles of 64 x 64 are few enough for its LDS (4,096 x 768 x 3,072, 768 tiles:
    // 36 us with three stages, 49 with four).
    // Tiles of 256 x 256 (half the operand bytes a product of 128 x 128 tiles brings in from L2) where
    // K is long and they fill whole rounds over the chip's 256 compute units, one a unit: 0.93-1.1
    // PFLOP/s against 0.8-0.95 at widths of 4,096 to 16,384 (4,096 x 4,096 x 16,384: 502 against 611
    // us); with 384 tiles (a round and a half), or a K of 1,600 and more than one round (8,192 x 6,400 x
    // 1,600: 289 against 248 us), the 128 x 128 tiles, two a unit, win. (Alone and added to the residual
    // stream, 2,048 x 2,304 x 768 runs 19.8 us in 64 x 64 tiles and 23.4 in 128 x 128; in a prefill
    // step, writing keys and values into their pages or through the GELU, the large tiles win.)
    if (tile == 0) {
        const long out = static_cast<long>(M) * N, tiles64 = static_cast<long>((M + 63) / 64) * ((N + 63) / 64);
        const long tiles256 = static_cast<long>((M + 255) / 256) * ((N + 255) / 256), rounds = (tiles256 + 255) / 256;
        if ((K >= 2048 || (K >= 1536 && rounds == 1)) && tiles256 >= 200 && tiles256 * 100 >= rounds * 256 * 78 && dl_takes_256(epi)) tile = 15;
        else if (out >= 2048L * 2048L || (out >= 2560L * 1024L && K >= 4096)) tile = 8;
        else tile = (K >= 2048 && tiles64 < 640) ? 6 : 2;
    }
    switch (tile) {
        case 2: return launch_dl<64, 64, 3>(a, lda, w, M, N, K, epi, stream);
        case 6: return launch_dl<64, 64, 4>(a, lda, w, M, N, K, epi, stream);
        case 8: return launch_dl<128, 128, 2, 4, 2>(a, lda, w, M, N, K, epi, stream);
        case 15:
            // 256 x 256 on eight waves of 128 x 64: with the epilogues that are compiled in (the others
            // would spill its 128 accumulation registers a lane) and tiles of 128 x 128 otherwise
            if (dl_takes_256(epi)) return launch_dl_256(a, lda, w, M, N, K, epi, stream);
            return launch_dl<128, 128, 2, 4, 2>(a, lda, w, M, N, K, epi, stream);
        case 16: return launch_dl<64, 32, 3, 2, 1, 4>(a, lda, w, M, N, K, epi, stream);
        case 17: return launch_dl<32, 32, 3, 1, 1, 4>(a, lda, w, M, N, K, epi, stream);
        // 102, 106, 108: the tiles of 2, 6 and 8 with four sums by unit of K, whose results are those of 16 and 17 bit for bit
        case 102: return launch_dl<64, 64, 3, 2, 2, 1, 4>(a, lda, w, M, N, K, epi, stream);
        case 106: return launch_dl<64, 64, 4, 2, 2, 1, 4>(a, lda, w, M, N, K, epi, stream);
        case 108: return launch_dl<128, 128, 2, 4, 2, 1, 4>(a, lda, w, M, N, K, epi, stream);
        default: return fail(1, "gemm_mfma_dl: unknown tile %d", tile);
    }
}

// The same product cut over K: parts[p * part_stride + m * N + n] = sum over the p-th of `kparts` parts
// of K (whole tiles of 64) of a[m, k] w[n, k]. With `base` (n_base planes [M, N], base_stride floats
// apart, not overlapping `parts`) the first plane also takes bias[n] and base[0] + base[1] + ...;
// without it `bias` must be null. tile: 6 = 64x64 tiles, 16 = 64x32 (for one tile of rows), 17 = 32x32.
extern "C" int liyab_gemm_mfma_dl_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts, int tile,
                                        float* parts, int64_t part_stride, const float* bias, const float* base, int n_base,
                                        int64_t base_stride, hipStream_t stream) {
    LIYAB_REQUIRE(a && w && parts, "gemm: null operand");
    LIYAB_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_mfma_dl_parts: bad sizes M=%d N=%d K=%d", M, N, K);
    LIYAB_REQUIRE(K % DBK == 0 && lda % 8 == 0 && lda >= K, "gemm_mfma_dl_parts: K %d must be a multiple of 64 and lda %lld of 8", K,
                  static_cast<long long>(lda));
    LIYAB_REQUIRE((reinterpret_cast<uintptr_t>(a) & 15) == 0 && (reinterpret_cast<uintptr_t>(w) & 15) == 0,
                  "gemm_mfma_dl_parts: operands must be 16-byte aligned");
    const int nk = K / DBK;
    LIYAB_REQUIRE(kparts >= 1 && kparts <= 16 && (kparts - 1) * ((nk + kparts - 1) / kparts) < nk,
                  "gemm_mfma_dl_parts: K = %d does not cut into %d parts of whole tiles of 64", K, kparts);
    LIYAB_REQUIRE(kparts == 1 || part_stride >= static_cast<int64_t>(M) * N, "gemm_mfma_dl_parts: planes of %lld overlap",
                  static_cast<long long>(part_stride));
    LIYAB_REQUIRE(base != nullptr || bias == nullptr, "gemm_mfma_dl_parts: a bias needs the rows it is added to");
    if (base != nullptr) {
        LIYAB_REQUIRE(n_base >= 1 && n_base <= 16 && (n_base == 1 || base_stride >= static_cast<int64_t>(M) * N),
                      "gemm_mfma_dl_parts: bad planes of rows to add to (%d, %lld apart)", n_base, static_cast<long long>(base_stride));
        const float* base_end = base + (n_base - 1) * base_stride + static_cast<int64_t>(M) * N;
        const float* parts_end = parts + (kparts - 1) * part_stride + static_cast<int64_t>(M) * N;
        LIYAB_REQUIRE(base_end <= parts || parts_end <= base, "gemm_mfma_dl_parts: the rows to add to overlap the planes written");
    }
    EpiParams epi{};
    epi.mode = kEpiNone;
    epi.out_dtype = kF32;
    epi.out = parts;
    epi.ldo = N;
    epi.bias = bias;
    const PartsParams pp{(nk + kparts - 1) / kparts, part_stride, base, n_base, base_stride};
    auto* pa = static_cast<const bf16_t*>(a);
    auto* pw = static_cast<const bf16_t*>(w);
    if (tile == 6) return launch_dl_parts<64, 64, 4>(pa, lda, pw, M, N, K, kparts, epi, pp, stream);
    if (tile == 16) return launch_dl_parts<64, 32, 3, 2, 1, 4>(pa, lda, pw, M, N, K, kparts, epi, pp, stream);
    if (tile == 17) return launch_dl_parts<32, 32, 3, 1, 1, 4>(pa, lda, pw, M, N, K, kparts, epi, pp, stream);
    return fail(1, "gemm_mfma_dl_parts: unknown tile %d (6, 16 or 17)", tile);
}
