// LayerNorm over rows of the 32-bit residual stream.
//
// y = (x - mean) / sqrt(var + eps) * w + b with the biased variance, the
// reference's `layernorm` (src/core/transformer.cpp:77-106). Mean and
// variance are two passes in 32-bit with a fixed reduction tree (the
// reference accumulates in double); the affine step is 32-bit and the result
// is rounded once to the output type. `rows`, when given, gathers: output
// row r normalises input row rows[r] (the final norm runs only on the rows
// whose logits are wanted, src/core/transformer.cpp:6569-6572).
//
// The rows may come as a sum of planes: a product cut over its inner dimension leaves one
// plane of 32-bit sums a part (the first of them holding the rows the product was added to),
// and the norm that reads the residual stream next adds the planes up, in their order, as it
// loads a row.
#include "common.h"
#include "launchers.h"

namespace liyab {

template <int THREADS>
__device__ __forceinline__ float block_sum(float v, float* red) {
    constexpr int WAVES = THREADS / kWave;
    v = wave_sum(v);
    if constexpr (WAVES == 1) return v;
    const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
    __syncthreads();  // red may still be read from a previous call
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < WAVES; ++i) total += red[i];
    return total;
}

template <typename T, int THREADS>
__global__ void __launch_bounds__(THREADS)
layernorm_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                 const float* __restrict__ b, const int* __restrict__ rows, int d, float eps) {
    __shared__ float red[THREADS / kWave];
    const int r = blockIdx.x;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const float* xr = x + src * d;
    T* o = out + static_cast<int64_t>(r) * d;
    float s = 0.0f;
    for (int i = threadIdx.x; i < d; i += THREADS) s += xr[i];
    const float mean = block_sum<THREADS>(s, red) / static_cast<float>(d);
    float ss = 0.0f;
    for (int i = threadIdx.x; i < d; i += THREADS) {
        const float dev = xr[i] - mean;
        ss += dev * dev;
    }
    const float var = block_sum<THREADS>(ss, red) / static_cast<float>(d);
    const float scale = 1.0f / sqrtf(var + eps);
    for (int i = threadIdx.x; i < d; i += THREADS) {
        float v = (xr[i] - mean) * scale;
        if (w != nullptr) v *= w[i];
        if (b != nullptr) v += b[i];
        o[i] = from_float<T>(v);
    }
}

// Rows given as a sum of planes: row r is x[r] + x[stride + r] + ... (n_parts planes, 1: x itself).
struct PartSums {
    int n_parts;
    int64_t stride;
};

// The same for rows that fit a wave's registers (d a multiple of 4, at most 256 * MAXV): a
// wave per row, four rows a workgroup. The row is read once, 16 bytes a lane; sums go over
// the wave only (no LDS, no barrier); weight and bias are fetched before the sums, so their
// latency hides behind them.
typedef __attribute__((ext_vector_type(4))) float f32x4;

template <typename T>
__device__ __forceinline__ void store_row4(T* dst, const f32x4& v);
template <>
__device__ __forceinline__ void store_row4<float>(float* dst, const f32x4& v) { *reinterpret_cast<f32x4*>(dst) = v; }
template <>
__device__ __forceinline__ void store_row4<bf16_t>(bf16_t* dst, const f32x4& v) {
    uint2 packed;
    packed.x = static_cast<uint32_t>(float_to_bf16(v[0])) | (static_cast<uint32_t>(float_to_bf16(v[1])) << 16);
    packed.y = static_cast<uint32_t>(float_to_bf16(v[2])) | (static_cast<uint32_t>(float_to_bf16(v[3])) << 16);
    *reinterpret_cast<uint2*>(dst) = packed;
}

template <typename T, int MAXV, bool PARTS>
__global__ void __launch_bounds__(256)
layernorm_wave_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                      const float* __restrict__ b, const int* __restrict__ rows, int n, int d, float eps, PartSums ps) {
    // a wave a row, blockDim.x / 64 rows a workgroup: one while the rows are few, so that they spread over
    // as many compute units (in a replayed chain, 64 rows of 1,600 in five planes: 3.5 us against 3.9 with
    // four rows a workgroup, of 768: 2.7 against 3.0; one plane 0.1-0.2 us less; from 2,048 rows on the same)
    const int lane = threadIdx.x % kWave, r = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (r >= n) return;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const float* row0 = x + src * d;
    const int nv = d / 4;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f}, one = {1.0f, 1.0f, 1.0f, 1.0f};
    f32x4 v[MAXV], gw[MAXV], gb[MAXV];
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = min(lane + kWave * j, nv - 1);  // past the row: its last piece again, unused
        v[j] = reinterpret_cast<const f32x4*>(row0)[i];
        gw[j] = w != nullptr ? reinterpret_cast<const f32x4*>(w)[i] : one;
        gb[j] = b != nullptr ? reinterpret_cast<const f32x4*>(b)[i] : zero;
    }
    if constexpr (PARTS) {
        // the further planes in their order, three planes' loads in flight together (a plane
        // past the last is the last one again, read and dropped: no load under a branch)
        constexpr int PB = MAXV <= 4 ? 3 : 1;
        for (int q0 = 1; q0 < ps.n_parts; q0 += PB) {
            f32x4 plane[PB][MAXV];
#pragma unroll
            for (int u = 0; u < PB; ++u) {
                const float* row = row0 + min(q0 + u, ps.n_parts - 1) * ps.stride;
#pragma unroll
                for (int j = 0; j < MAXV; ++j) plane[u][j] = reinterpret_cast<const f32x4*>(row)[min(lane + kWave * j, nv - 1)];
            }
#pragma unroll
            for (int u = 0; u < PB; ++u)
#pragma unroll
                for (int j = 0; j < MAXV; ++j)
                    if (q0 + u < ps.n_parts) v[j] += plane[u][j];
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (lane + kWave * j < nv) s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    const float mean = wave_sum(s) / static_cast<float>(d);
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (lane + kWave * j < nv) {
            const f32x4 dev = v[j] - mean;
            ss += (dev[0] * dev[0] + dev[1] * dev[1]) + (dev[2] * dev[2] + dev[3] * dev[3]);
        }
    const float scale = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(d) + eps);
    T* o = out + static_cast<int64_t>(r) * d;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (lane + kWave * j < nv) store_row4<T>(o + 4 * (lane + kWave * j), (v[j] - mean) * scale * gw[j] + gb[j]);
}

// The same for wider rows (d a multiple of 4, at most THREADS * 4 * MAXV): a workgroup a row,
// the row in its threads' registers, sums across the waves through LDS.
template <typename T, int THREADS, int MAXV, bool PARTS>
__global__ void __launch_bounds__(THREADS)
layernorm_block_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                       const float* __restrict__ b, const int* __restrict__ rows, int d, float eps, PartSums ps) {
    __shared__ float red[THREADS / kWave];
    const int r = blockIdx.x, tid = threadIdx.x;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const float* row0 = x + src * d;
    const int nv = d / 4;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f}, one = {1.0f, 1.0f, 1.0f, 1.0f};
    f32x4 v[MAXV], gw[MAXV], gb[MAXV];
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = min(tid + THREADS * j, nv - 1);  // past the row: its last piece again, unused
        v[j] = reinterpret_cast<const f32x4*>(row0)[i];
        gw[j] = w != nullptr ? reinterpret_cast<const f32x4*>(w)[i] : one;
        gb[j] = b != nullptr ? reinterpret_cast<const f32x4*>(b)[i] : zero;
    }
    if constexpr (PARTS) {
        // the further planes in their order, two planes' loads in flight together
        constexpr int PB = 2;
        for (int q0 = 1; q0 < ps.n_parts; q0 += PB) {
            f32x4 plane[PB][MAXV];
#pragma unroll
            for (int u = 0; u < PB; ++u) {
                const float* row = row0 + min(q0 + u, ps.n_parts - 1) * ps.stride;
#pragma unroll
                for (int j = 0; j < MAXV; ++j) plane[u][j] = reinterpret_cast<const f32x4*>(row)[min(tid + THREADS * j, nv - 1)];
            }
#pragma unroll
            for (int u = 0; u < PB; ++u)
#pragma unroll
                for (int j = 0; j < MAXV; ++j)
                    if (q0 + u < ps.n_parts) v[j] += plane[u][j];
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (tid + THREADS * j < nv) s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    const float mean = block_sum<THREADS>(s, red) / static_cast<float>(d);
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (tid + THREADS * j < nv) {
            const f32x4 dev = v[j] - mean;
            ss += (dev[0] * dev[0] + dev[1] * dev[1]) + (dev[2] * dev[2] + dev[3] * dev[3]);
        }
    const float scale = 1.0f / sqrtf(block_sum<THREADS>(ss, red) / static_cast<float>(d) + eps);
    T* o = out + static_cast<int64_t>(r) * d;
#pragma unroll
    for (int j = 0; j < MAXV; ++j)
        if (tid + THREADS * j < nv) store_row4<T>(o + 4 * (tid + THREADS * j), (v[j] - mean) * scale * gw[j] + gb[j]);
}

template <typename T, int THREADS>
void launch_block(T* out, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                  const PartSums& ps, hipStream_t stream) {
    if (ps.n_parts > 1) layernorm_block_kernel<T, THREADS, 4, true><<<n, THREADS, 0, stream>>>(out, x, w, b, rows, d, eps, ps);
    else layernorm_block_kernel<T, THREADS, 4, false><<<n, THREADS, 0, stream>>>(out, x, w, b, rows, d, eps, ps);
}

// out[i] = planes[0][i] + planes[1][i] + ..., added up in that order (the norm kernels' order).
__global__ void __launch_bounds__(256) sum_parts_kernel(float* out, const float* planes, int64_t total, PartSums ps) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    float v = planes[i];
    for (int q = 1; q < ps.n_parts; ++q) v += planes[q * ps.stride + i];
    out[i] = v;
}

template <typename T, int MAXV>
void launch_wave(T* out, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                 const PartSums& ps, hipStream_t stream) {
    const int waves = n <= 512 ? 1 : 4;  // rows a workgroup
    const int grid = (n + waves - 1) / waves;
    if (ps.n_parts > 1) layernorm_wave_kernel<T, MAXV, true><<<grid, kWave * waves, 0, stream>>>(out, x, w, b, rows, n, d, eps, ps);
    else layernorm_wave_kernel<T, MAXV, false><<<grid, kWave * waves, 0, stream>>>(out, x, w, b, rows, n, d, eps, ps);
}

// Whether the kernels that keep a row in registers take these operands (the only ones that add planes up):
// a wave a row up to a width of 2,048, a workgroup a row beyond.
constexpr int kWaveWidth = 2048, kBlockWidth = 16384;
static bool registers_take(const void* out, const float* x, const float* w, const float* b, int d, int64_t stride) {
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    return d % 4 == 0 && d <= kBlockWidth && al16(out) && al16(x) && al16(w) && al16(b) && stride % 4 == 0;
}

template <typename T>
int launch_layernorm(T* out, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                     const PartSums& ps, hipStream_t stream) {
    if (registers_take(out, x, w, b, d, ps.stride)) {
        if (d > 4096) launch_block<T, 1024>(out, x, w, b, rows, n, d, eps, ps, stream);
        else if (d > kWaveWidth) launch_block<T, 256>(out, x, w, b, rows, n, d, eps, ps, stream);
        else if (d <= 256) launch_wave<T, 1>(out, x, w, b, rows, n, d, eps, ps, stream);
        else if (d <= 512) launch_wave<T, 2>(out, x, w, b, rows, n, d, eps, ps, stream);
        else if (d <= 768) launch_wave<T, 3>(out, x, w, b, rows, n, d, eps, ps, stream);
        else if (d <= 1024) launch_wave<T, 4>(out, x, w, b, rows, n, d, eps, ps, stream);
        else launch_wave<T, 8>(out, x, w, b, rows, n, d, eps, ps, stream);
        return check_launch("layernorm");
    }
    LIYAB_REQUIRE(ps.n_parts <= 1, "layernorm: rows in %d planes need a width that is a multiple of 4, at most 16384 (got %d), and 16-byte alignment",
                  ps.n_parts, d);
    if (d <= 256) layernorm_kernel<T, 64><<<n, 64, 0, stream>>>(out, x, w, b, rows, d, eps);
    else layernorm_kernel<T, 256><<<n, 256, 0, stream>>>(out, x, w, b, rows, d, eps);
    return check_launch("layernorm");
}

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b,
                               const int* rows, int n, int d, float eps, hipStream_t stream) {
    LIYAB_REQUIRE(out && x, "layernorm: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "layernorm: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(eps >= 0.0f, "layernorm: negative eps");
    if (n == 0) return 0;
    const PartSums none{1, 0};
    if (out_dtype == kF32) return launch_layernorm(static_cast<float*>(out), x, w, b, rows, n, d, eps, none, stream);
    if (out_dtype == kBF16) return launch_layernorm(static_cast<bf16_t*>(out), x, w, b, rows, n, d, eps, none, stream);
    return fail(1, "layernorm: unknown output dtype %d", out_dtype);
}

// The same over rows given as a sum of planes: row r is planes[0][r] + planes[1][r] + ...
// (n_parts planes [x_rows, d], part_stride floats apart), added in that order. d must be a
// multiple of 4, at most 16,384, and the operands 16-byte aligned (liyab_sum_parts first otherwise).
extern "C" int liyab_layernorm_parts(void* out, int out_dtype, const float* planes, int n_parts, int64_t part_stride,
                                     int x_rows, const float* w, const float* b, const int* rows, int n, int d, float eps,
                                     hipStream_t stream) {
    LIYAB_REQUIRE(out && planes, "layernorm: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0 && x_rows >= 0, "layernorm: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(eps >= 0.0f, "layernorm: negative eps");
    LIYAB_REQUIRE(n_parts >= 1 && n_parts <= 16, "layernorm: bad number of planes %d", n_parts);
    LIYAB_REQUIRE(n_parts == 1 || part_stride >= static_cast<int64_t>(x_rows) * d, "layernorm: planes of sums overlap");
    LIYAB_REQUIRE(rows != nullptr || n <= x_rows, "layernorm: %d rows to normalise, %d rows given", n, x_rows);
    if (n == 0) return 0;
    const PartSums ps{n_parts, part_stride};
    if (out_dtype == kF32) return launch_layernorm(static_cast<float*>(out), planes, w, b, rows, n, d, eps, ps, stream);
    if (out_dtype == kBF16) return launch_layernorm(static_cast<bf16_t*>(out), planes, w, b, rows, n, d, eps, ps, stream);
    return fail(1, "layernorm: unknown output dtype %d", out_dtype);
}

// out [x_rows, d] = planes[0] + planes[1] + ..., for a reader of the rows that cannot add them up itself.
// `out` may be the first plane.
extern "C" int liyab_sum_parts(float* out, int x_rows, int d, const float* planes, int n_parts, int64_t part_stride,
                               hipStream_t stream) {
    LIYAB_REQUIRE(out && planes && x_rows >= 0 && d > 0, "sum_parts: bad operands");
    LIYAB_REQUIRE(n_parts >= 1 && n_parts <= 16, "sum_parts: bad number of planes %d", n_parts);
    LIYAB_REQUIRE(n_parts == 1 || part_stride >= static_cast<int64_t>(x_rows) * d, "sum_parts: planes of sums overlap");
    const int64_t total = static_cast<int64_t>(x_rows) * d;
    if (total == 0) return 0;
    sum_parts_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(out, planes, total, PartSums{n_parts, part_stride});
    return check_launch("sum_parts");
}
