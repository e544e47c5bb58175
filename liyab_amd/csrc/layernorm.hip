// LayerNorm over rows of the 32-bit residual stream.
//
// y = (x - mean) / sqrt(var + eps) * w + b with the biased variance, the
// reference's `layernorm` (src/core/transformer.cpp:77-106). Mean and
// variance are two passes in 32-bit with a fixed reduction tree (the
// reference accumulates in double); the affine step is 32-bit and the result
// is rounded once to the output type. `rows`, when given, gathers: output
// row r normalises input row rows[r] (the final norm runs only on the rows
// whose logits are wanted, src/core/transformer.cpp:6569-6572).
#include "common.h"

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

template <typename T, int MAXV>
__global__ void __launch_bounds__(256)
layernorm_wave_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ w,
                      const float* __restrict__ b, const int* __restrict__ rows, int n, int d, float eps) {
    const int lane = threadIdx.x % kWave, r = blockIdx.x * 4 + threadIdx.x / kWave;
    if (r >= n) return;
    const int64_t src = rows != nullptr ? rows[r] : r;
    const f32x4* xr = reinterpret_cast<const f32x4*>(x + src * d);
    const int nv = d / 4;
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f}, one = {1.0f, 1.0f, 1.0f, 1.0f};
    f32x4 v[MAXV], gw[MAXV], gb[MAXV];
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
        const int i = min(lane + kWave * j, nv - 1);  // past the row: its last piece again, unused
        v[j] = xr[i];
        gw[j] = w != nullptr ? reinterpret_cast<const f32x4*>(w)[i] : one;
        gb[j] = b != nullptr ? reinterpret_cast<const f32x4*>(b)[i] : zero;
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

template <typename T>
int launch_layernorm(T* out, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                     hipStream_t stream) {
    auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (d % 4 == 0 && d <= 2048 && al16(out) && al16(x) && al16(w) && al16(b)) {
        const int grid = (n + 3) / 4;
        if (d <= 256) layernorm_wave_kernel<T, 1><<<grid, 256, 0, stream>>>(out, x, w, b, rows, n, d, eps);
        else if (d <= 512) layernorm_wave_kernel<T, 2><<<grid, 256, 0, stream>>>(out, x, w, b, rows, n, d, eps);
        else if (d <= 768) layernorm_wave_kernel<T, 3><<<grid, 256, 0, stream>>>(out, x, w, b, rows, n, d, eps);
        else if (d <= 1024) layernorm_wave_kernel<T, 4><<<grid, 256, 0, stream>>>(out, x, w, b, rows, n, d, eps);
        else layernorm_wave_kernel<T, 8><<<grid, 256, 0, stream>>>(out, x, w, b, rows, n, d, eps);
    } else if (d <= 256) {
        layernorm_kernel<T, 64><<<n, 64, 0, stream>>>(out, x, w, b, rows, d, eps);
    } else {
        layernorm_kernel<T, 256><<<n, 256, 0, stream>>>(out, x, w, b, rows, d, eps);
    }
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
    if (out_dtype == kF32) return launch_layernorm(static_cast<float*>(out), x, w, b, rows, n, d, eps, stream);
    if (out_dtype == kBF16) return launch_layernorm(static_cast<bf16_t*>(out), x, w, b, rows, n, d, eps, stream);
    return fail(1, "layernorm: unknown output dtype %d", out_dtype);
}
