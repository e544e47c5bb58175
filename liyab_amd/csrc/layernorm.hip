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

}  // namespace liyab

using namespace liyab;

extern "C" int liyab_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b,
                               const int* rows, int n, int d, float eps, hipStream_t stream) {
    LIYAB_REQUIRE(out && x, "layernorm: null pointer");
    LIYAB_REQUIRE(n >= 0 && d > 0, "layernorm: bad sizes n=%d d=%d", n, d);
    LIYAB_REQUIRE(eps >= 0.0f, "layernorm: negative eps");
    if (n == 0) return 0;
    if (out_dtype == kF32) {
        if (d <= 256) layernorm_kernel<float, 64><<<n, 64, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, d, eps);
        else layernorm_kernel<float, 256><<<n, 256, 0, stream>>>(static_cast<float*>(out), x, w, b, rows, d, eps);
    } else if (out_dtype == kBF16) {
        if (d <= 256) layernorm_kernel<bf16_t, 64><<<n, 64, 0, stream>>>(static_cast<bf16_t*>(out), x, w, b, rows, d, eps);
        else layernorm_kernel<bf16_t, 256><<<n, 256, 0, stream>>>(static_cast<bf16_t*>(out), x, w, b, rows, d, eps);
    } else {
        return fail(1, "layernorm: unknown output dtype %d", out_dtype);
    }
    return check_launch("layernorm");
}
