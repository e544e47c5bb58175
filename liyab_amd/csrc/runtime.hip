// Error reporting shared by every launcher, and small utility kernels.
#include "common.h"
#include "launchers.h"

#include <cstring>

namespace liyab {

static thread_local char g_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof g_error, fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(2, "%s: %s", what, hipGetErrorString(e));
    return 0;
}

template <typename T>
__global__ void fill_kernel(T* p, T v, int64_t n) {
    int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += step) p[i] = v;
}

// y[i] += x[i] (fp32 residual += branch output in T)
template <typename T>
__global__ void add_into_kernel(float* y, const T* x, int64_t n) {
    int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const int64_t step = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (; i < n; i += step) y[i] += to_float<T>(x[i]);
}

}  // namespace liyab

using namespace liyab;

extern "C" const char* liyab_last_error() { return g_error; }

// The gfx target this library was built for must be the device's.
extern "C" int liyab_check_device() {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(2, "hipGetDevice: %s", hipGetErrorString(e));
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return fail(2, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        return fail(3, "this library holds gfx950 code; device %d is %s", dev, prop.gcnArchName);
    }
    return 0;
}

// Fills n 32-bit words (value given as bits) or n 16-bit words.
extern "C" int liyab_fill(void* p, int elem_bytes, uint32_t bits, int64_t n, hipStream_t stream) {
    LIYAB_REQUIRE(p != nullptr || n == 0, "fill: null pointer");
    LIYAB_REQUIRE(elem_bytes == 4 || elem_bytes == 2, "fill: element size %d is not 2 or 4", elem_bytes);
    LIYAB_REQUIRE(n >= 0, "fill: negative count");
    if (n == 0) return 0;
    const int threads = 256;
    const int blocks = static_cast<int>(std::min<int64_t>((n + threads - 1) / threads, 4096));
    if (elem_bytes == 4) {
        fill_kernel<uint32_t><<<blocks, threads, 0, stream>>>(static_cast<uint32_t*>(p), bits, n);
    } else {
        fill_kernel<uint16_t><<<blocks, threads, 0, stream>>>(static_cast<uint16_t*>(p), static_cast<uint16_t>(bits), n);
    }
    return check_launch("fill");
}

extern "C" int liyab_add_into(float* y, const void* x, int dtype, int64_t n, hipStream_t stream) {
    LIYAB_REQUIRE(y != nullptr && x != nullptr, "add_into: null pointer");
    LIYAB_REQUIRE(dtype == kF32 || dtype == kBF16, "add_into: unknown dtype %d", dtype);
    if (n <= 0) return 0;
    const int threads = 256;
    const int blocks = static_cast<int>(std::min<int64_t>((n + threads - 1) / threads, 4096));
    if (dtype == kF32) {
        add_into_kernel<float><<<blocks, threads, 0, stream>>>(y, static_cast<const float*>(x), n);
    } else {
        add_into_kernel<bf16_t><<<blocks, threads, 0, stream>>>(y, static_cast<const bf16_t*>(x), n);
    }
    return check_launch("add_into");
}
