// Shared declarations of the HIP kernels' host launchers (gfx950 / CDNA4).
//
// Every launcher is `extern "C"`, takes raw device pointers, sizes and the
// stream to launch on, checks its operands on the host, and returns 0 or a
// non-zero code after storing a message that `liyab_last_error()` returns.
// No launcher allocates device memory: callers pass outputs and workspaces.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

namespace liyab {

// Element types a launcher accepts for activations, weights and cache pages.
enum DType : int { kF32 = 0, kBF16 = 1 };

typedef uint16_t bf16_t;  // bfloat16 bits

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(static_cast<uint32_t>(v) << 16); }

// Round to nearest, ties to even; NaN stays NaN. The cast is gfx950's conversion instruction.
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
    const __bf16 b = static_cast<__bf16>(f);
    return __builtin_bit_cast(bf16_t, b);
}

template <typename T>
__device__ __forceinline__ float to_float(T v);
template <>
__device__ __forceinline__ float to_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T>
__device__ __forceinline__ T from_float(float v);
template <>
__device__ __forceinline__ float from_float<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// Stores `code`'s message for liyab_last_error(); returns `code`.
int fail(int code, const char* fmt, ...);
// 0, or fail(...) with the runtime's message when the last launch failed.
int check_launch(const char* what);

constexpr int kWave = 64;

// A workgroup barrier that orders LDS traffic only: this wave's LDS reads and writes are done
// before it, but global loads may stay in flight across it. __syncthreads() also waits for every
// outstanding global load, which throws away whatever a kernel prefetched into registers.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

}  // namespace liyab

#define LIYAB_REQUIRE(cond, ...)                          \
    do {                                                  \
        if (!(cond)) return ::liyab::fail(1, __VA_ARGS__); \
    } while (0)
