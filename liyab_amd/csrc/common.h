// Shared declarations of the HIP kernels' host launchers (gfx950 / CDNA4).
//
// Every launcher is `extern "C"`, takes raw device pointers, sizes and the
// stream to launch on, checks its operands on the host, and returns 0 or a
// non-zero code after storing a message that `liyab_last_error()` returns.
// No launcher allocates device memory: callers pass outputs and workspaces.
#pragma once

#include <type_traits>
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

// Sums and maxima over the 64 lanes of a wave, the same bits in every lane. Within a row of 16
// lanes the partners come through the lanes' own data path (DPP: neighbours in a quad, the other
// pair of the quad, the other quad of eight, the other eight of the row: a few cycles each);
// the four rows' results are then read as scalars and combined. An exchange through the LDS
// crossbar (__shfl_xor) takes about a hundred cycles to come back, six of them in a row a
// reduction: a norm's two sums were a microsecond of its kernel.
template <int CTRL>
__device__ __forceinline__ float lanes_dpp(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float lane_of(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
// The sum over each group of LANES consecutive lanes (a power of two up to 32), in every lane of
// the group; the partners' order is that of v += lane ^ 1, ^ 2, ^ 4, ^ 8.
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(LANES == 1 || LANES == 2 || LANES == 4 || LANES == 8 || LANES == 16 || LANES == 32, "a power of two up to 32");
    if constexpr (LANES > 1) v += lanes_dpp<0xB1>(v);
    if constexpr (LANES > 2) v += lanes_dpp<0x4E>(v);
    if constexpr (LANES > 4) v += lanes_dpp<0x141>(v);
    if constexpr (LANES > 8) v += lanes_dpp<0x140>(v);
    if constexpr (LANES > 16) v += __shfl_xor(v, 16, kWave);  // the next row of 16: no path but the crossbar
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v += lanes_dpp<0xB1>(v);   // quad_perm [1, 0, 3, 2]: lane ^ 1
    v += lanes_dpp<0x4E>(v);   // quad_perm [2, 3, 0, 1]: lane ^ 2
    v += lanes_dpp<0x141>(v);  // row_half_mirror: the other quad of eight (every lane of a quad holds the same)
    v += lanes_dpp<0x140>(v);  // row_mirror: the other eight of the row
    return (lane_of(v, 0) + lane_of(v, 16)) + (lane_of(v, 32) + lane_of(v, 48));
}
// The largest value of the wave and the lowest index that holds it (every lane gets both):
// the same steps, a pair at a time. KeyT is float or uint32_t.
template <typename KeyT>
__device__ __forceinline__ void wave_argmax(KeyT& bv, int& bi) {
    auto take = [&](KeyT ov, int oi) {
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    };
    auto step = [&](auto ctrl) {
        constexpr int CTRL = decltype(ctrl)::value;
        uint32_t bits;
        __builtin_memcpy(&bits, &bv, 4);
        const uint32_t ob = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(bits), CTRL, 0xf, 0xf, false));
        const int oi = __builtin_amdgcn_update_dpp(0, bi, CTRL, 0xf, 0xf, false);
        KeyT ov;
        __builtin_memcpy(&ov, &ob, 4);
        take(ov, oi);
    };
    step(std::integral_constant<int, 0xB1>{});
    step(std::integral_constant<int, 0x4E>{});
    step(std::integral_constant<int, 0x141>{});
    step(std::integral_constant<int, 0x140>{});
    // the four rows' pairs, read as scalars
    uint32_t bits;
    __builtin_memcpy(&bits, &bv, 4);
    KeyT rv[4];
    int ri[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t b = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(bits), 16 * q));
        __builtin_memcpy(&rv[q], &b, 4);
        ri[q] = __builtin_amdgcn_readlane(bi, 16 * q);
    }
    bv = rv[0];
    bi = ri[0];
#pragma unroll
    for (int q = 1; q < 4; ++q) take(rv[q], ri[q]);
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, lanes_dpp<0xB1>(v));
    v = fmaxf(v, lanes_dpp<0x4E>(v));
    v = fmaxf(v, lanes_dpp<0x141>(v));
    v = fmaxf(v, lanes_dpp<0x140>(v));
    return fmaxf(fmaxf(lane_of(v, 0), lane_of(v, 16)), fmaxf(lane_of(v, 32), lane_of(v, 48)));
}

}  // namespace liyab

#define LIYAB_REQUIRE(cond, ...)                          \
    do {                                                  \
        if (!(cond)) return ::liyab::fail(1, __VA_ARGS__); \
    } while (0)
