// Shared helpers for the gfx950 kernels of libinfllm_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/infllm_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kD = INFLLM_HEAD_DIM;       // head_dim
constexpr int kTile = INFLLM_KEY_TILE;    // keys per tile
constexpr int kWave = 64;

// thread-local error text, returned by infllm_last_error()
char *infllm_err_buf();
int infllm_fail(int code, const char *fmt, ...);

#define INFLLM_REQUIRE(cond, ...)                      \
    do {                                               \
        if (!(cond)) return infllm_fail(-1, __VA_ARGS__); \
    } while (0)

#define INFLLM_CHECK_LAUNCH(name)                                                     \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) return infllm_fail(-2, "%s: %s", name, hipGetErrorString(e_)); \
    } while (0)

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}
// round-to-nearest-even fp32 -> bf16 bits (inputs are finite here; NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
// two fp32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// acc + lo + hi of a packed bf16 pair, exactly (v_dot2c_f32_bf16 against a pair of ones)
__device__ __forceinline__ float sum_bf16x2(uint32_t pair, float acc) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), acc, false);
}
__device__ __forceinline__ float wave_xor32(float x) {
    return __shfl_xor(x, 32, 64);
}
