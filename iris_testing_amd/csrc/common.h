// Shared device/host helpers for libmoe_gfx950.so (gfx950 only, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/moe_gfx950.h"

#define WAVE 64

// ---- error text (per calling thread) ---------------------------------------------------------
char* moe_err_buf();
int moe_fail(int code, const char* fmt, ...);
int moe_check_launch(const char* what);

#define MOE_REQUIRE(cond, code, ...)                 \
    do {                                             \
        if (!(cond)) return moe_fail(code, __VA_ARGS__); \
    } while (0)

// ---- bf16 as raw bits ------------------------------------------------------------------------
typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even; NaN stays a (quiet) NaN
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

template <typename T>
__device__ __forceinline__ float load_f32(const T* p);
template <>
__device__ __forceinline__ float load_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }

__device__ __forceinline__ int lane_id() { return threadIdx.x & (WAVE - 1); }

static inline int dtype_size(int dtype) { return dtype == MOE_F32 ? 4 : (dtype == MOE_BF16 ? 2 : 0); }
static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
