// Diagnostic kernels, no part of the hot path: what the matrix cores of this device sustain when nothing else limits them.
// A register-only MFMA loop in the grouped GEMM's wave layout (four waves per compute unit, 128 x 128 outputs per wave: 8 x 8
// MFMAs of 16x16x32 for bf16, 4 x 4 of 32x32x64 for fp8), operands held in registers, no LDS, no memory traffic.  The figure
// depends on the operand VALUES: the chip runs against a power limit, and all-zero operands toggle no multiplier.  bench.py
// --mfma-ceiling times it with both kinds of data; the grouped GEMM's roofline fraction can then be read against what the
// cores deliver on data like the workload's, beside the published peak.
#include "common.h"

namespace {

typedef __bf16 dg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float dg_f4 __attribute__((ext_vector_type(4)));
typedef float dg_f16 __attribute__((ext_vector_type(16)));
typedef int dg_i8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ uint32_t dg_rand(uint32_t& s) {
    s = s * 1664525u + 1013904223u;
    return s ^ (s >> 15);
}
// one N(0,1) sample (Box-Muller on two 24-bit uniforms)
__device__ __forceinline__ float dg_normal(uint32_t& s) {
    const float u1 = ((dg_rand(s) >> 8) + 1) * (1.0f / 16777217.0f), u2 = (dg_rand(s) >> 8) * (1.0f / 16777216.0f);
    return sqrtf(-2.0f * __logf(u1)) * __cosf(6.2831853f * u2);
}
__device__ __forceinline__ uint32_t dg_bf16_pair(uint32_t& s) {
    return (uint32_t)f32_to_bf16(dg_normal(s)) | ((uint32_t)f32_to_bf16(dg_normal(s)) << 16);
}
// four e4m3 codes of N(0,1) samples scaled so that 4 sigma is the largest code (what per-row quantisation of such rows gives)
__device__ __forceinline__ uint32_t dg_fp8_quad(uint32_t& s) {
    int w = 0;
    w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(dg_normal(s) * 112.f, -448.f), 448.f), fminf(fmaxf(dg_normal(s) * 112.f, -448.f), 448.f), w, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(fminf(fmaxf(dg_normal(s) * 112.f, -448.f), 448.f), fminf(fmaxf(dg_normal(s) * 112.f, -448.f), 448.f), w, true);
    return (uint32_t)w;
}

template <bool FP8>
__global__ __launch_bounds__(256, 1) void diag_mfma_loop_kernel(float* __restrict__ sink, int iters, int random_data) {
    uint32_t seed = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
    float r = 0.f;
    if constexpr (FP8) {
        dg_i8 a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                a[i][v] = random_data ? (int)dg_fp8_quad(seed) : 0;
                b[i][v] = random_data ? (int)dg_fp8_quad(seed) : 0;
            }
        dg_f16 acc[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i * 4 + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i * 4 + j], 0, 0, 0, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) r += acc[i][v];
    } else {
        uint4 a[8], b[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a[i] = random_data ? make_uint4(dg_bf16_pair(seed), dg_bf16_pair(seed), dg_bf16_pair(seed), dg_bf16_pair(seed)) : make_uint4(0, 0, 0, 0);
            b[i] = random_data ? make_uint4(dg_bf16_pair(seed), dg_bf16_pair(seed), dg_bf16_pair(seed), dg_bf16_pair(seed)) : make_uint4(0, 0, 0, 0);
        }
        dg_f4 acc[64];
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][v] = 0.f;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    acc[i * 8 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(dg_bf16x8, a[i]), __builtin_bit_cast(dg_bf16x8, b[j]),
                                                                             acc[i * 8 + j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) r += acc[i][v];
    }
    sink[blockIdx.x * 256 + threadIdx.x] = r;
}

}  // namespace

extern "C" size_t moe_diag_mfma_loop_sink_floats(void) { return (size_t)1024 * 256; }

// flops of one launch: workgroups x 4 waves x iters x (128 x 128 outputs x K per iteration x 2)
extern "C" double moe_diag_mfma_loop_flops(int fp8, int iters, int workgroups) {
    return (double)workgroups * 4.0 * (double)iters * 2.0 * 128.0 * 128.0 * (fp8 ? 64.0 : 32.0);
}

extern "C" int moe_diag_mfma_loop(int fp8, int random_data, int iters, int workgroups, float* sink, moe_stream_t stream) {
    MOE_REQUIRE(iters >= 1 && workgroups >= 1 && workgroups <= 1024 && sink, MOE_ERR_INVALID, "diag_mfma_loop: bad arguments");
    if (fp8) diag_mfma_loop_kernel<true><<<workgroups, 256, 0, (hipStream_t)stream>>>(sink, iters, random_data);
    else diag_mfma_loop_kernel<false><<<workgroups, 256, 0, (hipStream_t)stream>>>(sink, iters, random_data);
    return moe_check_launch("diag_mfma_loop");
}
