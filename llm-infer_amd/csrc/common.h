// Shared device helpers for the gfx950 (CDNA4) kernels: element types, wave64
// reductions, MFMA wrappers and the layout of a cache page.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 f16;
typedef __bf16 bf16;

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define WAVE 64
#define PAGE 64   // tokens of a cache page

// dtype codes of the C interface
enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

// status codes of the C interface (0 = launched)
enum { LI_OK = 0, LI_BAD_ARG = 1, LI_UNSUPPORTED = 2, LI_HIP_ERROR = 3 };

template <class T> struct Vec;
template <> struct Vec<f16> { typedef f16x8 v8; typedef f16x4 v4; typedef f16x2 v2; };
template <> struct Vec<bf16> { typedef bf16x8 v8; typedef bf16x4 v4; typedef bf16x2 v2; };

template <class T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <class T> __device__ __forceinline__ T from_f32(float v) { return (T)v; }

__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float dot2(f16x2 a, f16x2 b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }
__device__ __forceinline__ float dot2(bf16x2 a, bf16x2 b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[w] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += scratch[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    v = wave_max(v);
    const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scratch[w] = v;
    __syncthreads();
    float t = scratch[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, scratch[i]);
    return t;
}

// A power of two near 1 / (8 rms) for a row whose root mean square is `rms`: what the rows of a residual
// stream are multiplied by before they are rounded to float16 on their way from one product to the norm
// inside the next (gemm.hip, RowsOut), so that they lie in the middle of that type's range whatever the
// model's own scale.  An element is at most sqrt(width) times the rms, so a row that has grown a hundredfold
// since the rms was taken still fits.
__device__ __forceinline__ float row_scale_for(float rms) {
    int e;
    frexpf(fminf(fmaxf(rms, 1e-30f), 1e30f), &e);        // rms = m 2^e, 0.5 <= m < 1
    return ldexpf(0.125f, -e);
}

// The gate's activation: silu(x) = x / (1 + exp(-x)) (include/kernels_cpu.hpp:186) or the tanh form of
// gelu that the reference computes, 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3)))
// (include/kernels_cpu.hpp:179-184).
__device__ __forceinline__ float gate_activation(float g, bool gelu) {
    if (gelu) return 0.5f * g * (1.f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    return g / (1.f + expf(-g));
}

// ---------------------------------------------------------------------------
// Layout of a cache page.  A page holds PAGE (64) tokens of one layer for all
// KV heads.  Keys and values are stored in the order in which a wave's lanes
// feed them to the 32x32x16 matrix instruction, so that attention reads every
// operand as one contiguous 1 KiB load per wave, with no transposition in LDS.
//
// Keys (operand A of S^T = K Q^T, rows = tokens, inner index = head dim):
//   [kv head][token block b = t/32][step s = d/16][lane = 32*((d%16)/8) + t%32][d%8]
// Values (operand A of O^T = V^T P^T, rows = head dim, inner index = tokens, in the
// order in which the score accumulators hold the tokens):
//   [kv head][dim block d/32][token group t/16][lane = 32*((t%8)/4) + d%32][4*((t%16)/8) + t%4]
// The value part of a page is padded to a multiple of 32 in the head dim.
// ---------------------------------------------------------------------------
__host__ __device__ __forceinline__ int round_up(int a, int b) { return (a + b - 1) / b * b; }

__host__ __device__ __forceinline__ int64_t k_head_elems(int hd) { return (int64_t)PAGE * hd; }
__host__ __device__ __forceinline__ int64_t v_head_elems(int hd) { return (int64_t)PAGE * round_up(hd, 32); }

__host__ __device__ __forceinline__ int k_offset(int t, int d, int hd) {
    const int b = t >> 5, s = d >> 4, lane = (((d & 15) >> 3) << 5) + (t & 31);
    return ((b * (hd >> 4) + s) * 64 + lane) * 8 + (d & 7);
}
__host__ __device__ __forceinline__ int v_offset(int t, int d, int hd) {
    (void)hd;
    const int db = d >> 5, tj = t >> 4, u = t & 15;
    const int lane = (((u & 7) >> 2) << 5) + (d & 31);
    const int idx = ((u >> 3) << 2) + (u & 3);
    return ((db * (PAGE / 16) + tj) * 64 + lane) * 8 + idx;
}

#define LI_CHECK_LAUNCH()                                        \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return LI_HIP_ERROR;               \
    } while (0)
