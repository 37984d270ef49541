// Shared device helpers for the gfx950 kernels: storage types, bf16 conversion,
// wave64 reductions.  Storage precision is separate from arithmetic: every
// reduction, softmax statistic and accumulator is float.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef uint16_t bf16_t;

// dtype codes shared with the Python wrappers
enum { DT_F32 = 0, DT_BF16 = 1 };

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
    return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even, NaN stays NaN (the rule of the reference's kernels/precision.cuh:13-20),
// done by the hardware conversion of gfx950 (v_cvt_pk_bf16_f32)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
    return __builtin_bit_cast(bf16_t, (__bf16)f);
}

// two floats to a pair of bf16 in one register (low half first)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ float load_f32(const float* p) { return *p; }
__device__ __forceinline__ float load_f32(const bf16_t* p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void store_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_f32(bf16_t* p, float v) { *p = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024).  `red`
// is LDS scratch of at least NT/64 floats.  Every thread gets the total.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < NT / WAVE; ++w) total += red[w];
    return total;
}

#define CISR_LAUNCH_CHECK() ((int)hipGetLastError())
