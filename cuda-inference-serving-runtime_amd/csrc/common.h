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

// The law of a gated activation act(gate, up), the epilogue of a product over [gate; up]:
//   limit <= 0:  silu(g) u
//   limit > 0:   g' sigmoid(slope g') (u' + shift) with g' = min(g, limit), u' = clamp(u, -limit, limit)
// A struct of zeros is the first law.
struct GateLaw { float limit, slope, shift; };

__device__ __forceinline__ float gated_activation(float g, float u, const GateLaw& law) {
    if (law.limit > 0.f) {
        g = fminf(g, law.limit);
        u = fminf(fmaxf(u, -law.limit), law.limit);
        return g / (1.0f + expf(-law.slope * g)) * (u + law.shift);
    }
    return g / (1.0f + expf(-g)) * u;
}

// An ungated activation, the epilogue of a product that feeds a feed-forward's second matrix:
//   1: z Phi(z), the gelu with the error function     2: its tanh form 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))
//   3: relu(z)^2
enum { ACT_NONE = 0, ACT_GELU = 1, ACT_GELU_TANH = 2, ACT_RELU2 = 3 };

__device__ __forceinline__ float unary_activation(float z, int act) {
    if (act == ACT_GELU) return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f));
    if (act == ACT_RELU2) { const float r = fmaxf(z, 0.f); return r * r; }
    return 0.5f * z * (1.0f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
}

// as the epilogue of a product: the sum is rounded to the output's type first, as the path of two kernels does
template <typename TC>
__device__ __forceinline__ float activated(float v, int act) {
    if (sizeof(TC) == 2) v = bf16_to_f32(f32_to_bf16(v));
    return unary_activation(v, act);
}

#define CISR_LAUNCH_CHECK() ((int)hipGetLastError())
