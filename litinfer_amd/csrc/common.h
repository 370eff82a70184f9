// Shared device helpers for the gfx950 kernels: element types, conversions,
// wave and block reductions with a fixed order.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LI_OK 0
#define LI_ERR_DTYPE 1
#define LI_ERR_SIZE 2
#define LI_ERR_LAUNCH 3

#define LI_F32 0
#define LI_BF16 1

#define LI_WAVE 64

struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_float(uint16_t b) {
    return __uint_as_float(((uint32_t)b) << 16);
}

// round to nearest even; NaN stays NaN (v_cvt_pk_bf16_f32, one instruction for one or two values)
__device__ __forceinline__ uint16_t float_to_bf16(float f) {
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

typedef __bf16 li_bf16x2 __attribute__((ext_vector_type(2)));
typedef float li_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {      // lo in bits 0..15
    li_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, li_bf16x2));
}

__device__ __forceinline__ float load_as_float(const float* p) { return *p; }
__device__ __forceinline__ float load_as_float(const bf16_t* p) { return bf16_to_float(p->bits); }
__device__ __forceinline__ void store_from_float(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_from_float(bf16_t* p, float v) { p->bits = float_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LI_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, LI_WAVE));
    return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every
// thread gets the result.  The order of additions depends on NT only.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* smem /* NT/64 floats */) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NT / LI_WAVE; ++i) t += smem[i];
    return t;
}

static inline int li_launch_status() {
    return hipGetLastError() == hipSuccess ? LI_OK : LI_ERR_LAUNCH;
}
