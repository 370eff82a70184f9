// Measuring kernels for the benchmark: what this GPU reaches when a kernel does nothing but
// stream memory, or nothing but matrix-core or FMA arithmetic.  The benchmark reports the
// engine's steps against these measured rates beside the published peaks.  Nothing on the
// product path calls them.
#include "common.h"

struct __attribute__((aligned(16))) probe_v4 { uint32_t w[4]; };

// Read `n16` 16-byte words once, every lane 16 bytes a load, UNROLL loads in flight a lane.
template <int UNROLL>
__global__ __launch_bounds__(256) void probe_read_kernel(const probe_v4* __restrict__ src, size_t n16,
                                                         uint32_t* __restrict__ sink) {
    uint32_t acc = 0;
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        probe_v4 a[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) a[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc += a[u].w[0] ^ a[u].w[1] ^ a[u].w[2] ^ a[u].w[3];
    }
    for (; i < n16; i += stride) { const probe_v4 a = src[i]; acc += a.w[0] ^ a.w[1] ^ a.w[2] ^ a.w[3]; }
    if (acc == 0x9e3779b9u) sink[0] = acc;        // keeps the loads alive; practically never taken
}

template <int UNROLL>
__global__ __launch_bounds__(256) void probe_copy_kernel(const probe_v4* __restrict__ src, probe_v4* __restrict__ dst,
                                                         size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        probe_v4 a[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) a[u] = src[i + u * stride];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) dst[i + u * stride] = a[u];
    }
    for (; i < n16; i += stride) dst[i] = src[i];
}

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));

// Four waves a block, each with four independent chains of 32x32x16 bfloat16 MFMAs on registers.
__global__ __launch_bounds__(256) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
    probe_bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(threadIdx.x * 0.001f + i); b[i] = (__bf16)(i * 0.5f); }
    probe_f32x16 c[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) c[t][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 4; ++t) c[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c[t], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += c[t][r];
    if (s == 12345.f) sink[0] = s;
}

// Eight independent chains of float32 FMAs a lane: the arithmetic of the 32-bit path's products.
__global__ __launch_bounds__(256) void probe_fma_kernel(float* __restrict__ sink, int iters, float x, float y) {
    float c[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) c[t] = threadIdx.x * 0.001f + t;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 8; ++t) c[t] = fmaf(c[t], x, y);
    }
    float s = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t) s += c[t];
    if (s == 12345.f) sink[0] = s;
}

extern "C" int li_probe_read(const void* src, long bytes, void* sink, int blocks, hipStream_t stream) {
    if (bytes < 16 || blocks <= 0 || ((uintptr_t)src & 15)) return LI_ERR_SIZE;
    probe_read_kernel<8><<<blocks, 256, 0, stream>>>((const probe_v4*)src, (size_t)bytes / 16, (uint32_t*)sink);
    return li_launch_status();
}

extern "C" int li_probe_copy(const void* src, void* dst, long bytes, int blocks, hipStream_t stream) {
    if (bytes < 16 || blocks <= 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return LI_ERR_SIZE;
    probe_copy_kernel<4><<<blocks, 256, 0, stream>>>((const probe_v4*)src, (probe_v4*)dst, (size_t)bytes / 16);
    return li_launch_status();
}

// flops of one launch = blocks * 4 waves * iters * 4 MFMAs * 2 * 32 * 32 * 16
extern "C" int li_probe_mfma(void* sink, int blocks, int iters, hipStream_t stream) {
    if (blocks <= 0 || iters <= 0) return LI_ERR_SIZE;
    probe_mfma_kernel<<<blocks, 256, 0, stream>>>((float*)sink, iters);
    return li_launch_status();
}

// flops of one launch = blocks * 256 lanes * iters * 8 FMAs * 2
extern "C" int li_probe_fma(void* sink, int blocks, int iters, hipStream_t stream) {
    if (blocks <= 0 || iters <= 0) return LI_ERR_SIZE;
    probe_fma_kernel<<<blocks, 256, 0, stream>>>((float*)sink, iters, 0.999f, 0.001f);
    return li_launch_status();
}
