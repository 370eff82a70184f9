// Choosing the next token from float32 logits: argmax (lowest index on ties)
// and temperature / top-k / top-p sampling by inverse CDF with a uniform
// number that the host derives from the request's own counter-based stream.
#include "common.h"
#include <math.h>

#define SMP_NT 1024

// (value, index) maximum with the lower index winning ties
__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi) {
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

__device__ __forceinline__ void block_argmax(float& v, int& i, float* sv, int* si) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, LI_WAVE);
        const int oi = __shfl_xor(i, o, LI_WAVE);
        argmax_combine(v, i, ov, oi);
    }
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) { sv[w] = v; si[w] = i; }
    __syncthreads();
    v = sv[0]; i = si[0];
    for (int k = 1; k < SMP_NT / LI_WAVE; ++k) argmax_combine(v, i, sv[k], si[k]);
}

__global__ __launch_bounds__(SMP_NT) void argmax_rows_kernel(const float* __restrict__ logits,
                                                             int* __restrict__ out, int V) {
    __shared__ float sv[SMP_NT / LI_WAVE];
    __shared__ int si[SMP_NT / LI_WAVE];
    const float* row = logits + (size_t)blockIdx.x * V;
    float v = -INFINITY;
    int i = 0x7fffffff;
    for (int j = threadIdx.x; j < V; j += SMP_NT) {
        const float x = row[j];
        if (x > v || i == 0x7fffffff) { v = x; i = j; }   // strictly greater: the first maximum stays
    }
    block_argmax(v, i, sv, si);
    if (threadIdx.x == 0) out[blockIdx.x] = i;
}

extern "C" int li_argmax_rows(const float* logits, int* out, int n, int V, hipStream_t stream) {
    if (n <= 0 || V <= 0) return LI_ERR_SIZE;
    argmax_rows_kernel<<<n, SMP_NT, 0, stream>>>(logits, out, V);
    return li_launch_status();
}
