// Causal grouped-query attention over the paged cache.
//
// Cache layout per layer: [pages, kv_heads, page_size, head_dim].  The query
// i of segment s stands at position p = ctx_len[s] - q_len[s] + i and sees the
// keys at positions max(0, p - window + 1) .. p (window 0: from 0).  Key t of a
// segment lies in page block_table[s][t / page_size] at offset t % page_size.
// Scores, the running maximum, the exponentials, the sums and the final
// division are float32 (online softmax); the output is rounded once.
#include "common.h"
#include <math.h>

#define ATT_MAX_DH 256

// One wave per (token, head).  Keys are taken 64 at a time: lane j computes the
// score of key j, the wave agrees on the new maximum, and then every lane owns
// head dimensions d = lane, lane + 64, ... of the weighted sum of values.
template <typename T>
__global__ __launch_bounds__(64) void paged_attention_wave_kernel(
    const T* __restrict__ q, int q_row_stride, T* __restrict__ out, const T* __restrict__ kc,
    const T* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ seg_of_token, const int* __restrict__ q_start,
    const int* __restrict__ q_len, const int* __restrict__ ctx_len, int nh, int nkv, int dh,
    int page_size, int num_pages, int window, float scale) {
    __shared__ float qs[ATT_MAX_DH];
    __shared__ float ps[LI_WAVE];
    __shared__ int rowoff[LI_WAVE];          // element offset / dh of each key's row, -1 = not there
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int kvh = h / (nh / nkv);
    const int* table = block_table + (size_t)s * max_blocks;
    const T* qrow = q + (size_t)t * q_row_stride + (size_t)h * dh;
    for (int d = lane; d < dh; d += LI_WAVE) qs[d] = load_as_float(qrow + d);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ATT_MAX_DH / LI_WAVE] = {0.f, 0.f, 0.f, 0.f};
    for (int t0 = lo; t0 <= p; t0 += LI_WAVE) {
        const int key = t0 + lane;
        float sc = -INFINITY;
        int ro = -1;
        if (key <= p) {
            const int page = table[key / page_size];
            if (page >= 0 && page < num_pages) {
                ro = (page * nkv + kvh) * page_size + key % page_size;
                const T* krow = kc + (size_t)ro * dh;
                float dot = 0.f;
                for (int d = 0; d < dh; ++d) dot = fmaf(qs[d], load_as_float(krow + d), dot);
                sc = dot * scale;
            }
        }
        const float m_new = fmaxf(m, wave_max(sc));
        const float alpha = (l == 0.f) ? 0.f : expf(m - m_new);
        const float e = (ro >= 0) ? expf(sc - m_new) : 0.f;
        l = l * alpha + wave_sum(e);
        __syncthreads();
        ps[lane] = e;
        rowoff[lane] = ro;
        __syncthreads();
        const int nkeys = (p - t0 + 1 < LI_WAVE) ? p - t0 + 1 : LI_WAVE;
#pragma unroll
        for (int c = 0; c < ATT_MAX_DH / LI_WAVE; ++c) {
            const int d = lane + c * LI_WAVE;
            if (d < dh) {
                float a = acc[c] * alpha;
                for (int j = 0; j < nkeys; ++j) {
                    const int r = rowoff[j];
                    if (r >= 0) a = fmaf(ps[j], load_as_float(vc + (size_t)r * dh + d), a);
                }
                acc[c] = a;
            }
        }
        m = m_new;
    }
    T* orow = out + (size_t)t * nh * dh + (size_t)h * dh;
#pragma unroll
    for (int c = 0; c < ATT_MAX_DH / LI_WAVE; ++c) {
        const int d = lane + c * LI_WAVE;
        if (d < dh) store_from_float(orow + d, l != 0.f ? acc[c] / l : 0.f);
    }
}

extern "C" int li_paged_attention(const void* q, int q_row_stride, void* out, const void* kc,
                                  const void* vc, int dtype, const int* block_table, int max_blocks,
                                  const int* seg_of_token, const int* q_start, const int* q_len,
                                  const int* ctx_len, int num_segments, int T, int max_q_len,
                                  int max_ctx_len, int nh, int nkv, int dh, int page_size,
                                  int num_pages, int window, float scale, hipStream_t stream) {
    if (T <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || dh <= 0 || dh > ATT_MAX_DH || nh > 65535 ||
        page_size <= 0 || max_blocks <= 0)
        return LI_ERR_SIZE;
    dim3 grid(T, nh);
    if (dtype == LI_F32)
        paged_attention_wave_kernel<float><<<grid, 64, 0, stream>>>(
            (const float*)q, q_row_stride, (float*)out, (const float*)kc, (const float*)vc, block_table,
            max_blocks, seg_of_token, q_start, q_len, ctx_len, nh, nkv, dh, page_size, num_pages, window, scale);
    else if (dtype == LI_BF16)
        paged_attention_wave_kernel<bf16_t><<<grid, 64, 0, stream>>>(
            (const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, block_table,
            max_blocks, seg_of_token, q_start, q_len, ctx_len, nh, nkv, dh, page_size, num_pages, window, scale);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
