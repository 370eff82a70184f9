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
    const int* __restrict__ token_list, const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int nh, int nkv, int dh, int page_size, int num_pages, int window, float scale) {
    __shared__ float qs[ATT_MAX_DH];
    __shared__ float ps[LI_WAVE];
    __shared__ int rowoff[LI_WAVE];          // element offset / dh of each key's row, -1 = not there
    const int t = token_list ? token_list[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
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

// ------------------------------------------------------ single-query tokens
// Decode: one query per sequence, so the work is reading the keys and values
// once.  A block of 4 waves takes one (token, kv head, split of the keys) and
// all the query heads of that kv head, so a page is read once for the whole
// group.  A key's row is spread over LPK lanes (16 bytes each); a wave handles
// 64 / LPK keys a round and U rounds are in flight.  Every lane group keeps an
// online softmax (m, l, acc) per head over its keys; the groups of a wave are
// merged by a butterfly, the waves through LDS in wave order, the splits by
// `attention_merge_kernel` in split order: all fixed orders.
template <typename T> struct raw16;
template <> struct raw16<bf16_t> { static constexpr int E = 8; };
template <> struct raw16<float> { static constexpr int E = 4; };

struct __attribute__((aligned(16))) u32x4 { uint32_t w[4]; };

template <typename T, int E>
__device__ __forceinline__ void unpack16(const u32x4& r, float* f) {
    if constexpr (E == 8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(r.w[i] << 16);
            f[2 * i + 1] = __uint_as_float(r.w[i] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(r.w[i]);
    }
}

// Sum over the LPK lanes that share a key; every one of them gets the total.
// Steps within a row of 16 lanes are DPP moves inside the vector ALU (swap
// neighbours, swap pairs, mirror the half row, mirror the row), which keep
// their place in the instruction stream; only steps across rows go through
// the LDS crossbar.
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
    if constexpr (LPK >= 2) v = dpp_add<0xB1>(v);      // quad_perm [1,0,3,2]
    if constexpr (LPK >= 4) v = dpp_add<0x4E>(v);      // quad_perm [2,3,0,1]
    if constexpr (LPK >= 8) v = dpp_add<0x141>(v);     // row_half_mirror
    if constexpr (LPK >= 16) v = dpp_add<0x140>(v);    // row_mirror
    if constexpr (LPK >= 32) v += __shfl_xor(v, 16, LI_WAVE);
    if constexpr (LPK >= 64) v += __shfl_xor(v, 32, LI_WAVE);
    return v;
}

__device__ __forceinline__ void softmax_merge(float& m, float& l, float* acc, int n, float mo, float lo,
                                              const float* acco) {
    const float mx = fmaxf(m, mo);
    if (mx == -INFINITY) return;                       // both sides empty
    const float a = expf(m - mx), b = expf(mo - mx);   // exp(-inf) = 0 for an empty side
    l = l * a + lo * b;
    for (int j = 0; j < n; ++j) acc[j] = acc[j] * a + acco[j] * b;
    m = mx;
}

template <typename T, int LPK, int GB>
__global__ __launch_bounds__(256) void paged_attention_decode_kernel(
    const T* __restrict__ q, int q_row_stride, T* __restrict__ out, const T* __restrict__ kc,
    const T* __restrict__ vc, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ token_list, const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    float* __restrict__ part_acc, float* __restrict__ part_ml, int nh, int nkv, int dh, int page_size,
    int num_pages, int window, float scale, int nsplit) {
    constexpr int E = raw16<T>::E;
    constexpr int KPW = 64 / LPK;
    constexpr int U = 4;
    __shared__ float sm_acc[4][GB][ATT_MAX_DH];
    __shared__ float sm_ml[4][GB][2];
    const int ti = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
    const int t = token_list ? token_list[ti] : ti;
    const int G = nh / nkv;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int nkeys = p - lo + 1;
    const int per = (((nkeys + nsplit - 1) / nsplit) + 63) & ~63;
    const int k_begin = lo + split * per;
    const int k_end = (k_begin + per < p + 1) ? k_begin + per : p + 1;
    const int* table = block_table + (size_t)s * max_blocks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int grp = lane / LPK, sub = lane % LPK;
    const int d0 = sub * E;

    for (int h0 = 0; h0 < G; h0 += GB) {
        const int gcount = (G - h0 < GB) ? G - h0 : GB;
        float qr[GB][E], acc[GB][E], m[GB], l[GB];
#pragma unroll
        for (int h = 0; h < GB; ++h) {
            m[h] = -INFINITY;
            l[h] = 0.f;
#pragma unroll
            for (int j = 0; j < E; ++j) { acc[h][j] = 0.f; qr[h][j] = 0.f; }
            if (h < gcount) {
                const T* qp = q + (size_t)t * q_row_stride + (size_t)(kvh * G + h0 + h) * dh + d0;
                u32x4 r = *reinterpret_cast<const u32x4*>(qp);
                unpack16<T, E>(r, qr[h]);
            }
        }
        for (int r0 = 0;; r0 += U) {
            const int wbase = k_begin + (r0 * 4 + wave) * KPW;
            if (wbase >= k_end) break;
            u32x4 kraw[U], vraw[U];
            bool ok[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int key = wbase + u * 4 * KPW + grp;
                ok[u] = key < k_end;
                kraw[u] = u32x4{{0u, 0u, 0u, 0u}};
                vraw[u] = kraw[u];
                if (ok[u]) {
                    const int page = table[key / page_size];
                    ok[u] = page >= 0 && page < num_pages;
                    if (ok[u]) {
                        const size_t off = (((size_t)page * nkv + kvh) * page_size + key % page_size) * dh + d0;
                        kraw[u] = *reinterpret_cast<const u32x4*>(kc + off);
                        vraw[u] = *reinterpret_cast<const u32x4*>(vc + off);
                    }
                }
            }
            float sc[U][GB];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float kf[E];
                unpack16<T, E>(kraw[u], kf);
#pragma unroll
                for (int h = 0; h < GB; ++h) {
                    float dot = 0.f;
#pragma unroll
                    for (int j = 0; j < E; ++j) dot = fmaf(qr[h][j], kf[j], dot);
                    dot = group_sum<LPK>(dot);
                    sc[u][h] = ok[u] ? dot * scale : -INFINITY;
                }
            }
            float vf[U][E];
#pragma unroll
            for (int u = 0; u < U; ++u) unpack16<T, E>(vraw[u], vf[u]);
#pragma unroll
            for (int h = 0; h < GB; ++h) {
                float mx = m[h];
#pragma unroll
                for (int u = 0; u < U; ++u) mx = fmaxf(mx, sc[u][h]);
                if (mx == -INFINITY) continue;
                const float alpha = expf(m[h] - mx);
                float pu[U], ps = 0.f;
#pragma unroll
                for (int u = 0; u < U; ++u) { pu[u] = expf(sc[u][h] - mx); ps += pu[u]; }
                l[h] = l[h] * alpha + ps;
#pragma unroll
                for (int j = 0; j < E; ++j) {
                    float a = acc[h][j] * alpha;
#pragma unroll
                    for (int u = 0; u < U; ++u) a = fmaf(pu[u], vf[u][j], a);
                    acc[h][j] = a;
                }
                m[h] = mx;
            }
        }
        // the lane groups of the wave
#pragma unroll
        for (int o = LPK; o < 64; o <<= 1) {
#pragma unroll
            for (int h = 0; h < GB; ++h) {
                const float mo = __shfl_xor(m[h], o, LI_WAVE), lo2 = __shfl_xor(l[h], o, LI_WAVE);
                float ao[E];
#pragma unroll
                for (int j = 0; j < E; ++j) ao[j] = __shfl_xor(acc[h][j], o, LI_WAVE);
                softmax_merge(m[h], l[h], acc[h], E, mo, lo2, ao);
            }
        }
        __syncthreads();                               // the last pass's readers are done
        if (grp == 0) {
#pragma unroll
            for (int h = 0; h < GB; ++h) {
#pragma unroll
                for (int j = 0; j < E; ++j) sm_acc[wave][h][d0 + j] = acc[h][j];
                if (sub == 0) { sm_ml[wave][h][0] = m[h]; sm_ml[wave][h][1] = l[h]; }
            }
        }
        __syncthreads();
        for (int idx = threadIdx.x; idx < gcount * dh; idx += 256) {
            const int h = idx / dh, d = idx - h * dh;
            float mx = sm_ml[0][h][0];
#pragma unroll
            for (int w = 1; w < 4; ++w) mx = fmaxf(mx, sm_ml[w][h][0]);
            float lt = 0.f, at = 0.f;
            if (mx != -INFINITY) {
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float f = expf(sm_ml[w][h][0] - mx);
                    lt += sm_ml[w][h][1] * f;
                    at += sm_acc[w][h][d] * f;
                }
            }
            const int head = kvh * G + h0 + h;
            if (nsplit == 1) {
                store_from_float(out + (size_t)t * nh * dh + (size_t)head * dh + d, lt != 0.f ? at / lt : 0.f);
            } else {
                const size_t pi = ((size_t)ti * nh + head) * nsplit + split;
                part_acc[pi * dh + d] = at;
                if (d == 0) { part_ml[pi * 2] = mx; part_ml[pi * 2 + 1] = lt; }
            }
        }
    }
}

// Merging the splits of a (token, head), in split order.  The weights exp(m_s - m) are
// computed once per split by the first lanes, then every thread adds up one output
// dimension with all its loads independent of each other.
#define MERGE_MAX_SPLITS 64

template <typename T>
__global__ __launch_bounds__(128) void attention_merge_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int* __restrict__ token_list, T* __restrict__ out, int nh, int dh, int nsplit_all,
    const int* __restrict__ nruns = nullptr) {
    __shared__ float wgt[MERGE_MAX_SPLITS];
    __shared__ float inv_l;
    const int ti = blockIdx.x, head = blockIdx.y;
    const int t = token_list ? token_list[ti] : ti;
    const size_t base = ((size_t)ti * nh + head) * nsplit_all;
    // nruns: the token's runs that were written (the others of its nsplit_all places hold anything)
    int nsplit = nsplit_all;
    if (nruns) {
        nsplit = nruns[ti];
        nsplit = nsplit < 1 ? 1 : (nsplit > nsplit_all ? nsplit_all : nsplit);
    }
    // The partial results of this thread's first dimension are asked for before the weights
    // are known (up to 32 splits, all loads at once and never conditional): their way from
    // memory then runs beside the weights' way and arithmetic, not behind them.
    constexpr int AHEAD = 32;
    float pa[AHEAD];
    const int d0 = threadIdx.x < dh ? threadIdx.x : 0;
    if (nruns) {                                     // (the number of runs is not known yet: the first place is always written)
#pragma unroll
        for (int sp = 0; sp < AHEAD; ++sp) pa[sp] = part_acc[(base + (sp < nsplit_all ? sp : 0)) * dh + d0];
    } else {
#pragma unroll
        for (int sp = 0; sp < AHEAD; ++sp) pa[sp] = part_acc[(base + (sp < nsplit ? sp : nsplit - 1)) * dh + d0];
    }
    if (threadIdx.x < 64) {
        const int sp = threadIdx.x;
        const float ms = sp < nsplit ? part_ml[(base + sp) * 2] : -INFINITY;
        const float ls = sp < nsplit ? part_ml[(base + sp) * 2 + 1] : 0.f;
        const float mx = wave_max(ms);
        const float f = (mx == -INFINITY) ? 0.f : expf(ms - mx);
        if (sp < nsplit) wgt[sp] = f;
        // the sum over splits in split order (one lane adds them up: at most 64 terms)
        float lt = 0.f;
        for (int i = 0; i < nsplit; ++i) lt += __shfl(ls * f, i, LI_WAVE);
        if (sp == 0) inv_l = lt != 0.f ? 1.0f / lt : 0.f;
    }
    __syncthreads();
    for (int d = threadIdx.x; d < dh; d += 128) {
        float at = 0.f;
        if (d == d0) {                               // (the same order of additions as below)
#pragma unroll
            for (int sp = 0; sp < AHEAD; ++sp) at += sp < nsplit ? pa[sp] * wgt[sp] : 0.f;
#pragma unroll 8
            for (int sp = AHEAD; sp < nsplit; ++sp) at += part_acc[(base + sp) * dh + d] * wgt[sp];
        } else {
#pragma unroll 8
            for (int sp = 0; sp < nsplit; ++sp) at += part_acc[(base + sp) * dh + d] * wgt[sp];
        }
        store_from_float(out + (size_t)t * nh * dh + (size_t)head * dh + d, at * inv_l);
    }
}

// The same for the runs of a prompt portion's keys, whose tokens are many: a block takes four heads of a
// token (a block per token and head, as above, is tens of thousands of blocks with little to do each).
// The partial results lie by the token's row in the batch.  Up to MERGE_RUNS_MAX runs.
#define MERGE_RUNS_MAX 16
#define MERGE_RUNS_HEADS 4
template <typename T>
__global__ __launch_bounds__(256) void attention_merge_runs_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml,
    const int* __restrict__ token_list, T* __restrict__ out, int nh, int dh, int runs) {
    __shared__ float wgt[MERGE_RUNS_HEADS][MERGE_RUNS_MAX];
    __shared__ float inv[MERGE_RUNS_HEADS];
    const int ti = blockIdx.x, h0 = blockIdx.y * MERGE_RUNS_HEADS;
    const int heads = nh - h0 < MERGE_RUNS_HEADS ? nh - h0 : MERGE_RUNS_HEADS;
    const int t = token_list ? token_list[ti] : ti;
    const size_t base = ((size_t)t * nh + h0) * runs;
    if (threadIdx.x < heads) {
        const float* ml = part_ml + (base + (size_t)threadIdx.x * runs) * 2;
        float mx = -INFINITY;
        for (int sp = 0; sp < runs; ++sp) mx = fmaxf(mx, ml[2 * sp]);
        float lt = 0.f;                          // the sum over the runs in their order
        for (int sp = 0; sp < runs; ++sp) {
            const float f = (mx == -INFINITY) ? 0.f : expf(ml[2 * sp] - mx);
            wgt[threadIdx.x][sp] = f;
            lt += ml[2 * sp + 1] * f;
        }
        inv[threadIdx.x] = lt != 0.f ? 1.0f / lt : 0.f;
    }
    __syncthreads();
    const int n = heads * dh;
    for (int i = threadIdx.x; i < n; i += 256) {
        const int hd = i / dh, d = i - hd * dh;
        const float* pa = part_acc + (base + (size_t)hd * runs) * dh + d;
        float v[MERGE_RUNS_MAX];
#pragma unroll
        for (int sp = 0; sp < MERGE_RUNS_MAX; ++sp) v[sp] = pa[(size_t)(sp < runs ? sp : runs - 1) * dh];    // (all loads at once, never conditional)
        float at = 0.f;
#pragma unroll
        for (int sp = 0; sp < MERGE_RUNS_MAX; ++sp) at += sp < runs ? v[sp] * wgt[hd][sp] : 0.f;
        store_from_float(out + ((size_t)t * nh + h0) * dh + i, at * inv[hd]);
    }
}

// ---------------------------------------- single-query tokens, bfloat16, MFMA
// One WAVE per (token, kv head, split of the keys); up to 16 query heads of the
// kv head form the rows of the MFMA tiles, so the keys and values are read
// once for the whole group and nothing is reduced across lanes per key.
// Per block of 32 keys:
//   S[16 heads, 32 keys] = Q K^T by v_mfma_f32_16x16x32_bf16 (row operand Q,
//   column operand K; lane l holds row/column l % 16 and the 8 head dimensions
//   (DH/4) * (l / 16) + 8 j .. + 7 in step j: both operands share that order);
//   the result's register r of lane l is head 4 * (l / 16) + r, key l % 16.
//   Online softmax per head: a row's 16 keys lie in the 16 lanes of one DPP row.
//   P goes through LDS as bfloat16 to become the row operand of P V.
//   V[32 keys, DH]: lane (c = l % 16, g = l / 16) loads 8 dimensions 8c .. 8c+7
//   of the keys 8g .. 8g+7 and transposes them in registers, so MFMA jj yields
//   the output dimension 8c + jj in column c.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true)));
}
__device__ __forceinline__ float row16_max(float v) {
    v = dpp_max<0xB1>(v); v = dpp_max<0x4E>(v); v = dpp_max<0x141>(v); v = dpp_max<0x140>(v);
    return v;
}
__device__ __forceinline__ float row16_sum(float v) { return group_sum<16>(v); }

// The larger of a lane's value and that of the lane 32 further on (or back), inside the vector ALU:
// v_permlane32_swap exchanges the upper half of its first operand with the lower half of its second, so that
// with the same value in both, one result holds the lower half's value in every lane and the other the upper
// half's.  (A shuffle across the halves goes through the LDS crossbar, and its wait is a wait for every LDS
// read before it.)
__device__ __forceinline__ float both_halves_max(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

union frag8 { u32x4 raw; bf16x8_t v; };

// Loads in these kernels are never conditional: a load under a branch is waited for at once,
// and so is one whose result is replaced by zeros right away.  A key that must not be read is
// replaced by the nearest one of the same request that may (its score is masked to -inf, so its
// probability is exactly 0 and the finite value it brings adds nothing); a lane without a head or
// a dimension of its own repeats a neighbour's work and stores nothing.

// Orders a wave's own LDS writes before its own later LDS reads (other lanes' data included: a wave's LDS
// instructions are carried out in the order of their issue), without the block's barrier.
__device__ __forceinline__ void wave_lds_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Stores and loads that other compute units' blocks of the SAME kernel can rely on: they go through to
// memory (each of the chip's eight L2 caches serves its own compute units only, and ordinary stores may
// stay in the writer's).  A device-wide fence would do the same for ordinary accesses, but it writes back
// and invalidates a whole L2 every time: with hundreds of blocks doing so a decode attention took 27 us more.
__device__ __forceinline__ void store_through(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_through(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// two floats that lie side by side (8-byte aligned), in one load
__device__ __forceinline__ void load_through2(const float* p, float& a, float& b) {
    const unsigned long long v = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
    a = __uint_as_float((unsigned)(v & 0xffffffffull));
    b = __uint_as_float((unsigned)(v >> 32));
}
// all of this wave's loads and stores have been carried out (stores: have arrived where they go)
#define LI_WAIT_ALL_VMEM() __builtin_amdgcn_s_waitcnt(0x0F70)

#define DEC_TABLE_CAP 1024      // pages of one split that fit the kernel's copy of the block table

// The most pages one of `nsplit` splits can touch, for block tables of max_blocks pages.
extern "C" long li_decode_split_blocks(int max_blocks, int page_size, int window, int nsplit) {
    if (max_blocks <= 0 || page_size <= 0 || nsplit <= 0) return -1;
    long keys = (long)max_blocks * page_size;
    if (window > 0 && window < keys) keys = window;
    const long per = (((keys + nsplit - 1) / nsplit) + 31) & ~31L;
    return (per + page_size - 2) / page_size + 1;
}

// The length of a run of keys for the decode kernel below, chosen on the device for the batch at hand
// (a recorded step is replayed for other context lengths than it was recorded with).  Cut into nsplit
// runs each, tokens with short contexts would give short waves and the longest context would set the
// time; with one run length for all of them a short context fills few of its nsplit runs (the others
// find no keys and end at once) and the waves that work are equally long.  Every candidate length
// (multiples of 32, from what the longest context needs to fit nsplit runs up to what the block
// table's width would need) costs rounds of the working waves over the SIMDs x (length + a wave's
// start and end, 24 keys' time); the cheapest is taken, of equal ones the shortest.  out: [0] that length,
// [1] the number of (token, run) items, i.e. of runs with keys, [2 .. 2 + n_tokens) the runs of every token,
// then the items, token | run << 16, a token's runs in a row: the decode kernel starts a block for every
// item the grid could hold (tokens x nsplit) and those beyond [1] end at once, without a look at their
// token.  At most RUN_KEYS_MAX_TOKENS tokens (the host checks).
// `group` > 1: the decode kernel's blocks take `group` runs of a token that follow each other, one a wave
// (a block with fewer runs still holds `group` SIMDs): the items are then the FIRST runs of such groups
// (run 0, group, 2 group, ...), [1] counts them, and a candidate length costs its groups x `group` waves.
#define RUN_KEYS_MAX_TOKENS 4096
__global__ __launch_bounds__(256) void decode_run_keys_kernel(
    const int* __restrict__ token_list, int n_tokens, const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    int cap_keys, int window, int nkv, int nsplit, int simds, int group, int* __restrict__ out) {
    __shared__ int nkeys[RUN_KEYS_MAX_TOKENS];
    __shared__ int red_i[4];
    __shared__ unsigned long long red_c[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (n_tokens > RUN_KEYS_MAX_TOKENS) return;      // (refused by the host)
    int mx = 0;
    for (int i = tid; i < n_tokens; i += 256) {
        const int t = token_list ? token_list[i] : i;
        const int s = seg_of_token[t];
        const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
        const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
        const int n = p - lo + 1;
        nkeys[i] = n;
        mx = n > mx ? n : mx;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { const int v = __shfl_xor(mx, o, 64); mx = v > mx ? v : mx; }
    if (lane == 0) red_i[wave] = mx;
    __syncthreads();
    mx = red_i[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) mx = red_i[w] > mx ? red_i[w] : mx;
    const int lower = (((mx + nsplit - 1) / nsplit) + 31) & ~31;
    int cap = (((cap_keys + nsplit - 1) / nsplit) + 31) & ~31;
    cap = cap < lower ? lower : cap;
    const int ncand = (cap - lower) / 32 + 1;
    const int stride = (ncand + 255) / 256;             // (more candidates than threads: every stride-th)
    // cost and length in one number: the least of them is the cheapest, of equal ones the shortest
    unsigned long long best = ~0ull;
    const int c = lower + 32 * stride * tid;
    if (c <= cap) {
        long waves = 0;
        for (int i = 0; i < n_tokens; ++i) waves += ((nkeys[i] + c - 1) / c + group - 1) / group * group;
        waves *= nkv;
        const long rounds = (waves + simds - 1) / simds;
        best = ((unsigned long long)(rounds * (c + 24)) << 32) | (unsigned)c;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long v = __shfl_xor(best, o, 64);
        best = v < best ? v : best;
    }
    __syncthreads();
    if (lane == 0) red_c[wave] = best;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 4; ++w) best = red_c[w] < best ? red_c[w] : best;
    const int per = (int)(unsigned)(best & 0xffffffffull);
    // the runs of every token at that length, and the (token, run) items one after the other: thread t
    // takes a stretch of tokens, the stretches' first items come from a scan over the threads
    __shared__ int first[256];
    const int each = (n_tokens + 255) / 256;
    const int i0 = tid * each, i1 = i0 + each < n_tokens ? i0 + each : n_tokens;
    int mine = 0;
    for (int i = i0; i < i1; ++i) mine += ((nkeys[i] + per - 1) / per + group - 1) / group;
    first[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int w = 0; w < 256; ++w) { const int n = first[w]; first[w] = at; at += n; }
        out[0] = per;
        out[1] = at;
    }
    __syncthreads();
    int at = first[tid];
    int* nruns = out + 2;
    int* items = out + 2 + n_tokens;
    for (int i = i0; i < i1; ++i) {
        const int n = (nkeys[i] + per - 1) / per;
        nruns[i] = n;
        const int ng = (n + group - 1) / group;
        for (int r = 0; r < ng; ++r) items[at + r] = i | ((r * group) << 16);
        at += ng;
    }
}

extern "C" int li_decode_run_keys(const int* token_list, int n_tokens, const int* seg_of_token, const int* q_start,
                                  const int* q_len, const int* ctx_len, int max_blocks, int page_size, int window,
                                  int nkv, int nsplit, int simds, int group, int* out, hipStream_t stream) {
    if (n_tokens <= 0 || n_tokens > RUN_KEYS_MAX_TOKENS || max_blocks <= 0 || page_size <= 0 || nkv <= 0 ||
        nsplit <= 0 || nsplit > 0x7fff || simds <= 0 || group <= 0 || !out)
        return LI_ERR_SIZE;
    long keys = (long)max_blocks * page_size;
    if (window > 0 && window < keys) keys = window;
    if (keys > 0x7fffffffL - 64) return LI_ERR_SIZE;
    decode_run_keys_kernel<<<1, 256, 0, stream>>>(token_list, n_tokens, seg_of_token, q_start, q_len, ctx_len,
                                                  (int)keys, window, nkv, nsplit, simds, group, out);
    return li_launch_status();
}

// WAVES is 1 or 4.  With four, a block takes four runs of the keys of its (token, kv head) that follow each
// other, one a wave (a wave works alone through its run: no barrier in the loop, the runs' lengths may differ),
// and joins their results in LDS, in the order of the runs; `nsplit` then counts such blocks ("quads") and is
// the number of partial results a (token, head) has in part_acc / part_ml.  With one quad the block writes
// the output itself.  With more, the block that finishes last for a (token, kv head) joins the quads'
// results in quad order and writes the output, so that no second kernel is needed: every block adds 1 to
// `done[token * nkv + kv head]` after its results have been made visible to the device, and the block that
// finds the count complete sets it back to 0 (the array is zero before the first call and after every
// call).  Nobody waits for anybody.
template <int WAVES> struct DecodeJoin {
    float ml[WAVES][16][2];                       // per wave and head of the pass: maximum, sum
    float acc[WAVES][16][ATT_MAX_DH / 2];         // per wave and head: the unscaled output (DH <= 128)
    int last;
};
template <> struct DecodeJoin<1> { int last; };

template <typename T, int DH, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void paged_attention_decode_mfma_kernel(
    const T* __restrict__ q, int q_row_stride, T* __restrict__ out,
    const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ token_list, const int* __restrict__ seg_of_token,
    const int* __restrict__ q_start, const int* __restrict__ q_len, const int* __restrict__ ctx_len,
    float* __restrict__ part_acc, float* __restrict__ part_ml, int nh, int nkv, int page_size,
    int num_pages, int window, float scale, int nsplit, const int* __restrict__ run_keys, int n_list,
    int* __restrict__ done) {
    static_assert(DH <= ATT_MAX_DH / 2, "the join buffer holds head sizes up to 128");
    constexpr bool F32 = sizeof(T) == 4;        // float32: v_mfma_f32_16x16x4f32 on float32 operands
    constexpr int KS = DH / 32;                 // bfloat16: MFMA steps of Q K^T
    constexpr int NS = (DH + 127) / 128;        // bfloat16: slabs of 128 output dimensions
    constexpr int QD = DH / 4;                  // head dimensions owned by one lane group in Q K^T
    constexpr int KJ = QD / 4;                  // float32: 16-byte pieces of those
    constexpr int NP = (DH + 63) / 64;          // float32: slabs of 64 output dimensions
    // the output's registers: acc[i] holds, for the lane's four heads, dimension dim_of(i) (below)
    constexpr int NACC = F32 ? 4 * NP : 8 * NS;
    constexpr int PSTRIDE = F32 ? 36 : 40;      // elements per row of P in LDS (32 keys + pad; rows 16-byte aligned)
    __shared__ __attribute__((aligned(16))) T p_lds_all[WAVES][16 * PSTRIDE];
    __shared__ int pages_all[WAVES][DEC_TABLE_CAP];
    __shared__ DecodeJoin<WAVES> join;
    const int wave = WAVES > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
    T* p_lds = p_lds_all[wave];
    int* pages = pages_all[wave];
    const int nruns_all = nsplit * WAVES;       // runs that the keys are cut into at most
    // run_keys given: block x takes the x-th item of the list behind it, a (token, first run) pair, and ends
    // at once if the list is shorter (blocks go to the XCDs in turn, in the order of their numbers, so every
    // XCD gets its share of the runs that have keys).  Else block (token, kv head, quad) of the grid.
    int ti = blockIdx.x, quad = blockIdx.z;
    const int kvh = blockIdx.y;
    int quads_of_token = nsplit;
    if (run_keys) {
        const int count = run_keys[1];
        const int item = run_keys[2 + n_list + blockIdx.x];
        if ((int)blockIdx.x >= count) return;
        ti = item & 0xffff;
        quad = (item >> 16) / WAVES;
        const int nr = run_keys[2 + ti];
        quads_of_token = (nr + WAVES - 1) / WAVES;
        quads_of_token = quads_of_token < 1 ? 1 : (quads_of_token > nsplit ? nsplit : quads_of_token);
    }
    const int split = quad * WAVES + wave;
    const int t = token_list ? token_list[ti] : ti;
    const int G = nh / nkv;
    const int s = seg_of_token[t];
    const int p = ctx_len[s] - q_len[s] + (t - q_start[s]);
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int nkeys = p - lo + 1;
    int per = (((nkeys + nruns_all - 1) / nruns_all) + 31) & ~31;
    if (run_keys) {
        // one run length for the whole batch (decode_run_keys_kernel): never shorter than this token's keys
        // need to fit the runs, never longer than the runs the host sized the page table in LDS for
        long widest = (long)max_blocks * page_size;
        if (window > 0 && window < widest) widest = window;
        const int cap = (int)((((widest + nruns_all - 1) / nruns_all) + 31) & ~31L);
        int given = (run_keys[0] + 31) & ~31;
        given = given < cap ? given : cap;
        per = given > per ? given : per;
    }
    const int k_begin = lo + split * per;
    const int k_end = (k_begin + per < p + 1) ? k_begin + per : p + 1;
    const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
    auto dim_of = [&](int i) -> int { return F32 ? 64 * (i >> 2) + 4 * c + (i & 3) : 128 * (i >> 3) + 8 * c + (i & 7); };
    // The block table of this split goes to LDS first: a page number fetched from global
    // memory in the loop would make every wait for it a wait for all loads issued before.
    const float inv_page = 1.0f / (float)page_size;
    const float scale2 = scale * 1.44269504088896341f;  // scores in units of log 2: the exponentials are the instruction's own
    const int first_block = k_begin / page_size;
    if (k_begin < k_end) {
        const int nblocks = (k_end - 1) / page_size - first_block + 1;       // the host keeps this <= DEC_TABLE_CAP
        const int* table = block_table + (size_t)s * max_blocks + first_block;
        for (int i = lane; i < nblocks && i < DEC_TABLE_CAP; i += 64) pages[i] = table[i];
    }
    wave_lds_sync();
    auto row_of = [&](int key, bool& ok) -> size_t {       // element offset of the key's row in a cache layer
        ok = key < k_end;
        key = ok ? key : k_end - 1;                        // (only called when k_begin < k_end)
        // key / page_size as a float32 product: (key + 1/2) / page_size is at least 1 / (2 page_size) away from
        // a whole number and the product's error is below (key + 1/2) / page_size * 2^-23, so the truncation is
        // the quotient while key < 2^22 (the host refuses longer tables).  The integer division by a number
        // only known when the kernel runs is some twenty instructions, and a choice between it and a shift
        // becomes a branch between the loads, behind which every wait is for all of them.
        const int blk = (int)(((float)key + 0.5f) * inv_page);
        const int in_page = key - __mul24(blk, page_size);
        int page = pages[blk - first_block];
        ok = ok && page >= 0 && page < num_pages;
        page = page < 0 ? 0 : (page >= num_pages ? num_pages - 1 : page);
        return (((size_t)page * nkv + kvh) * page_size + in_page) * DH;
    };

    for (int h0 = 0; h0 < G; h0 += 16) {
        const int gcount = (G - h0 < 16) ? G - h0 : 16;
        f32x4_t acc[NACC];
#pragma unroll
        for (int i = 0; i < NACC; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        float m[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY}, l[4] = {0.f, 0.f, 0.f, 0.f};
        if constexpr (!F32) {
            frag8 qa[KS];
#pragma unroll
            for (int j = 0; j < KS; ++j)
                qa[j].raw = *reinterpret_cast<const u32x4*>(
                    q + (size_t)t * q_row_stride + (size_t)(kvh * G + h0 + (c < gcount ? c : gcount - 1)) * DH + QD * g + 8 * j);

            // K of a block: two tiles of 16 keys; lane (c, g) holds key 16 tt + c, dimensions QD g + 8 j ..
            frag8 kf[2][KS];
            bool kok[2];
            auto load_k = [&](int kb) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const size_t off = row_of(kb + 16 * tt + c, kok[tt]);
#pragma unroll
                    for (int j = 0; j < KS; ++j)
                        kf[tt][j].raw = *reinterpret_cast<const u32x4*>(kc + off + QD * g + 8 * j);
                }
            };
            // V rows of this lane: keys kb + 8g + i, dimensions 128 ns + 8c ..  Two sets of registers
            // take turns, so that the values of the NEXT block are in flight while this one is worked on
            u32x4 va[NS][8], vb[NS][8];
#define LI_DEC_LOAD_V(kbv, dst)                                                                      \
            _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                              \
                bool ok_;                                                                                \
                const size_t off_ = row_of((kbv) + 8 * g + i, ok_);                                      \
                _Pragma("unroll") for (int ns = 0; ns < NS; ++ns) {                                      \
                    const int d_ = 128 * ns + 8 * c;                                                     \
                    dst[ns][i] = *reinterpret_cast<const u32x4*>(vc + off_ + (d_ < DH ? d_ : DH - 8));   \
                }                                                                                        \
            }
#define LI_DEC_STEP(kbv, vcur, vnext, more)                                                             \
            {                                                                                            \
                /* ---- S = Q K^T */                                                                     \
                f32x4_t sv[2];                                                                           \
                const bool sok[2] = {kok[0], kok[1]};                                                    \
                _Pragma("unroll") for (int tt = 0; tt < 2; ++tt) {                                       \
                    sv[tt] = f32x4_t{0.f, 0.f, 0.f, 0.f};                                                \
                    _Pragma("unroll") for (int j = 0; j < KS; ++j)                                       \
                        sv[tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa[j].v, kf[tt][j].v, sv[tt], 0, 0, 0); \
                }                                                                                        \
                /* ---- the next block's K and V: in flight during the softmax and P V (in the loop `more` */ \
                /* is the constant: behind a branch every wait is for all loads)                         */ \
                if (more) {                                                                              \
                    load_k((kbv) + 32);                                                                  \
                    LI_DEC_LOAD_V((kbv) + 32, vnext)                                                     \
                }                                                                                        \
                /* ---- online softmax; lanes whose key is past the end hold -inf */                     \
                float alpha[4], pr[2][4];                                                                \
                _Pragma("unroll") for (int r = 0; r < 4; ++r) {                                          \
                    const float s0 = sok[0] ? sv[0][r] * scale2 : -INFINITY;                             \
                    const float s1 = sok[1] ? sv[1][r] * scale2 : -INFINITY;                             \
                    const float mx = fmaxf(m[r], row16_max(fmaxf(s0, s1)));     /* the block has a key: mx is finite */ \
                    alpha[r] = __builtin_amdgcn_exp2f(m[r] - mx);                                        \
                    pr[0][r] = __builtin_amdgcn_exp2f(s0 - mx);                                          \
                    pr[1][r] = __builtin_amdgcn_exp2f(s1 - mx);                                          \
                    l[r] = l[r] * alpha[r] + pr[0][r] + pr[1][r];                                        \
                    m[r] = mx;                                                                           \
                }                                                                                        \
                wave_lds_sync();                                    /* readers of the last block's P are done */ \
                _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                                         \
                    _Pragma("unroll") for (int r = 0; r < 4; ++r)                                        \
                        p_lds[(4 * g + r) * PSTRIDE + 16 * tt + c].bits = float_to_bf16(pr[tt][r]);           \
                wave_lds_sync();                                                                         \
                frag8 pa;                                                                                \
                pa.raw = *reinterpret_cast<const u32x4*>(&p_lds[c * PSTRIDE + 8 * g]);                   \
                /* ---- O = alpha O + P V */                                                             \
                _Pragma("unroll") for (int ns = 0; ns < NS; ++ns) {                                      \
                    _Pragma("unroll") for (int jj = 0; jj < 8; ++jj) {                                   \
                        frag8 vf;                                                                        \
                        _Pragma("unroll") for (int ii = 0; ii < 4; ++ii)                                 \
                            vf.raw.w[ii] = __builtin_amdgcn_perm(vcur[ns][2 * ii + 1].w[jj >> 1], vcur[ns][2 * ii].w[jj >> 1], \
                                                                 (jj & 1) ? 0x07060302u : 0x05040100u);  \
                        _Pragma("unroll") for (int r = 0; r < 4; ++r) acc[8 * ns + jj][r] *= alpha[r];        \
                        acc[8 * ns + jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa.v, vf.v, acc[8 * ns + jj], 0, 0, 0); \
                    }                                                                                    \
                }                                                                                        \
            }
            // One condition around the first loads and the loop, and no way out of the loop between a step's
            // loads and the step that uses them: the compiler moves loads whose values one of two paths does
            // not use to the other path's start, where the wait for them follows at once.
            if (k_begin < k_end) {
                load_k(k_begin);
                LI_DEC_LOAD_V(k_begin, va)
                int kb = k_begin;
                for (; kb + 64 < k_end; kb += 64) {
                    LI_DEC_STEP(kb, va, vb, true)
                    LI_DEC_STEP(kb + 32, vb, va, true)
                }
                const bool two = kb + 32 < k_end;
                LI_DEC_STEP(kb, va, vb, two)
                if (two) LI_DEC_STEP(kb + 32, vb, va, false)
            }
#undef LI_DEC_STEP
#undef LI_DEC_LOAD_V
        } else {
            // ---- float32.  Lane (c, g) of v_mfma_f32_16x16x4f32 gives A[row c][k = g] and B[k = g][column c] and gets
            // D[row 4 g + r][column c].  Q K^T: rows are heads, columns 16 keys, and the MFMA for piece jj and
            // element i sums over the dimensions QD g + 4 jj + i of the four lane groups, so that a lane loads
            // its keys' dimensions in 16-byte pieces.  P V: rows are heads, k the keys 16 tt + 4 g + s (s the step:
            // a lane reads its four P values of a tile as one 16-byte LDS read), columns the dimensions
            // 64 n + 4 c + i, which a lane loads as one 16-byte piece of a value row.
            f32x4_t qa[KJ];
#pragma unroll
            for (int j = 0; j < KJ; ++j)
                qa[j] = *reinterpret_cast<const f32x4_t*>(
                    q + (size_t)t * q_row_stride + (size_t)(kvh * G + h0 + (c < gcount ? c : gcount - 1)) * DH + QD * g + 4 * j);
            f32x4_t kf[2][KJ];
            bool kok[2];
            auto load_k = [&](int kb) {
#pragma unroll
                for (int tt = 0; tt < 2; ++tt) {
                    const size_t off = row_of(kb + 16 * tt + c, kok[tt]);
#pragma unroll
                    for (int j = 0; j < KJ; ++j)
                        kf[tt][j] = *reinterpret_cast<const f32x4_t*>(kc + off + QD * g + 4 * j);
                }
            };
            // V rows of this lane: keys kb + 16 tt + 4 g + s, dimensions 64 n + 4 c ..; two sets of registers in turn
            f32x4_t va[2][4][NP], vb[2][4][NP];
#define LI_DEC_LOAD_V(kbv, dst)                                                                      \
            _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                                         \
                _Pragma("unroll") for (int s_ = 0; s_ < 4; ++s_) {                                   \
                    bool ok_;                                                                        \
                    const size_t off_ = row_of((kbv) + 16 * tt + 4 * g + s_, ok_);                   \
                    _Pragma("unroll") for (int n = 0; n < NP; ++n) {                                 \
                        const int d_ = 64 * n + 4 * c;                                               \
                        dst[tt][s_][n] = *reinterpret_cast<const f32x4_t*>(vc + off_ + (d_ < DH ? d_ : DH - 4)); \
                    }                                                                                \
                }
#define LI_DEC_STEP(kbv, vcur, vnext, more)                                                             \
            {                                                                                        \
                f32x4_t sv[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};          \
                const bool sok[2] = {kok[0], kok[1]};                                                \
                _Pragma("unroll") for (int j = 0; j < KJ; ++j)                                       \
                    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                    \
                        _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                             \
                            sv[tt] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa[j][i], kf[tt][j][i], sv[tt], 0, 0, 0); \
                if (more) {                                                                          \
                    load_k((kbv) + 32);                                                              \
                    LI_DEC_LOAD_V((kbv) + 32, vnext)                                                 \
                }                                                                                    \
                float alpha[4], pr[2][4];                                                            \
                _Pragma("unroll") for (int r = 0; r < 4; ++r) {                                      \
                    const float s0 = sok[0] ? sv[0][r] * scale2 : -INFINITY;                         \
                    const float s1 = sok[1] ? sv[1][r] * scale2 : -INFINITY;                         \
                    const float mx = fmaxf(m[r], row16_max(fmaxf(s0, s1)));                          \
                    alpha[r] = __builtin_amdgcn_exp2f(m[r] - mx);                                    \
                    pr[0][r] = __builtin_amdgcn_exp2f(s0 - mx);                                      \
                    pr[1][r] = __builtin_amdgcn_exp2f(s1 - mx);                                      \
                    l[r] = l[r] * alpha[r] + pr[0][r] + pr[1][r];                                    \
                    m[r] = mx;                                                                       \
                }                                                                                    \
                wave_lds_sync();                                                                     \
                _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                                     \
                    _Pragma("unroll") for (int r = 0; r < 4; ++r)                                    \
                        p_lds[(4 * g + r) * PSTRIDE + 16 * tt + c] = pr[tt][r];                      \
                wave_lds_sync();                                                                     \
                f32x4_t pa[2];                                                                       \
                _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                                     \
                    pa[tt] = *reinterpret_cast<const f32x4_t*>(&p_lds[c * PSTRIDE + 16 * tt + 4 * g]); \
                _Pragma("unroll") for (int i = 0; i < NACC; ++i)                                     \
                    _Pragma("unroll") for (int r = 0; r < 4; ++r) acc[i][r] *= alpha[r];             \
                _Pragma("unroll") for (int tt = 0; tt < 2; ++tt)                                     \
                    _Pragma("unroll") for (int s_ = 0; s_ < 4; ++s_)                                 \
                        _Pragma("unroll") for (int i = 0; i < NACC; ++i)                             \
                            acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[tt][s_], vcur[tt][s_][i >> 2][i & 3], acc[i], 0, 0, 0); \
            }
            // One condition around the first loads and the loop, and no way out of the loop between a step's
            // loads and the step that uses them: the compiler moves loads whose values one of two paths does
            // not use to the other path's start, where the wait for them follows at once.
            if (k_begin < k_end) {
                load_k(k_begin);
                LI_DEC_LOAD_V(k_begin, va)
                int kb = k_begin;
                for (; kb + 64 < k_end; kb += 64) {
                    LI_DEC_STEP(kb, va, vb, true)
                    LI_DEC_STEP(kb + 32, vb, va, true)
                }
                const bool two = kb + 32 < k_end;
                LI_DEC_STEP(kb, va, vb, two)
                if (two) LI_DEC_STEP(kb + 32, vb, va, false)
            }
#undef LI_DEC_STEP
#undef LI_DEC_LOAD_V
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            l[r] = row16_sum(l[r]);
            m[r] *= 0.69314718055994531f;               // (the loop counts in powers of 2, what joins the runs in powers of e)
        }
        if constexpr (WAVES == 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int hr = 4 * g + r;
                if (hr >= gcount) continue;
                const int head = kvh * G + h0 + hr;
                if (nsplit == 1) {
                    const float inv = l[r] != 0.f ? 1.0f / l[r] : 0.f;
                    T* orow = out + (size_t)t * nh * DH + (size_t)head * DH;
#pragma unroll
                    for (int i = 0; i < NACC; ++i) {
                        const int d = dim_of(i);
                        if (d < DH) store_from_float(orow + d, acc[i][r] * inv);
                    }
                } else {
                    const size_t pi = ((size_t)ti * nh + head) * nsplit + split;
#pragma unroll
                    for (int i = 0; i < NACC; ++i) {
                        const int d = dim_of(i);
                        if (d < DH) part_acc[pi * DH + d] = acc[i][r];
                    }
                    if (c == 0) { part_ml[pi * 2] = m[r]; part_ml[pi * 2 + 1] = l[r]; }
                }
            }
        } else {
            // ---- the four runs of this block, joined in LDS in the order of the runs
            __syncthreads();                                        // (the last pass's readers are done)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int hr = 4 * g + r;
#pragma unroll
                for (int i = 0; i < NACC; ++i) {
                    const int d = dim_of(i);
                    if (d < DH) join.acc[wave][hr][d] = acc[i][r];
                }
                if (c == 0) { join.ml[wave][hr][0] = m[r]; join.ml[wave][hr][1] = l[r]; }
            }
            __syncthreads();
            for (int e = threadIdx.x; e < gcount * DH; e += 64 * WAVES) {
                const int hr = e / DH, d = e - hr * DH;
                float mx = join.ml[0][hr][0];
#pragma unroll
                for (int w = 1; w < WAVES; ++w) mx = fmaxf(mx, join.ml[w][hr][0]);
                float lt = 0.f, at = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    const float f = (mx == -INFINITY) ? 0.f : expf(join.ml[w][hr][0] - mx);
                    lt += join.ml[w][hr][1] * f;
                    at += join.acc[w][hr][d] * f;
                }
                const int head = kvh * G + h0 + hr;
                if (nsplit == 1) {
                    store_from_float(out + (size_t)t * nh * DH + (size_t)head * DH + d, lt != 0.f ? at / lt : 0.f);
                } else {
                    const size_t pi = ((size_t)ti * nh + head) * nsplit + quad;
                    store_through(&part_acc[pi * DH + d], at);
                    if (d == 0) { store_through(&part_ml[pi * 2], mx); store_through(&part_ml[pi * 2 + 1], lt); }
                }
            }
        }
    }
    if constexpr (WAVES > 1) {
        if (nsplit > 1 && done) {
            // ---- the quads of this (token, kv head): the block that finishes last joins them, in quad order.
            // The partial results were stored through to memory; once every thread's stores have arrived,
            // the block counts itself (an atomic carried out in memory), and the block that completes the
            // count reads the others' results from memory, past its own L2.
            LI_WAIT_ALL_VMEM();
            __syncthreads();
            if (threadIdx.x == 0) {
                const int before = atomicAdd(&done[ti * nkv + kvh], 1);
                join.last = before == quads_of_token - 1;
                if (join.last) atomicExch(&done[ti * nkv + kvh], 0);   // as the next call expects it
            }
            __syncthreads();
            if (!join.last) return;
            // A thread takes four neighbouring dimensions of one head and asks for everything it needs of all
            // quads at once, never conditionally (a quad or head past the last repeats the last): one trip to
            // memory for the whole join.
            constexpr int TPH = DH / 4, HPC = 64 * WAVES / TPH;        // threads a head, heads a chunk of the block
            for (int hb = 0; hb < G; hb += HPC) {
                const int hg_own = hb + (int)threadIdx.x / TPH, hg = hg_own < G ? hg_own : G - 1;
                const int d = 4 * ((int)threadIdx.x % TPH);
                const int head = kvh * G + hg;
                const size_t base = ((size_t)ti * nh + head) * nsplit;
                float mq[16], lq[16], aq[16][4];                   // (quads <= MERGE_MAX_SPLITS / WAVES = 16)
#pragma unroll
                for (int qd = 0; qd < 16; ++qd) {
                    const int q_ = qd < quads_of_token ? qd : quads_of_token - 1;
                    load_through2(&part_ml[(base + q_) * 2], mq[qd], lq[qd]);
                    load_through2(&part_acc[(base + q_) * DH + d], aq[qd][0], aq[qd][1]);
                    load_through2(&part_acc[(base + q_) * DH + d + 2], aq[qd][2], aq[qd][3]);
                }
                float mx = -INFINITY;
#pragma unroll
                for (int qd = 0; qd < 16; ++qd) mx = fmaxf(mx, mq[qd]);
                float lt = 0.f, at[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int qd = 0; qd < 16; ++qd) {
                    const float f = (qd < quads_of_token && mx != -INFINITY) ? expf(mq[qd] - mx) : 0.f;
                    lt += lq[qd] * f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) at[i] += aq[qd][i] * f;
                }
                if (hg_own < G) {
                    const float inv = lt != 0.f ? 1.0f / lt : 0.f;
                    T* dst = out + (size_t)t * nh * DH + (size_t)head * DH + d;
                    if constexpr (F32) {
                        *reinterpret_cast<f32x4_t*>(dst) = f32x4_t{at[0] * inv, at[1] * inv, at[2] * inv, at[3] * inv};
                    } else {
                        uint32_t* dw = reinterpret_cast<uint32_t*>(dst);
                        dw[0] = pack2_bf16(at[0] * inv, at[1] * inv);
                        dw[1] = pack2_bf16(at[2] * inv, at[3] * inv);
                    }
                }
            }
        }
    }
}

// ------------------------------------------- portions of prompts, bfloat16, MFMA
// A block takes a tile of up to 32 consecutive tokens of one segment and one kv head; its
// waves are query heads of that kv head (PRE_WAVES at a time; blockIdx.z picks which), so
// the keys and values of a block of 32 keys are fetched once, into LDS, for all of them.
//
// A wave holds 32 queries of one head and works with the TRANSPOSED score tile
// S^T[key, query] = K Q^T (v_mfma_f32_32x32x16_bf16; row operand K from LDS, column operand
// Q in registers; lane l: row/column l % 32 and the 64 head dimensions 64 * (l / 32) ..): in
// the result a lane holds 16 keys of ITS query (register r: key 8 (r / 4) + 4 (l / 32) + r % 4),
// so the softmax over keys is arithmetic inside a lane plus one exchange with lane l ^ 32.
// These registers, rounded to bfloat16, are already the column operand of
// O^T[d, query] = V^T P^T: MFMA step s takes registers 8 s .. 8 s + 7, i.e. the keys
// {16 s + 4 h + i, 16 s + 8 + 4 h + i : i < 4} for lane half h.  The row operand V^T wants those
// same keys next to each other for one dimension d: the values are transposed in registers
// when they are put into LDS (8 keys x 8 dimensions a thread), in that key order.
#define PRE_TABLE_CAP 8192
#define PRE_WAVES 4
typedef float f32x16_t __attribute__((ext_vector_type(16)));

// the largest of three in one instruction (no NaN can occur among scores and -inf)
__device__ __forceinline__ float max3f(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

template <int DH>
__global__ __launch_bounds__(PRE_WAVES * 64) void paged_attention_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tiles, const int* __restrict__ q_start,
    const int* __restrict__ q_len, const int* __restrict__ ctx_len, int nh, int nkv, int page_size,
    int num_pages, int window, float scale, int ncu) {
    constexpr int KS = DH / 16;                 // MFMA steps of K Q^T (16 head dimensions each)
    constexpr int HD = DH / 2;                  // head dimensions owned by one lane half
    constexpr int DT = DH / 32;                 // tiles of 32 output dimensions
    constexpr int CPR = DH / 8;                 // 16-byte chunks in a row of K
    constexpr int NT = PRE_WAVES * 64;
    constexpr int VS = 40;                      // row stride of Vt in elements: 32 key positions and a pad that spreads the banks
    __shared__ __attribute__((aligned(16))) uint16_t Ks[2][32 * DH];      // [key][dimension], chunks swizzled by key
    __shared__ __attribute__((aligned(16))) uint16_t Vt[2][DH * VS];      // [dimension][key position]
    __shared__ int pages[PRE_TABLE_CAP];
    // The last tiles of a long segment have the most keys: they are started first.  Blocks are handed to
    // the compute units in the order of their numbers, one each and then again from the first unit, and
    // a unit's blocks share it: the work is dealt in a snake (every other round of `ncu` blocks backwards),
    // so that the unit with the longest tile of one round gets the shortest of the next.
    const int per_tile = gridDim.y * gridDim.z;
    const int total = gridDim.x * per_tile;
    const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int round = lin / ncu, pos = lin - round * ncu;
    const int in_round = total - round * ncu < ncu ? total - round * ncu : ncu;
    const int item = round * ncu + ((round & 1) ? in_round - 1 - pos : pos);
    const int tile = gridDim.x - 1 - item / per_tile;
    const int s = tiles[tile * 4], t0 = tiles[tile * 4 + 1], nrows = tiles[tile * 4 + 2];
    const int kvh = (item % per_tile) / gridDim.z;      // (the parts of a group of heads are neighbours: they read the same keys)
    const int G = nh / nkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hw = ((item % per_tile) % gridDim.z) * PRE_WAVES + wave;       // this wave's head within the group
    const bool active = hw < G;                         // (idle waves still help to fetch and keep the barriers)
    const int head = kvh * G + (active ? hw : 0);
    const int ql = lane & 31, h = lane >> 5;
    const int p0 = ctx_len[s] - q_len[s] + (t0 - q_start[s]);           // position of the tile's first token
    const int p_last = p0 + nrows - 1;
    const int lo0 = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int k_begin = lo0 & ~31, k_end = p_last + 1;
    const int first_block = lo0 / page_size;
    const int nblocks = (k_end - 1) / page_size - first_block + 1;     // <= PRE_TABLE_CAP (checked by the host)
    const int* table = block_table + (size_t)s * max_blocks + first_block;
    for (int i = tid; i < nblocks; i += NT) pages[i] = table[i];
    __syncthreads();
    // ---- fetching a block of 32 keys.  K: 16-byte chunks tid, tid + NT, ...  V: units of two
    // neighbouring key positions x 8 dimensions; position p of the key order holds the key
    // 16 (p / 16) + 4 ((p / 8) % 2) + (p % 8 < 4 ? p % 8 : p % 8 + 4).
    // A thread fetches the same rows of every block, 32 keys further on each turn: it keeps each
    // row's page block and place in the page and moves them on without a division.  Rows before
    // the first or past the last key of the tile (their scores are masked) read whatever page the
    // clamped table entry names: the cache holds finite numbers everywhere.
    constexpr int KCH = (32 * CPR + NT - 1) / NT;
    constexpr int VU = 16 * CPR, VCH = (VU + NT - 1) / NT;
    constexpr int NROW = KCH + 2 * VCH;                 // rows this thread fetches: K rows, then pairs of V rows
    u32x4 kreg[KCH], vreg[VCH][2];
    int row_blk[NROW], row_in[NROW], row_col[NROW];     // page block (relative to first_block), place in the page, column
    {
        int keys[NROW];
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            int ch = tid + i * NT;
            ch = ch < 32 * CPR ? ch : 32 * CPR - 1;
            keys[i] = ch / CPR;
            row_col[i] = 8 * (ch % CPR);
        }
#pragma unroll
        for (int i = 0; i < VCH; ++i) {
            int u = tid + i * NT;
            u = u < VU ? u : VU - 1;
            const int dg = (u & 3) + 4 * (u >> 6), pp = (u >> 2) & 15, pc = pp >> 2, ip = 2 * (pp & 3);
            keys[KCH + 2 * i] = 16 * (pc >> 1) + 4 * (pc & 1) + (ip < 4 ? ip : ip + 4);
            keys[KCH + 2 * i + 1] = keys[KCH + 2 * i] + 1;
            row_col[KCH + 2 * i] = row_col[KCH + 2 * i + 1] = 8 * dg;
        }
#pragma unroll
        for (int i = 0; i < NROW; ++i) {
            const int key = k_begin + keys[i];
            row_blk[i] = key / page_size - first_block;
            row_in[i] = key % page_size;
        }
    }
    const int step_blk = 32 / page_size, step_in = 32 % page_size;      // a turn moves every row 32 keys on
    const size_t page_bytes = (size_t)nkv * page_size * DH * 2;
    const char* kbase = reinterpret_cast<const char*>(kc) + (size_t)kvh * page_size * DH * 2;
    const char* vbase = reinterpret_cast<const char*>(vc) + (size_t)kvh * page_size * DH * 2;
    // the row's address in a cache layer, then on to the next block of keys
#define LI_PRE_ROW(i, base)                                                                          \
    ({                                                                                               \
        int ix_ = row_blk[i] < 0 ? 0 : (row_blk[i] > PRE_TABLE_CAP - 1 ? PRE_TABLE_CAP - 1 : row_blk[i]); \
        int page_ = pages[ix_];                                                                      \
        page_ = page_ < 0 ? 0 : (page_ >= num_pages ? num_pages - 1 : page_);                        \
        const char* p_ = (base) + (size_t)(unsigned)page_ * page_bytes + (unsigned)((row_in[i] * DH + row_col[i]) * 2); \
        row_in[i] += step_in;                                                                        \
        row_blk[i] += step_blk;                                                                      \
        if (row_in[i] >= page_size) { row_in[i] -= page_size; row_blk[i] += 1; }                     \
        p_;                                                                                          \
    })
    // (fetches are made for consecutive blocks: k_begin, k_begin + 32, ...)
#define LI_PRE_FETCH(kb)                                                                             \
    {                                                                                                \
        _Pragma("unroll") for (int i = 0; i < KCH; ++i)                                              \
            kreg[i] = *reinterpret_cast<const u32x4*>(LI_PRE_ROW(i, kbase));                         \
        _Pragma("unroll") for (int i = 0; i < VCH; ++i) {                                            \
            vreg[i][0] = *reinterpret_cast<const u32x4*>(LI_PRE_ROW(KCH + 2 * i, vbase));            \
            vreg[i][1] = *reinterpret_cast<const u32x4*>(LI_PRE_ROW(KCH + 2 * i + 1, vbase));        \
        }                                                                                            \
    }
#define LI_PRE_STASH(stage)                                                                          \
    {                                                                                                \
        _Pragma("unroll") for (int i = 0; i < KCH; ++i) {                                            \
            const int ch = tid + i * NT;                                                             \
            if (ch < 32 * CPR) {                                                                     \
                const int key = ch / CPR, c = ch % CPR;                                              \
                *reinterpret_cast<u32x4*>(&Ks[stage][key * DH + ((c ^ (key & (CPR - 1))) << 3)]) =   \
                    kreg[i];                                                                         \
            }                                                                                        \
        }                                                                                            \
        _Pragma("unroll") for (int i = 0; i < VCH; ++i) {                                            \
            const int u = tid + i * NT;                                                              \
            if (u < VU) {                                                                            \
                const int dg = (u & 3) + 4 * (u >> 6), pp = (u >> 2) & 15;                           \
                const u32x4 v0 = vreg[i][0], v1 = vreg[i][1];                                        \
                _Pragma("unroll") for (int jj = 0; jj < 8; ++jj)                                     \
                    *reinterpret_cast<uint32_t*>(&Vt[stage][(8 * dg + jj) * VS + 2 * pp]) =          \
                        __builtin_amdgcn_perm(v1.w[jj >> 1], v0.w[jj >> 1], (jj & 1) ? 0x07060302u : 0x05040100u); \
            }                                                                                        \
        }                                                                                            \
    }
    // ---- this wave's queries
    frag8 qf[KS];
    {
        const bf16_t* qrow = q + (size_t)(t0 + (ql < nrows ? ql : nrows - 1)) * q_row_stride + (size_t)head * DH + HD * h;
#pragma unroll
        for (int st = 0; st < KS; ++st) qf[st].raw = *reinterpret_cast<const u32x4*>(qrow + 8 * st);
    }
    const int pq = p0 + (ql < nrows ? ql : nrows - 1);       // last visible key of this lane's query (lanes past the tile repeat its last row)
    const int lq = (window > 0 && pq - window + 1 > 0) ? pq - window + 1 : 0;
    const int l_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
    const float scale2 = scale * 1.44269504088896341f;                       // scores in units of log 2
    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    // Order of a turn: the block fetched during the LAST turn goes from the registers into the
    // other stage of LDS, the block after it is fetched into the same registers, and then the
    // block in this stage is worked on: a fetch has a whole turn to arrive.
    LI_PRE_FETCH(k_begin);
    LI_PRE_STASH(0);
    if (k_begin + 32 < k_end) LI_PRE_FETCH(k_begin + 32);
    __syncthreads();
    // where this lane reads its fragments of K in a stage (the swizzle depends on the lane only)
    int kaddr[KS];
#pragma unroll
    for (int st = 0; st < KS; ++st) kaddr[st] = ql * DH + ((((HD / 8) * h + st) ^ (ql & (CPR - 1))) << 3);
    const int vaddr = ql * VS + 8 * h;
    // two turns a trip, so that the stage is a constant of the code and the LDS addresses are
    // a register plus an immediate
    for (int kb2 = k_begin; kb2 < k_end; kb2 += 64) {
#pragma unroll
      for (int stage = 0; stage < 2; ++stage) {
        const int kb = kb2 + 32 * stage;
        if (kb >= k_end) break;
        if (kb + 32 < k_end) LI_PRE_STASH(stage ^ 1);      // (its readers of the turn before are past the barrier)
        if (kb + 64 < k_end) LI_PRE_FETCH(kb + 64);
        if (active) {
            // ---- S^T = K Q^T
            f32x16_t sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
            frag8 kf[KS];
#pragma unroll
            for (int st = 0; st < KS; ++st) kf[st].raw = *reinterpret_cast<const u32x4*>(&Ks[stage][kaddr[st]]);
#pragma unroll
            for (int st = 0; st < KS; ++st) sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st].v, qf[st].v, sv, 0, 0, 0);
            // ---- softmax over the keys of this lane's query.  The running maximum m is only moved
            // (and the sums so far rescaled, for the whole wave) when some query's scores pass it by
            // more than 2^8: until then the exponentials are taken against the older maximum, which
            // changes no result (numerator and denominator carry the same factor) and stays far
            // inside the range of float and bfloat16.
            // A block that every query of the tile sees whole (most are) needs no masks.
            if (!(kb + 31 <= p0 && kb >= l_last)) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 8 * (r >> 2) + 4 * h + (r & 3);
                    sv[r] = (key <= pq && key >= lq) ? sv[r] : -INFINITY;
                }
            }
            float mx = max3f(sv[0], sv[1], sv[2]);
#pragma unroll
            for (int r = 3; r < 15; r += 2) mx = max3f(mx, sv[r], sv[r + 1]);
            mx = max3f(mx, sv[15], sv[15]);
            mx = both_halves_max(mx) * scale2;                          // (scale2 > 0)
            if (__any(mx > m + 8.0f)) {
                const float mn = fmaxf(m, mx);
                const float alpha = (mn == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m - mn);   // (m = -inf: nothing summed yet)
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
                m = mn;
            }
            const float ms = (m == -INFINITY) ? 0.f : m;         // a query may see no key yet
            float ps = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sv[r] = __builtin_amdgcn_exp2f(fmaf(sv[r], scale2, -ms)); ps += sv[r]; }
            l += ps;
            frag8 pf[2];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[st].raw.w[i] = pack2_bf16(sv[8 * st + 2 * i], sv[8 * st + 2 * i + 1]);
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    frag8 vf;
                    vf.raw = *reinterpret_cast<const u32x4*>(&Vt[stage][vaddr + 32 * dt * VS + 16 * st]);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[st].v, acc[dt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
      }
    }
    if (!active || ql >= nrows) return;
    l += __shfl_xor(l, 32, LI_WAVE);               // (both halves of a query are past the return together)
    const float inv = l != 0.f ? 1.0f / l : 0.f;
    bf16_t* orow = out + (size_t)(t0 + ql) * nh * DH + (size_t)head * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {           // registers 4 rg .. 4 rg + 3: dimensions 32 dt + 8 rg + 4 h ..
            uint32_t w0 = pack2_bf16(acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv);
            uint32_t w1 = pack2_bf16(acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv);
            uint32_t* dst = reinterpret_cast<uint32_t*>(orow + 32 * dt + 8 * rg + 4 * h);
            dst[0] = w0;
            dst[1] = w1;
        }
}

#undef LI_PRE_FETCH
#undef LI_PRE_ROW
#undef LI_PRE_STASH
// The same with the loads of K and V going straight into LDS (no registers, no transposing on the way in:
// that way of filling LDS took as long as the arithmetic) and V turned by the LDS read that transposes
// 16-bit elements (ds_read_b64_tr_b16).  Three stages of LDS, so a block of keys has two turns to arrive.
#define PRE2_TABLE_CAP 4096
typedef short tr4 __attribute__((ext_vector_type(4)));
#define LI_ATT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)
// (inline assembly, so that the compiler neither counts these loads nor waits for them before LDS
// reads: `s_waitcnt vmcnt` is placed by hand; M0 carries the wave's LDS address, lane i's 16 bytes land 16 i on)
#define LI_ATT_LOAD_TO_LDS(gptr, lptr)                                                                    \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"                        \
                 :: "s"((uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(lptr)), "v"(gptr) : "memory", "m0")
// P32: the page size divides 32, so a row keeps its place in its page from block to block
template <int DH, bool P32>
__global__ __launch_bounds__(PRE_WAVES * 64) void paged_attention_prefill_dma_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tiles, const int* __restrict__ q_start,
    const int* __restrict__ q_len, const int* __restrict__ ctx_len, int nh, int nkv, int page_size,
    int num_pages, int window, float scale, int ncu, int ksplit, float* __restrict__ part_acc,
    float* __restrict__ part_ml) {
    // ksplit > 1: the tile's blocks of keys are cut into ksplit runs, blockIdx.z = part of the heads x
    // ksplit + run; a block then leaves its sums, unscaled, in part_acc [token, head, run, dh] and its
    // (maximum, sum) in part_ml, and attention_merge_runs_kernel joins the runs in their order
    constexpr int KS = DH / 16;                 // MFMA steps of K Q^T (16 head dimensions each)
    constexpr int HD = DH / 2;                  // head dimensions owned by one lane half
    constexpr int DT = DH / 32;                 // tiles of 32 output dimensions
    constexpr int CPR = DH / 8;                 // 16-byte chunks in a row of K
    constexpr int NT = PRE_WAVES * 64;
    constexpr int NST = 3;                      // stages of LDS: one worked on, two on their way
    __shared__ __attribute__((aligned(16))) uint16_t Ks[NST][32 * DH];    // [key][dimension], chunks swizzled by key
    __shared__ __attribute__((aligned(16))) uint16_t Vs[NST][32 * DH];    // the same for V, another swizzle
    __shared__ uint32_t pageoff[PRE2_TABLE_CAP];                          // byte offset / 128 of each page of the tile's part of the table
    // The last tiles of a long segment have the most keys: they are started first.  Blocks are handed to
    // the compute units in the order of their numbers, one each and then again from the first unit, and
    // a unit's blocks share it: the work is dealt in a snake (every other round of `ncu` blocks backwards),
    // so that the unit with the longest tile of one round gets the shortest of the next.
    const int per_tile = gridDim.y * gridDim.z;
    const int total = gridDim.x * per_tile;
    const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int round = lin / ncu, pos = lin - round * ncu;
    const int in_round = total - round * ncu < ncu ? total - round * ncu : ncu;
    const int item = round * ncu + ((round & 1) ? in_round - 1 - pos : pos);
    const int tile = gridDim.x - 1 - item / per_tile;
    const int s = tiles[tile * 4], t0 = tiles[tile * 4 + 1], nrows = tiles[tile * 4 + 2];
    const int kvh = (item % per_tile) / gridDim.z;      // (the parts of a group of heads are neighbours: they read the same keys)
    const int G = nh / nkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int zz = (item % per_tile) % gridDim.z, run = zz % ksplit;
    const int hw = (zz / ksplit) * PRE_WAVES + wave;    // this wave's head within the group
    const bool active = hw < G;                         // (idle waves still help to fetch and keep the barriers)
    const int head = kvh * G + (active ? hw : 0);
    const int ql = lane & 31, h = lane >> 5;
    const int p0 = ctx_len[s] - q_len[s] + (t0 - q_start[s]);           // position of the tile's first token
    const int p_last = p0 + nrows - 1;
    const int lo0 = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    int k_begin = lo0 & ~31, k_end = p_last + 1;
    int first_key = lo0;
    if (ksplit > 1) {                                   // this run's blocks of 32 keys
        const int all = (k_end - k_begin + 31) / 32, per = (all + ksplit - 1) / ksplit;
        const int b0 = run * per, b1 = (run + 1) * per < all ? (run + 1) * per : all;
        if (b0 >= b1) {                                 // no keys for this run: it says so and is done (before any barrier)
            if (active && ql < nrows && h == 0) {
                const size_t at = ((size_t)(t0 + ql) * nh + head) * ksplit + run;
                part_ml[at * 2] = -INFINITY;
                part_ml[at * 2 + 1] = 0.f;
            }
            if (active && ql < nrows) {
                float* pa = part_acc + (((size_t)(t0 + ql) * nh + head) * ksplit + run) * DH + HD * h;
#pragma unroll
                for (int d = 0; d < HD; d += 4) *reinterpret_cast<float4*>(pa + d) = float4{0.f, 0.f, 0.f, 0.f};
            }
            return;
        }
        const int kb0 = k_begin + 32 * b0;
        k_end = k_begin + 32 * b1 < k_end ? k_begin + 32 * b1 : k_end;
        k_begin = kb0;
        first_key = kb0 > lo0 ? kb0 : lo0;
    }
    const int first_block = first_key / page_size;
    const int nblocks = (k_end - 1) / page_size - first_block + 1;     // <= PRE2_TABLE_CAP (checked by the host)
    const int* table = block_table + (size_t)s * max_blocks + first_block;
    const size_t page_bytes = (size_t)nkv * page_size * DH * 2;
    for (int i = tid; i < nblocks; i += NT) {
        int pg = table[i];
        pg = pg < 0 ? 0 : (pg >= num_pages ? num_pages - 1 : pg);
        pageoff[i] = (uint32_t)(((unsigned long long)(unsigned)pg * page_bytes) >> 7);     // (a page is a multiple of 128 bytes: dh >= 64; 512 GB of cache)
    }
    const int last_entry = nblocks - 1;
    __syncthreads();
    // ---- fetching a block of 32 keys: the loads go straight into LDS (16 bytes a lane, a wave's
    // 64 lanes to 1 KB in a row), so a stage's K and V are [key][16-byte chunk] in the order of
    // the lanes: chunk index ci = 64 (NL wave + i) + lane, key ci / CPR, place ci % CPR.  The
    // bank swizzle is made on the way in: the place holds the chunk (place ^ swizzle(key)) of the
    // key's row, for K swizzle = key % CPR, for V 2 (key % 8) (% CPR), see the reads below.
    // A thread fetches the same rows of every block, 32 keys further on each turn: it keeps each
    // row's page block and place in the page and moves them on without a division; K and V of a
    // row lie at the same place of their cache layers.  Rows before the first or past the last
    // key of the tile (their scores are masked) read whatever page the clamped table entry
    // names: the cache holds finite numbers everywhere.
    constexpr int NL = (32 * CPR) / NT;                 // loads of K (and of V) a thread makes per block
    static_assert(NL * NT == 32 * CPR, "whole load instructions a block of keys");
    int row_blk[NL], row_in[NL], kcol[NL], vcol[NL];
    const char* kbase = reinterpret_cast<const char*>(kc) + (size_t)kvh * page_size * DH * 2;
    const char* vbase = reinterpret_cast<const char*>(vc) + (size_t)kvh * page_size * DH * 2;
    const char* krow[NL];                               // P32: the row's place in its page and its chunk, once and for all
    const char* vrow[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int ci = 64 * (NL * wave + i) + lane, key = ci / CPR, place = ci % CPR;
        kcol[i] = 8 * (place ^ (key & (CPR - 1)));
        vcol[i] = 8 * (place ^ ((2 * (key & 7)) & (CPR - 1)));
        const int kk = k_begin + key;
        row_blk[i] = kk / page_size - first_block;
        row_in[i] = kk % page_size;
        krow[i] = kbase + (size_t)(row_in[i] * DH + kcol[i]) * 2;
        vrow[i] = vbase + (size_t)(row_in[i] * DH + vcol[i]) * 2;
    }
    const int step_blk = 32 / page_size, step_in = 32 % page_size;      // a turn moves every row 32 keys on
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    // (fetches are made for consecutive blocks: k_begin, k_begin + 32, ...)
#define LI_PRE_FETCH(stage)                                                                          \
    {                                                                                                \
        unsigned long long off_[NL];                                                                 \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                             \
            const int ix_ = row_blk[i] < 0 ? 0 : (row_blk[i] > last_entry ? last_entry : row_blk[i]); \
            off_[i] = (unsigned long long)pageoff[ix_] << 7;                                         \
        }                                                                                            \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                             \
            if constexpr (P32) {                                                                     \
                row_blk[i] += step_blk;                                                              \
                LI_ATT_LOAD_TO_LDS(krow[i] + off_[i], &Ks[stage][512 * (NL * uwave + i)]);           \
                LI_ATT_LOAD_TO_LDS(vrow[i] + off_[i], &Vs[stage][512 * (NL * uwave + i)]);           \
            } else {                                                                                 \
                const size_t o_ = off_[i] + (unsigned)(row_in[i] * DH * 2);                          \
                row_in[i] += step_in;                                                                \
                row_blk[i] += step_blk;                                                              \
                if (row_in[i] >= page_size) { row_in[i] -= page_size; row_blk[i] += 1; }             \
                LI_ATT_LOAD_TO_LDS(kbase + o_ + 2 * kcol[i], &Ks[stage][512 * (NL * uwave + i)]);    \
                LI_ATT_LOAD_TO_LDS(vbase + o_ + 2 * vcol[i], &Vs[stage][512 * (NL * uwave + i)]);    \
            }                                                                                        \
        }                                                                                            \
    }
    // ---- this wave's queries
    frag8 qf[KS];
    {
        const bf16_t* qrow = q + (size_t)(t0 + (ql < nrows ? ql : nrows - 1)) * q_row_stride + (size_t)head * DH + HD * h;
#pragma unroll
        for (int st = 0; st < KS; ++st) qf[st].raw = *reinterpret_cast<const u32x4*>(qrow + 8 * st);
    }
    const int pq = p0 + (ql < nrows ? ql : nrows - 1);       // last visible key of this lane's query (lanes past the tile repeat its last row)
    const int lq = (window > 0 && pq - window + 1 > 0) ? pq - window + 1 : 0;
    const int l_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
    const float scale2 = scale * 1.44269504088896341f;                       // scores in units of log 2
    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    // Order of a turn: the block two on is asked for, into the stage that the turn before read
    // (its readers are past the barrier); then the block in this stage is worked on; then the wave
    // waits for its own loads of the NEXT block (the loads of the block after it may stay in
    // flight: a wave's loads retire in order) and meets the others at the barrier.
    const int nblk = (k_end - k_begin + 31) / 32;
    LI_PRE_FETCH(0);
    if (nblk > 1) { LI_PRE_FETCH(1); LI_ATT_VMCNT(2 * NL); } else { LI_ATT_VMCNT(0); }
    // The queries have arrived by now: they were asked for before the blocks of keys, and a wave's loads retire
    // in order.  The compiler counts only the loads it made itself and would wait for "its" eight at their first
    // use, inside the loop, where the same count stands for the blocks of keys that are on their way: every turn
    // would then wait for ALL of them (found in the kernel's code: s_waitcnt vmcnt(7) .. vmcnt(0) before the first
    // eight MFMAs of a turn).  Using the registers here puts that wait here, once.
#pragma unroll
    for (int st = 0; st < KS; ++st)
        asm volatile("" :: "v"(qf[st].raw.w[0]), "v"(qf[st].raw.w[1]), "v"(qf[st].raw.w[2]), "v"(qf[st].raw.w[3]));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // where this lane reads its fragments of K in a stage (the swizzle depends on the lane only)
    int kaddr[KS];
#pragma unroll
    for (int st = 0; st < KS; ++st) kaddr[st] = ql * DH + ((((HD / 8) * h + st) ^ (ql & (CPR - 1))) << 3);
    // where this lane reads V for the row operand of O^T = V^T P^T.  The transposing LDS read (64
    // bits a lane) hands lane i of a group of 16 the element i % 4 of the 4 x 16-bit pieces that the
    // group's lanes 4 j + i / 4 point at, j = 0 .. 3.  Lane i of a group points at key base + i / 4,
    // dimensions d0 + 4 (i % 4) ..: it receives the keys base .. base + 3 of dimension d0 + i.  The
    // lane's group gives d0 (16 (group % 2) within the tile of 32) and the k-group (group / 2), whose
    // 8 keys of MFMA step st are 16 st + 4 h + {0 .. 3} and 16 st + 8 + 4 h + {0 .. 3}: two reads.
    // With the swizzle 2 (key % 8) the four keys of a read lie in eight different 16-byte columns.
    int vaddr[DT];
    {
        const int gi = lane & 15, grp = lane >> 4;
        const int vkey = 4 * (grp >> 1) + (gi >> 2);            // + 16 st + 8 r: the swizzle does not see those
        const int swz = (2 * (vkey & 7)) & (CPR - 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int chunk = 4 * dt + 2 * (grp & 1) + ((gi & 3) >> 1);
            vaddr[dt] = vkey * DH + 8 * (chunk ^ swz) + 4 * (gi & 1);
        }
    }
    // three turns a trip, so that the stage is a constant of the code and the LDS addresses are
    // a register plus an immediate
    for (int j3 = 0; j3 < nblk; j3 += NST) {
#pragma unroll
      for (int stage = 0; stage < NST; ++stage) {
        const int jb = j3 + stage;
        if (jb >= nblk) break;
        const int kb = k_begin + 32 * jb;
        if (jb + 2 < nblk) LI_PRE_FETCH((stage + 2) % NST);
        if (active) {
            // ---- S^T = K Q^T
            f32x16_t sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
            frag8 kf[KS];
#pragma unroll
            for (int st = 0; st < KS; ++st) kf[st].raw = *reinterpret_cast<const u32x4*>(&Ks[stage][kaddr[st]]);
            // (raising the wave's priority while it issues its MFMAs, so that the SIMD's other wave does its
            // softmax meanwhile, was measured in turn with this form on one machine: 2 to 5 % SLOWER at 2,048 to
            // 30,000 keys, so the waves keep the default priority)
#pragma unroll
            for (int st = 0; st < KS; ++st) sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st].v, qf[st].v, sv, 0, 0, 0);
            // ---- softmax over the keys of this lane's query.  The running maximum m is only moved
            // (and the sums so far rescaled, for the whole wave) when some query's scores pass it by
            // more than 2^8: until then the exponentials are taken against the older maximum, which
            // changes no result (numerator and denominator carry the same factor) and stays far
            // inside the range of float and bfloat16.
            // A block that every query of the tile sees whole (most are) needs no masks.
            if (!(kb + 31 <= p0 && kb >= l_last)) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 8 * (r >> 2) + 4 * h + (r & 3);
                    sv[r] = (key <= pq && key >= lq) ? sv[r] : -INFINITY;
                }
            }
            float mx = max3f(sv[0], sv[1], sv[2]);
#pragma unroll
            for (int r = 3; r < 15; r += 2) mx = max3f(mx, sv[r], sv[r + 1]);
            mx = max3f(mx, sv[15], sv[15]);
            mx = both_halves_max(mx) * scale2;                          // (scale2 > 0)
            if (__any(mx > m + 8.0f)) {
                const float mn = fmaxf(m, mx);
                const float alpha = (mn == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m - mn);   // (m = -inf: nothing summed yet)
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
                m = mn;
            }
            const float ms = (m == -INFINITY) ? 0.f : m;         // a query may see no key yet
            float ps = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sv[r] = __builtin_amdgcn_exp2f(fmaf(sv[r], scale2, -ms)); ps += sv[r]; }
            l += ps;
            frag8 pf[2];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[st].raw.w[i] = pack2_bf16(sv[8 * st + 2 * i], sv[8 * st + 2 * i + 1]);
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    frag8 vf;
                    const tr4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr4 __attribute__((address_space(3)))*)&Vs[stage][vaddr[dt] + (16 * st) * DH]);
                    const tr4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr4 __attribute__((address_space(3)))*)&Vs[stage][vaddr[dt] + (16 * st + 8) * DH]);
                    vf.raw.w[0] = (uint32_t)(uint16_t)v0[0] | ((uint32_t)(uint16_t)v0[1] << 16);
                    vf.raw.w[1] = (uint32_t)(uint16_t)v0[2] | ((uint32_t)(uint16_t)v0[3] << 16);
                    vf.raw.w[2] = (uint32_t)(uint16_t)v1[0] | ((uint32_t)(uint16_t)v1[1] << 16);
                    vf.raw.w[3] = (uint32_t)(uint16_t)v1[2] | ((uint32_t)(uint16_t)v1[3] << 16);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[st].v, acc[dt], 0, 0, 0);
                }
            }
        }
        if (jb + 2 < nblk) { LI_ATT_VMCNT(2 * NL); } else { LI_ATT_VMCNT(0); }
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
    }
    if (!active || ql >= nrows) return;
    l += __shfl_xor(l, 32, LI_WAVE);               // (both halves of a query are past the return together)
    if (ksplit > 1) {
        const size_t at = ((size_t)(t0 + ql) * nh + head) * ksplit + run;
        if (h == 0) {
            part_ml[at * 2] = m * 0.69314718055994531f;          // (the kernel that joins the runs counts in powers of e)
            part_ml[at * 2 + 1] = l;
        }
        float* pa = part_acc + at * DH;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int rg = 0; rg < 4; ++rg)
                *reinterpret_cast<float4*>(pa + 32 * dt + 8 * rg + 4 * h) =
                    float4{acc[dt][4 * rg], acc[dt][4 * rg + 1], acc[dt][4 * rg + 2], acc[dt][4 * rg + 3]};
        return;
    }
    const float inv = l != 0.f ? 1.0f / l : 0.f;
    bf16_t* orow = out + (size_t)(t0 + ql) * nh * DH + (size_t)head * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {           // registers 4 rg .. 4 rg + 3: dimensions 32 dt + 8 rg + 4 h ..
            uint32_t w0 = pack2_bf16(acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv);
            uint32_t w1 = pack2_bf16(acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv);
            uint32_t* dst = reinterpret_cast<uint32_t*>(orow + 32 * dt + 8 * rg + 4 * h);
            dst[0] = w0;
            dst[1] = w1;
        }
}

#undef LI_PRE_FETCH
// The same for prompts of so few tiles that a compute unit holds one or two blocks and the time is that of
// the longest tile, one block of keys after the other: eight waves a block, two groups of four, each group
// with its own stages of LDS takes half of the tile's blocks of keys (the first half, the second half), and
// at the end the second group hands its sums, maxima and outputs to the first through LDS.
template <int DH, bool P32>
__global__ __launch_bounds__(2 * PRE_WAVES * 64) void paged_attention_prefill_split_kernel(
    const bf16_t* __restrict__ q, int q_row_stride, bf16_t* __restrict__ out,
    const bf16_t* __restrict__ kc, const bf16_t* __restrict__ vc, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tiles, const int* __restrict__ q_start,
    const int* __restrict__ q_len, const int* __restrict__ ctx_len, int nh, int nkv, int page_size,
    int num_pages, int window, float scale, int ncu) {
    constexpr int KS = DH / 16;                 // MFMA steps of K Q^T (16 head dimensions each)
    constexpr int HD = DH / 2;                  // head dimensions owned by one lane half
    constexpr int DT = DH / 32;                 // tiles of 32 output dimensions
    constexpr int CPR = DH / 8;                 // 16-byte chunks in a row of K
    constexpr int NT = PRE_WAVES * 64;
    constexpr int NST = 3;                      // stages of LDS: one worked on, two on their way
    __shared__ __attribute__((aligned(16))) uint16_t kv[2][2][NST][32 * DH];   // [K, V][group][stage][key][dimension], chunks swizzled by key
    __shared__ uint32_t pageoff[PRE2_TABLE_CAP];                          // byte offset / 128 of each page of the tile's part of the table
    // The last tiles of a long segment have the most keys: they are started first.  Blocks are handed to
    // the compute units in the order of their numbers, one each and then again from the first unit, and
    // a unit's blocks share it: the work is dealt in a snake (every other round of `ncu` blocks backwards),
    // so that the unit with the longest tile of one round gets the shortest of the next.
    const int per_tile = gridDim.y * gridDim.z;
    const int total = gridDim.x * per_tile;
    const int lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const int round = lin / ncu, pos = lin - round * ncu;
    const int in_round = total - round * ncu < ncu ? total - round * ncu : ncu;
    const int item = round * ncu + ((round & 1) ? in_round - 1 - pos : pos);
    const int tile = gridDim.x - 1 - item / per_tile;
    const int s = tiles[tile * 4], t0 = tiles[tile * 4 + 1], nrows = tiles[tile * 4 + 2];
    const int kvh = (item % per_tile) / gridDim.z;      // (the parts of a group of heads are neighbours: they read the same keys)
    const int G = nh / nkv;
    const int tid = threadIdx.x, lane = tid & 63, half = tid >> 8, wave = (tid >> 6) & 3;     // group of waves, wave within it
    const int hw = ((item % per_tile) % gridDim.z) * PRE_WAVES + wave;       // this wave's head within the group
    const bool active = hw < G;                         // (idle waves still help to fetch and keep the barriers)
    const int head = kvh * G + (active ? hw : 0);
    const int ql = lane & 31, h = lane >> 5;
    const int p0 = ctx_len[s] - q_len[s] + (t0 - q_start[s]);           // position of the tile's first token
    const int p_last = p0 + nrows - 1;
    const int lo0 = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int k_begin = lo0 & ~31, k_end = p_last + 1;
    const int first_block = lo0 / page_size;
    const int nblocks = (k_end - 1) / page_size - first_block + 1;     // <= PRE2_TABLE_CAP (checked by the host)
    const int* table = block_table + (size_t)s * max_blocks + first_block;
    const size_t page_bytes = (size_t)nkv * page_size * DH * 2;
    for (int i = tid; i < nblocks; i += 2 * NT) {
        int pg = table[i];
        pg = pg < 0 ? 0 : (pg >= num_pages ? num_pages - 1 : pg);
        pageoff[i] = (uint32_t)(((unsigned long long)(unsigned)pg * page_bytes) >> 7);     // (a page is a multiple of 128 bytes: dh >= 64; 512 GB of cache)
    }
    const int last_entry = nblocks - 1;
    __syncthreads();
    const int nblk = (k_end - k_begin + 31) / 32;        // blocks of 32 keys of the tile
    const int n0 = (nblk + 1) / 2;                       // ... of the first group; turns of the loop
    const int nb = half ? nblk - n0 : n0;                // ... of this group
    const int kb0 = k_begin + 32 * n0 * half;            // this group's first key
    // ---- fetching a block of 32 keys: the loads go straight into LDS (16 bytes a lane, a wave's
    // 64 lanes to 1 KB in a row), so a stage's K and V are [key][16-byte chunk] in the order of
    // the lanes: chunk index ci = 64 (NL wave + i) + lane, key ci / CPR, place ci % CPR.  The
    // bank swizzle is made on the way in: the place holds the chunk (place ^ swizzle(key)) of the
    // key's row, for K swizzle = key % CPR, for V 2 (key % 8) (% CPR), see the reads below.
    // A thread fetches the same rows of every block, 32 keys further on each turn: it keeps each
    // row's page block and place in the page and moves them on without a division; K and V of a
    // row lie at the same place of their cache layers.  Rows before the first or past the last
    // key of the tile (their scores are masked) read whatever page the clamped table entry
    // names: the cache holds finite numbers everywhere.
    constexpr int NL = (32 * CPR) / NT;                 // loads of K (and of V) a thread makes per block
    static_assert(NL * NT == 32 * CPR, "whole load instructions a block of keys");
    int row_blk[NL], row_in[NL], kcol[NL], vcol[NL];
    const char* kbase = reinterpret_cast<const char*>(kc) + (size_t)kvh * page_size * DH * 2;
    const char* vbase = reinterpret_cast<const char*>(vc) + (size_t)kvh * page_size * DH * 2;
    const char* krow[NL];                               // P32: the row's place in its page and its chunk, once and for all
    const char* vrow[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int ci = 64 * (NL * wave + i) + lane, key = ci / CPR, place = ci % CPR;
        kcol[i] = 8 * (place ^ (key & (CPR - 1)));
        vcol[i] = 8 * (place ^ ((2 * (key & 7)) & (CPR - 1)));
        const int kk = kb0 + key;
        row_blk[i] = kk / page_size - first_block;
        row_in[i] = kk % page_size;
        krow[i] = kbase + (size_t)(row_in[i] * DH + kcol[i]) * 2;
        vrow[i] = vbase + (size_t)(row_in[i] * DH + vcol[i]) * 2;
    }
    const int step_blk = 32 / page_size, step_in = 32 % page_size;      // a turn moves every row 32 keys on
    const int uwave = __builtin_amdgcn_readfirstlane(wave), uhalf = __builtin_amdgcn_readfirstlane(half);
    // (fetches are made for consecutive blocks: k_begin, k_begin + 32, ...)
#define LI_PRE_FETCH(stage)                                                                          \
    {                                                                                                \
        unsigned long long off_[NL];                                                                 \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                             \
            const int ix_ = row_blk[i] < 0 ? 0 : (row_blk[i] > last_entry ? last_entry : row_blk[i]); \
            off_[i] = (unsigned long long)pageoff[ix_] << 7;                                         \
        }                                                                                            \
        _Pragma("unroll") for (int i = 0; i < NL; ++i) {                                             \
            if constexpr (P32) {                                                                     \
                row_blk[i] += step_blk;                                                              \
                LI_ATT_LOAD_TO_LDS(krow[i] + off_[i], &kv[0][uhalf][stage][512 * (NL * uwave + i)]);           \
                LI_ATT_LOAD_TO_LDS(vrow[i] + off_[i], &kv[1][uhalf][stage][512 * (NL * uwave + i)]);           \
            } else {                                                                                 \
                const size_t o_ = off_[i] + (unsigned)(row_in[i] * DH * 2);                          \
                row_in[i] += step_in;                                                                \
                row_blk[i] += step_blk;                                                              \
                if (row_in[i] >= page_size) { row_in[i] -= page_size; row_blk[i] += 1; }             \
                LI_ATT_LOAD_TO_LDS(kbase + o_ + 2 * kcol[i], &kv[0][uhalf][stage][512 * (NL * uwave + i)]);    \
                LI_ATT_LOAD_TO_LDS(vbase + o_ + 2 * vcol[i], &kv[1][uhalf][stage][512 * (NL * uwave + i)]);    \
            }                                                                                        \
        }                                                                                            \
    }
    // ---- this wave's queries
    frag8 qf[KS];
    {
        const bf16_t* qrow = q + (size_t)(t0 + (ql < nrows ? ql : nrows - 1)) * q_row_stride + (size_t)head * DH + HD * h;
#pragma unroll
        for (int st = 0; st < KS; ++st) qf[st].raw = *reinterpret_cast<const u32x4*>(qrow + 8 * st);
    }
    const int pq = p0 + (ql < nrows ? ql : nrows - 1);       // last visible key of this lane's query (lanes past the tile repeat its last row)
    const int lq = (window > 0 && pq - window + 1 > 0) ? pq - window + 1 : 0;
    const int l_last = (window > 0 && p_last - window + 1 > 0) ? p_last - window + 1 : 0;
    const float scale2 = scale * 1.44269504088896341f;                       // scores in units of log 2
    f32x16_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;

    // Order of a turn: the block two on is asked for, into the stage that the turn before read
    // (its readers are past the barrier); then the block in this stage is worked on; then the wave
    // waits for its own loads of the NEXT block (the loads of the block after it may stay in
    // flight: a wave's loads retire in order) and meets the others at the barrier.
    if (nb > 0) LI_PRE_FETCH(0);
    if (nb > 1) { LI_PRE_FETCH(1); LI_ATT_VMCNT(2 * NL); } else { LI_ATT_VMCNT(0); }
    // (the compiler's own wait for the queries, here and not inside the loop: see the kernel above)
#pragma unroll
    for (int st = 0; st < KS; ++st)
        asm volatile("" :: "v"(qf[st].raw.w[0]), "v"(qf[st].raw.w[1]), "v"(qf[st].raw.w[2]), "v"(qf[st].raw.w[3]));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // where this lane reads its fragments of K in a stage (the swizzle depends on the lane only)
    int kaddr[KS];
#pragma unroll
    for (int st = 0; st < KS; ++st) kaddr[st] = ql * DH + ((((HD / 8) * h + st) ^ (ql & (CPR - 1))) << 3);
    // where this lane reads V for the row operand of O^T = V^T P^T.  The transposing LDS read (64
    // bits a lane) hands lane i of a group of 16 the element i % 4 of the 4 x 16-bit pieces that the
    // group's lanes 4 j + i / 4 point at, j = 0 .. 3.  Lane i of a group points at key base + i / 4,
    // dimensions d0 + 4 (i % 4) ..: it receives the keys base .. base + 3 of dimension d0 + i.  The
    // lane's group gives d0 (16 (group % 2) within the tile of 32) and the k-group (group / 2), whose
    // 8 keys of MFMA step st are 16 st + 4 h + {0 .. 3} and 16 st + 8 + 4 h + {0 .. 3}: two reads.
    // With the swizzle 2 (key % 8) the four keys of a read lie in eight different 16-byte columns.
    int vaddr[DT];
    {
        const int gi = lane & 15, grp = lane >> 4;
        const int vkey = 4 * (grp >> 1) + (gi >> 2);            // + 16 st + 8 r: the swizzle does not see those
        const int swz = (2 * (vkey & 7)) & (CPR - 1);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            const int chunk = 4 * dt + 2 * (grp & 1) + ((gi & 3) >> 1);
            vaddr[dt] = vkey * DH + 8 * (chunk ^ swz) + 4 * (gi & 1);
        }
    }
    // three turns a trip, so that the stage is a constant of the code and the LDS addresses are
    // a register plus an immediate
    for (int j3 = 0; j3 < n0; j3 += NST) {
#pragma unroll
      for (int stage = 0; stage < NST; ++stage) {
        const int jb = j3 + stage;
        if (jb >= n0) break;
        const int kb = kb0 + 32 * jb;
        if (jb + 2 < nb) LI_PRE_FETCH((stage + 2) % NST);
        if (active && jb < nb) {                         // (the second group may have a block less: it keeps the barriers)
            // ---- S^T = K Q^T
            f32x16_t sv;
#pragma unroll
            for (int r = 0; r < 16; ++r) sv[r] = 0.f;
            frag8 kf[KS];
#pragma unroll
            for (int st = 0; st < KS; ++st) kf[st].raw = *reinterpret_cast<const u32x4*>(&kv[0][half][stage][kaddr[st]]);
#pragma unroll
            for (int st = 0; st < KS; ++st) sv = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st].v, qf[st].v, sv, 0, 0, 0);
            // ---- softmax over the keys of this lane's query.  The running maximum m is only moved
            // (and the sums so far rescaled, for the whole wave) when some query's scores pass it by
            // more than 2^8: until then the exponentials are taken against the older maximum, which
            // changes no result (numerator and denominator carry the same factor) and stays far
            // inside the range of float and bfloat16.
            // A block that every query of the tile sees whole (most are) needs no masks.
            if (!(kb + 31 <= p0 && kb >= l_last)) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = kb + 8 * (r >> 2) + 4 * h + (r & 3);
                    sv[r] = (key <= pq && key >= lq) ? sv[r] : -INFINITY;
                }
            }
            float mx = max3f(sv[0], sv[1], sv[2]);
#pragma unroll
            for (int r = 3; r < 15; r += 2) mx = max3f(mx, sv[r], sv[r + 1]);
            mx = max3f(mx, sv[15], sv[15]);
            mx = both_halves_max(mx) * scale2;                          // (scale2 > 0)
            if (__any(mx > m + 8.0f)) {
                const float mn = fmaxf(m, mx);
                const float alpha = (mn == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m - mn);   // (m = -inf: nothing summed yet)
                l *= alpha;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
                m = mn;
            }
            const float ms = (m == -INFINITY) ? 0.f : m;         // a query may see no key yet
            float ps = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) { sv[r] = __builtin_amdgcn_exp2f(fmaf(sv[r], scale2, -ms)); ps += sv[r]; }
            l += ps;
            frag8 pf[2];
#pragma unroll
            for (int st = 0; st < 2; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) pf[st].raw.w[i] = pack2_bf16(sv[8 * st + 2 * i], sv[8 * st + 2 * i + 1]);
            // ---- O^T += V^T P^T
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int st = 0; st < 2; ++st) {
                    frag8 vf;
                    const tr4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr4 __attribute__((address_space(3)))*)&kv[1][half][stage][vaddr[dt] + (16 * st) * DH]);
                    const tr4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr4 __attribute__((address_space(3)))*)&kv[1][half][stage][vaddr[dt] + (16 * st + 8) * DH]);
                    vf.raw.w[0] = (uint32_t)(uint16_t)v0[0] | ((uint32_t)(uint16_t)v0[1] << 16);
                    vf.raw.w[1] = (uint32_t)(uint16_t)v0[2] | ((uint32_t)(uint16_t)v0[3] << 16);
                    vf.raw.w[2] = (uint32_t)(uint16_t)v1[0] | ((uint32_t)(uint16_t)v1[1] << 16);
                    vf.raw.w[3] = (uint32_t)(uint16_t)v1[2] | ((uint32_t)(uint16_t)v1[3] << 16);
                    acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf[st].v, acc[dt], 0, 0, 0);
                }
            }
        }
        if (jb + 2 < nb) { LI_ATT_VMCNT(2 * NL); } else { LI_ATT_VMCNT(0); }
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
      }
    }
    // ---- the second group's results go to the first through LDS (the stages are free now)
    __syncthreads();
    float* mrg = reinterpret_cast<float*>(&kv[0][0][0][0]) + (size_t)wave * ((DT * 16 + 2) * 64);
    static_assert(sizeof(kv) >= (size_t)PRE_WAVES * (DT * 16 + 2) * 64 * 4, "the groups' exchange fits the stages");
    if (half == 1 && active) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) mrg[(dt * 16 + r) * 64 + lane] = acc[dt][r];
        mrg[(DT * 16) * 64 + lane] = m;
        mrg[(DT * 16 + 1) * 64 + lane] = l;
    }
    __syncthreads();
    if (half == 1 || !active || ql >= nrows) return;
    {
        const float m1 = mrg[(DT * 16) * 64 + lane], l1 = mrg[(DT * 16 + 1) * 64 + lane];
        const float mn = fmaxf(m, m1);
        const float a0 = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - mn);        // (a group that saw no key brings nothing)
        const float a1 = (m1 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m1 - mn);
        l = l * a0 + l1 * a1;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] = acc[dt][r] * a0 + mrg[(dt * 16 + r) * 64 + lane] * a1;
    }
    l += __shfl_xor(l, 32, LI_WAVE);               // (both halves of a query are past the return together)
    const float inv = l != 0.f ? 1.0f / l : 0.f;
    bf16_t* orow = out + (size_t)(t0 + ql) * nh * DH + (size_t)head * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {           // registers 4 rg .. 4 rg + 3: dimensions 32 dt + 8 rg + 4 h ..
            uint32_t w0 = pack2_bf16(acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv);
            uint32_t w1 = pack2_bf16(acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv);
            uint32_t* dst = reinterpret_cast<uint32_t*>(orow + 32 * dt + 8 * rg + 4 * h);
            dst[0] = w0;
            dst[1] = w1;
        }
}


#define PF_T 32
// ------------------------------------------------ portions of prompts, float32
// The true 32-bit path's kernel for prompts, on the float32 matrix cores (v_mfma_f32_32x32x2_f32: float32
// operands, products and sums; no
// operand is rounded to a shorter format).  A block takes a tile of up to 32 tokens and one kv head; its four
// waves are query heads of that kv head (blockIdx.z picks which four), so a block of 32 keys is fetched once,
// into LDS, for all of them.  As in the bfloat16 kernel a wave works on the TRANSPOSED scores S^T = K Q^T: in
// the result a lane holds 16 keys of ITS query (register r: key 8 (r / 4) + 4 (l / 32) + r % 4), so the softmax
// is arithmetic inside a lane plus one exchange with lane l ^ 32, and those registers are the column operand
// of O^T = V^T P^T as they are: MFMA step s takes register s, i.e. the keys 8 (s / 4) + s % 4 (lane half 0)
// and that + 4 (lane half 1), and the row operand V^T reads the same two keys' values from LDS.  For the
// scores the two k-slots of an MFMA are the head's two halves: lane half h multiplies the dimensions
// (DH / 2) h + s, which it keeps of its query in registers and reads of the keys in 16-byte pieces.
typedef float f32x16m_t __attribute__((ext_vector_type(16)));
template <int DH>
__global__ __launch_bounds__(256) void paged_attention_prefill_f32_mfma_kernel(
    const float* __restrict__ q, int q_row_stride, float* __restrict__ out,
    const float* __restrict__ kc, const float* __restrict__ vc, const int* __restrict__ block_table,
    int max_blocks, const int* __restrict__ tiles, const int* __restrict__ q_start,
    const int* __restrict__ q_len, const int* __restrict__ ctx_len, int nh, int nkv, int page_size,
    int num_pages, int window, float scale) {
    constexpr int RS = DH + 4;                      // row stride in LDS
    constexpr int C4 = DH / 4;                      // float4 pieces of a row
    constexpr int PER = PF_T * C4 / 256;            // pieces of K (and of V) a thread fetches per block of keys
    constexpr int HD = DH / 2, DT = DH / 32;
    static_assert(PER * 256 == PF_T * C4, "head sizes 64 and 128");
    __shared__ __attribute__((aligned(16))) float Ks[PF_T * RS];
    __shared__ __attribute__((aligned(16))) float Vs[PF_T * RS];
    const int tile = gridDim.x - 1 - blockIdx.x, kvh = blockIdx.y;           // (the longest tiles of a segment first)
    const int s = tiles[tile * 4], t0 = tiles[tile * 4 + 1], nrows = tiles[tile * 4 + 2];
    const int G = nh / nkv;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hw = blockIdx.z * 4 + wave;
    const bool active = hw < G;                     // (idle waves still help to fetch and keep the barriers)
    const int head = kvh * G + (active ? hw : 0);
    const int ql = lane & 31, h = lane >> 5;
    const int p0 = ctx_len[s] - q_len[s] + (t0 - q_start[s]);               // position of the tile's first token
    const int p_last = p0 + nrows - 1;
    const int lo0 = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
    const int k_begin = lo0 & ~(PF_T - 1), k_end = p_last + 1;
    const int* table = block_table + (size_t)s * max_blocks;
    // this lane's half of its query (rows past the tile's end repeat the last one and store nothing)
    float qf[HD];
    {
        const float* src = q + (size_t)(t0 + (ql < nrows ? ql : nrows - 1)) * q_row_stride + (size_t)head * DH + HD * h;
#pragma unroll
        for (int c = 0; c < HD / 4; ++c) {
            const float4 v = *reinterpret_cast<const float4*>(src + 4 * c);
            qf[4 * c] = v.x; qf[4 * c + 1] = v.y; qf[4 * c + 2] = v.z; qf[4 * c + 3] = v.w;
        }
    }
    float4 kreg[PER], vreg[PER];
    auto fetch = [&](int kb) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int ci = tid + 256 * i, key = kb + ci / C4, c = ci % C4;
            const int kk = key < k_end ? key : k_end - 1;                    // (masked below; the address stays inside the request)
            int page = table[kk / page_size];
            page = page < 0 ? 0 : (page >= num_pages ? num_pages - 1 : page);
            const size_t off = (((size_t)page * nkv + kvh) * page_size + kk % page_size) * DH + 4 * c;
            kreg[i] = *reinterpret_cast<const float4*>(kc + off);
            vreg[i] = *reinterpret_cast<const float4*>(vc + off);
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int ci = tid + 256 * i, key = ci / C4, c = ci % C4;
            *reinterpret_cast<float4*>(&Ks[key * RS + 4 * c]) = kreg[i];
            *reinterpret_cast<float4*>(&Vs[key * RS + 4 * c]) = vreg[i];
        }
    };
    const int pq = p0 + (ql < nrows ? ql : nrows - 1);       // last visible key of this lane's query
    const int lq = (window > 0 && pq - window + 1 > 0) ? pq - window + 1 : 0;
    f32x16m_t acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[dt][r] = 0.f;
    float m = -INFINITY, l = 0.f;
    fetch(k_begin);
    for (int kb = k_begin; kb < k_end; kb += PF_T) {
        __syncthreads();                            // the block before is done with K and V
        stash();
        __syncthreads();
        if (kb + PF_T < k_end) fetch(kb + PF_T);    // on its way while this block is worked on
        if (!active) continue;
        // ---- S^T = K Q^T
        f32x16m_t sv;
#pragma unroll
        for (int r = 0; r < 16; ++r) sv[r] = 0.f;
#pragma unroll
        for (int c = 0; c < HD / 4; ++c) {
            const float4 kv = *reinterpret_cast<const float4*>(&Ks[ql * RS + HD * h + 4 * c]);
            sv = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qf[4 * c], sv, 0, 0, 0);
            sv = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qf[4 * c + 1], sv, 0, 0, 0);
            sv = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qf[4 * c + 2], sv, 0, 0, 0);
            sv = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qf[4 * c + 3], sv, 0, 0, 0);
        }
        // ---- softmax over the keys of this lane's query (its other half is lane ^ 32)
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int key = kb + 8 * (r >> 2) + 4 * h + (r & 3);
            sv[r] = (key <= pq && key >= lq) ? sv[r] * scale : -INFINITY;
            mx = fmaxf(mx, sv[r]);
        }
        mx = both_halves_max(mx);
        const float mn = fmaxf(m, mx);
        const float alpha = (mn == -INFINITY) ? 1.0f : expf(m - mn);        // (nothing seen yet: nothing to rescale)
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) { sv[r] = (sv[r] == -INFINITY) ? 0.f : expf(sv[r] - mn); ps += sv[r]; }
        l = l * alpha + ps;
        m = mn;
        // ---- O^T = alpha O^T + V^T P^T
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[dt][r] *= alpha;
#pragma unroll
            for (int st = 0; st < 16; ++st) {
                const float v = Vs[(8 * (st >> 2) + 4 * h + (st & 3)) * RS + 32 * dt + ql];
                acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(v, sv[st], acc[dt], 0, 0, 0);
            }
        }
    }
    if (!active || ql >= nrows) return;
    l += __shfl_xor(l, 32, LI_WAVE);               // (both halves of a query are past the return together)
    const float inv = l != 0.f ? 1.0f / l : 0.f;
    float* orow = out + (size_t)(t0 + ql) * nh * DH + (size_t)head * DH;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)              // registers 4 rg .. 4 rg + 3: dimensions 32 dt + 8 rg + 4 h ..
            *reinterpret_cast<float4*>(orow + 32 * dt + 8 * rg + 4 * h) =
                float4{acc[dt][4 * rg] * inv, acc[dt][4 * rg + 1] * inv, acc[dt][4 * rg + 2] * inv, acc[dt][4 * rg + 3] * inv};
}

extern "C" int li_paged_attention_prefill_f32(const void* q, int q_row_stride, void* out, const void* kc,
                                              const void* vc, const int* block_table, int max_blocks,
                                              const int* tiles, int ntiles, const int* q_start, const int* q_len,
                                              const int* ctx_len, int nh, int nkv, int dh, int page_size,
                                              int num_pages, int window, float scale, hipStream_t stream) {
    if (ntiles <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || nh > 65535 || page_size <= 0 || max_blocks <= 0 ||
        num_pages <= 0 || !(scale > 0.f) || (q_row_stride % 4))
        return LI_ERR_SIZE;
    if (nkv > 65535 || (nh / nkv + 3) / 4 > 65535) return LI_ERR_SIZE;
    dim3 grid(ntiles, nkv, (nh / nkv + 3) / 4);
#define LI_PF(DHV) paged_attention_prefill_f32_mfma_kernel<DHV><<<grid, 256, 0, stream>>>( \
        (const float*)q, q_row_stride, (float*)out, (const float*)kc, (const float*)vc, block_table, max_blocks, \
        tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, scale)
    if (dh == 128) LI_PF(128); else if (dh == 64) LI_PF(64); else return LI_ERR_SIZE;
#undef LI_PF
    return li_launch_status();
}

// Into how many runs the keys of every tile are cut (1: not at all).  A block is one tile x kv head x
// four heads of the group x run; a compute unit holds two blocks, each as long as its run of keys,
// and the blocks go over the units in rounds: with few tiles against long contexts (a portion of a
// prompt behind a long cached part, few kv heads) whole units stand idle or a few blocks make a
// round of their own, and a prompt from its start has one tile as long as all its keys while the
// mean is half that.  q_len, ctx_len: the batch's segments in HOST memory (those with one token are
// not the business of this kernel).  Estimated in blocks of 32 keys: the longer of the longest run
// and (rounds of blocks over the units) x (the mean run), each with 8 for a block's start and end,
// + what writing the runs' results and joining them costs; the form with eight waves a block (two halves of the
// keys, no joining kernel), which takes up to one block a unit, is the yardstick where it applies.
// Runs of at least 16 blocks of keys, at most 16 runs, and the partial results within max_bytes.
extern "C" int li_paged_attention_prefill_runs(int nseg, const int* q_len, const int* ctx_len, int nh, int nkv, int dh,
                                               int max_blocks, int window, int tokens, long max_bytes) {
    if (nseg <= 0 || !q_len || !ctx_len || nh <= 0 || nh > 4 * 65535 || nkv <= 0 || nh % nkv || max_blocks > PRE2_TABLE_CAP) return 1;
    int dev = 0, ncu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || ncu <= 0) {
        (void)hipGetLastError();
        ncu = 256;
    }
    long ntiles = 0, work = 0;
    int len = 0;                                                        // the longest tile's blocks of keys
    for (int i = 0; i < nseg; ++i) {
        if (q_len[i] <= 1) continue;
        for (int a = 0; a < q_len[i]; a += 32) {
            const int p0 = ctx_len[i] - q_len[i] + a, rows = q_len[i] - a < 32 ? q_len[i] - a : 32;
            const int lo0 = (window > 0 && p0 - window + 1 > 0) ? p0 - window + 1 : 0;
            const int blocks = (p0 + rows - (lo0 & ~31) + 31) / 32;
            ++ntiles;
            work += blocks;
            len = blocks > len ? blocks : len;
        }
    }
    if (ntiles == 0) return 1;
    const int G = nh / nkv, parts = (G + PRE_WAVES - 1) / PRE_WAVES;
    const long blocks = ntiles * nkv * parts;
    const double mean = (double)work / ntiles;
    auto cost = [&](int runs) {
        const long rounds = (blocks * runs + 2l * ncu - 1) / (2l * ncu);
        const double longest = (len + runs - 1) / runs + 8, all = (double)rounds * (mean / runs + 8);
        // (the runs' results are written and read again, a block of keys takes about 1.1 us)
        const double joining = runs > 1 ? 5.0 + (double)tokens * nh * runs * dh * 8.0 / 6.0e12 / 1.1e-6 : 0.0;
        return (longest > all ? longest : all) + joining;
    };
    double base = cost(1);
    if (blocks <= ncu) {                                                // the form with eight waves a block
        const double halves = (len + 1) / 2 + 8;
        if (halves < base) base = halves;
    }
    int pick = 1;
    double best = 0.9 * base;                                           // (only for a clear gain)
    for (int runs = 2; runs <= MERGE_RUNS_MAX && len / runs >= 16; ++runs) {
        if ((long)tokens * nh * runs * (dh + 2) * 4 > max_bytes) break;
        const double c = cost(runs);
        if (c < best) { best = c; pick = runs; }
    }
    return pick;
}

// tiles: int [ntiles, 4] = (segment, first token of the tile in the batch, rows <= 32, unused)
// runs > 1 (see li_paged_attention_prefill_runs): part_acc [tokens, nh, runs, dh] and part_ml
// [tokens, nh, runs, 2] float32 take the runs' results, which are then joined for the n_merge tokens
// of merge_tokens (null: the tokens 0 .. n_merge - 1).
extern "C" int li_paged_attention_prefill(const void* q, int q_row_stride, void* out, const void* kc,
                                          const void* vc, const int* block_table, int max_blocks,
                                          const int* tiles, int ntiles, const int* q_start, const int* q_len,
                                          const int* ctx_len, int nh, int nkv, int dh, int page_size,
                                          int num_pages, int window, float scale, int runs, float* part_acc,
                                          float* part_ml, const int* merge_tokens, int n_merge, hipStream_t stream) {
    if (ntiles <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || nkv > 65535 || page_size <= 0 || max_blocks <= 0 ||
        max_blocks > PRE_TABLE_CAP || (long long)max_blocks * page_size > (1ll << 21) || !(scale > 0.f))
        return LI_ERR_SIZE;
    if (runs < 1 || runs > MERGE_RUNS_MAX || (runs > 1 && (!part_acc || !part_ml || n_merge <= 0 || nh > 4 * 65535 || max_blocks > PRE2_TABLE_CAP)))
        return LI_ERR_SIZE;
    const int G = nh / nkv;
    const int parts = (G + PRE_WAVES - 1) / PRE_WAVES;
    if ((long)parts * runs > 65535) return LI_ERR_SIZE;
    dim3 grid(ntiles, nkv, parts);
    int dev = 0, ncu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&ncu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || ncu <= 0) {
        (void)hipGetLastError();
        ncu = 256;
    }
#define LI_PRE(DHV) paged_attention_prefill_mfma_kernel<DHV><<<grid, PRE_WAVES * 64, 0, stream>>>( \
        (const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, block_table, max_blocks, \
        tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, scale, ncu)
#define LI_PRE2(DHV, P32V) paged_attention_prefill_dma_kernel<DHV, P32V><<<grid, PRE_WAVES * 64, 0, stream>>>( \
        (const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, block_table, max_blocks, \
        tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, scale, ncu, runs, part_acc, part_ml)
#define LI_PRE3(DHV, P32V) paged_attention_prefill_split_kernel<DHV, P32V><<<grid, 2 * PRE_WAVES * 64, 0, stream>>>( \
        (const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, block_table, max_blocks, \
        tiles, q_start, q_len, ctx_len, nh, nkv, page_size, num_pages, window, scale, ncu)
    if (runs == 1 && max_blocks <= PRE2_TABLE_CAP && (long)ntiles * nkv * parts <= (long)ncu) {      // at most a block a compute unit: the tile's keys in two halves
        const bool p32 = 32 % page_size == 0;
        if (dh == 128) { if (p32) LI_PRE3(128, true); else LI_PRE3(128, false); }
        else if (dh == 64) { if (p32) LI_PRE3(64, true); else LI_PRE3(64, false); }
        else return LI_ERR_SIZE;
    } else
    if (max_blocks <= PRE2_TABLE_CAP) {                       // (longer block tables: the form that keeps 8,192 entries in LDS)
        grid.z = parts * runs;
        const bool p32 = 32 % page_size == 0;
        if (dh == 128) { if (p32) LI_PRE2(128, true); else LI_PRE2(128, false); }
        else if (dh == 64) { if (p32) LI_PRE2(64, true); else LI_PRE2(64, false); }
        else return LI_ERR_SIZE;
        if (runs > 1) {
            if (li_launch_status() != LI_OK) return LI_ERR_LAUNCH;
            attention_merge_runs_kernel<bf16_t><<<dim3(n_merge, (nh + MERGE_RUNS_HEADS - 1) / MERGE_RUNS_HEADS), 256, 0, stream>>>(part_acc, part_ml, merge_tokens, (bf16_t*)out, nh, dh, runs);
        }
    } else
    if (dh == 128) LI_PRE(128); else if (dh == 64) LI_PRE(64); else return LI_ERR_SIZE;
#undef LI_PRE2
#undef LI_PRE3
#undef LI_PRE
#undef LI_PRE_FETCH
#undef LI_PRE_ROW
#undef LI_PRE_STASH
    return li_launch_status();
}

template <typename T>
static int launch_decode(const T* q, int q_row_stride, T* out, const T* kc, const T* vc,
                         const int* block_table, int max_blocks, const int* token_list, int n_tokens,
                         const int* seg_of_token, const int* q_start, const int* q_len, const int* ctx_len,
                         float* part_acc, float* part_ml, int nh, int nkv, int dh, int page_size,
                         int num_pages, int window, float scale, int nsplit, hipStream_t stream) {
    constexpr int E = raw16<T>::E;
    if (dh % E) return LI_ERR_SIZE;
    const int lpk = dh / E;
    if (n_tokens > 0x7fffffff / 1 || nkv > 65535 || nsplit > 65535 || nsplit < 1) return LI_ERR_SIZE;
    dim3 grid(n_tokens, nkv, nsplit);
#define LI_DEC(LPK) paged_attention_decode_kernel<T, LPK, 8><<<grid, 256, 0, stream>>>( \
        q, q_row_stride, out, kc, vc, block_table, max_blocks, token_list, seg_of_token, q_start, q_len, \
        ctx_len, part_acc, part_ml, nh, nkv, dh, page_size, num_pages, window, scale, nsplit)
    switch (lpk) {
        case 1: LI_DEC(1); break;
        case 2: LI_DEC(2); break;
        case 4: LI_DEC(4); break;
        case 8: LI_DEC(8); break;
        case 16: LI_DEC(16); break;
        case 32: LI_DEC(32); break;
        case 64: LI_DEC(64); break;
        default: return LI_ERR_SIZE;
    }
#undef LI_DEC
    if (nsplit > 1) {
        dim3 g2(n_tokens, nh);
        attention_merge_kernel<T><<<g2, 128, 0, stream>>>(part_acc, part_ml, token_list, out, nh, dh, nsplit);
    }
    return li_launch_status();
}

// The matrix-core decode kernel (bfloat16 or float32, head sizes 64 and 128), in its three forms: one run a
// (token, kv head); single-wave blocks with the merge kernel behind them (use_mfma 2); blocks of LI_DECODE_QUAD
// waves that join their runs themselves.
#define LI_DECODE_QUAD 4
template <typename T>
static int launch_decode_mfma(const T* q, int q_row_stride, T* out, const T* kc, const T* vc, const int* block_table,
                              int max_blocks, const int* token_list, int n_tokens, const int* seg_of_token,
                              const int* q_start, const int* q_len, const int* ctx_len, float* part_acc,
                              float* part_ml, int nh, int nkv, int dh, int page_size, int num_pages, int window,
                              float scale, int nsplit, int use_mfma, const int* run_keys, int* done,
                              hipStream_t stream) {
    if (nkv > 65535) return LI_ERR_SIZE;
    // a split's pages must fit the kernel's copy of the block table: `per` keys that begin
    // anywhere in a page touch at most (per + page_size - 2) / page_size + 1 pages
    if (li_decode_split_blocks(max_blocks, page_size, window, nsplit) > DEC_TABLE_CAP) return LI_ERR_SIZE;
    if (dh != 128 && dh != 64) return LI_ERR_SIZE;
    if ((long)max_blocks * page_size > (1L << 21) || page_size > (1 << 16)) return LI_ERR_SIZE;   // (the kernel's key / page_size)
    if (nsplit == 1) {
        dim3 grid(n_tokens, nkv, 1);
#define LI_DM(DHV) paged_attention_decode_mfma_kernel<T, DHV, 1><<<grid, 64, 0, stream>>>( \
        q, q_row_stride, out, kc, vc, block_table, max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, \
        part_acc, part_ml, nh, nkv, page_size, num_pages, window, scale, 1, nullptr, n_tokens, nullptr)
        if (dh == 128) LI_DM(128); else LI_DM(64);
#undef LI_DM
        return li_launch_status();
    }
    const bool listed = run_keys != nullptr;
    if (listed && (n_tokens > RUN_KEYS_MAX_TOKENS || nsplit > 0x7fff)) return LI_ERR_SIZE;
    if (use_mfma == 2) {
        if (!part_acc || !part_ml) return LI_ERR_SIZE;
        dim3 grid(listed ? n_tokens * nsplit : n_tokens, nkv, listed ? 1 : nsplit);
#define LI_DM(DHV) paged_attention_decode_mfma_kernel<T, DHV, 1><<<grid, 64, 0, stream>>>( \
        q, q_row_stride, out, kc, vc, block_table, max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, \
        part_acc, part_ml, nh, nkv, page_size, num_pages, window, scale, nsplit, listed ? run_keys : nullptr, n_tokens, \
        nullptr)
        if (dh == 128) LI_DM(128); else LI_DM(64);
#undef LI_DM
        dim3 g2(n_tokens, nh);
        attention_merge_kernel<T><<<g2, 128, 0, stream>>>(part_acc, part_ml, token_list, out, nh, dh, nsplit,
                                                          listed ? run_keys + 2 : nullptr);
        return li_launch_status();
    }
    if (nsplit % LI_DECODE_QUAD) return LI_ERR_SIZE;
    const int quads = nsplit / LI_DECODE_QUAD;
    if (quads > 1 && (!done || !part_acc || !part_ml)) return LI_ERR_SIZE;
    if ((long)n_tokens * quads > 0x7fffffffL) return LI_ERR_SIZE;
    dim3 grid(listed ? n_tokens * quads : n_tokens, nkv, listed ? 1 : quads);
#define LI_DM(DHV) paged_attention_decode_mfma_kernel<T, DHV, LI_DECODE_QUAD><<<grid, 64 * LI_DECODE_QUAD, 0, stream>>>( \
        q, q_row_stride, out, kc, vc, block_table, max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, \
        part_acc, part_ml, nh, nkv, page_size, num_pages, window, scale, quads, listed ? run_keys : nullptr, n_tokens, done)
    if (dh == 128) LI_DM(128); else LI_DM(64);
#undef LI_DM
    return li_launch_status();
}

// Single-query tokens of the batch (token_list, or all tokens when it is null).
// part_acc: float [n_tokens, nh, nsplit, dh]; part_ml: float [n_tokens, nh, nsplit, 2] (unused when nsplit is 1).
// run_keys (may be null; the matrix-core kernel with nsplit > 1 only): what li_decode_run_keys (with group
// LI_DECODE_QUAD) left on the device for this batch: the run length and the list of the runs that have keys.
// The matrix-core kernel with nsplit > 1 takes nsplit as a multiple of LI_DECODE_QUAD (a block works through
// that many runs and joins them) and needs `done`: int [n_tokens * nkv], zero before the first call; every
// call leaves it zero.  Its blocks join their results themselves; the other kernels run a merge kernel.
extern "C" int li_decode_quad(void) { return LI_DECODE_QUAD; }
extern "C" int li_paged_attention_decode(const void* q, int q_row_stride, void* out, const void* kc,
                                         const void* vc, int dtype, const int* block_table, int max_blocks,
                                         const int* token_list, int n_tokens, const int* seg_of_token,
                                         const int* q_start, const int* q_len, const int* ctx_len,
                                         float* part_acc, float* part_ml, int nh, int nkv, int dh,
                                         int page_size, int num_pages, int window, float scale, int nsplit,
                                         int use_mfma, const int* run_keys, int* done, hipStream_t stream) {
    if (n_tokens <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || dh <= 0 || dh > ATT_MAX_DH || page_size <= 0 ||
        max_blocks <= 0)
        return LI_ERR_SIZE;
    if (nsplit < 1 || nsplit > MERGE_MAX_SPLITS) return LI_ERR_SIZE;      // the merge kernel keeps a weight per split in LDS
    if (dtype == LI_F32 && !use_mfma)
        return launch_decode<float>((const float*)q, q_row_stride, (float*)out, (const float*)kc, (const float*)vc,
                                    block_table, max_blocks, token_list, n_tokens, seg_of_token, q_start, q_len,
                                    ctx_len, part_acc, part_ml, nh, nkv, dh, page_size, num_pages, window, scale,
                                    nsplit, stream);
    if (dtype == LI_F32)
        return launch_decode_mfma<float>((const float*)q, q_row_stride, (float*)out, (const float*)kc, (const float*)vc,
                                         block_table, max_blocks, token_list, n_tokens, seg_of_token, q_start, q_len,
                                         ctx_len, part_acc, part_ml, nh, nkv, dh, page_size, num_pages, window, scale,
                                         nsplit, use_mfma, run_keys, done, stream);
    if (dtype == LI_BF16 && use_mfma)
        return launch_decode_mfma<bf16_t>((const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc,
                                          (const bf16_t*)vc, block_table, max_blocks, token_list, n_tokens, seg_of_token,
                                          q_start, q_len, ctx_len, part_acc, part_ml, nh, nkv, dh, page_size, num_pages,
                                          window, scale, nsplit, use_mfma, run_keys, done, stream);
    if (dtype == LI_BF16)
        return launch_decode<bf16_t>((const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc,
                                     (const bf16_t*)vc, block_table, max_blocks, token_list, n_tokens,
                                     seg_of_token, q_start, q_len, ctx_len, part_acc, part_ml, nh, nkv, dh,
                                     page_size, num_pages, window, scale, nsplit, stream);
    return LI_ERR_DTYPE;
}

extern "C" int li_paged_attention(const void* q, int q_row_stride, void* out, const void* kc,
                                  const void* vc, int dtype, const int* block_table, int max_blocks,
                                  const int* token_list, const int* seg_of_token, const int* q_start,
                                  const int* q_len, const int* ctx_len, int num_segments, int T, int max_q_len,
                                  int max_ctx_len, int nh, int nkv, int dh, int page_size,
                                  int num_pages, int window, float scale, hipStream_t stream) {
    if (T <= 0 || nh <= 0 || nkv <= 0 || nh % nkv || dh <= 0 || dh > ATT_MAX_DH || nh > 65535 ||
        page_size <= 0 || max_blocks <= 0)
        return LI_ERR_SIZE;
    dim3 grid(T, nh);
    if (dtype == LI_F32)
        paged_attention_wave_kernel<float><<<grid, 64, 0, stream>>>(
            (const float*)q, q_row_stride, (float*)out, (const float*)kc, (const float*)vc, block_table,
            max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, nh, nkv, dh, page_size, num_pages, window, scale);
    else if (dtype == LI_BF16)
        paged_attention_wave_kernel<bf16_t><<<grid, 64, 0, stream>>>(
            (const bf16_t*)q, q_row_stride, (bf16_t*)out, (const bf16_t*)kc, (const bf16_t*)vc, block_table,
            max_blocks, token_list, seg_of_token, q_start, q_len, ctx_len, nh, nkv, dh, page_size, num_pages, window, scale);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
