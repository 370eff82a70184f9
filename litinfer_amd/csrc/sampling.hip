// Choosing the next token from float32 logits: argmax (lowest index on ties)
// and temperature / top-k / top-p sampling by inverse CDF with a uniform
// number from the request's own counter-based stream, which the host derives or,
// for requests whose sampling state lies in the per-slot table on the device
// (li_sample_prepare), the device itself.
#include "common.h"
#include "li_noalloc.h"
#include <math.h>
#include <mutex>
#include <stdio.h>

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

// Two stages, so that a few rows still use many compute units: stage 1 finds the
// (maximum, lowest index) of each of ARGMAX_CHUNKS contiguous chunks of a row, stage 2
// combines a row's chunks.  Ties go to the lower index in both.
#define ARGMAX_CHUNKS 32

__global__ __launch_bounds__(SMP_NT) void argmax_partial_kernel(const float* __restrict__ logits,
                                                                float* __restrict__ pv, int* __restrict__ pi,
                                                                int V, int chunk) {
    __shared__ float sv[SMP_NT / LI_WAVE];
    __shared__ int si[SMP_NT / LI_WAVE];
    const float* row = logits + (size_t)blockIdx.x * V;
    const int c0 = blockIdx.y * chunk, c1 = (c0 + chunk < V) ? c0 + chunk : V;
    float v = -INFINITY;
    int i = 0x7fffffff;
    for (int j = c0 + threadIdx.x; j < c1; j += SMP_NT) {
        const float x = row[j];
        if (x > v || i == 0x7fffffff) { v = x; i = j; }   // strictly greater: the first maximum stays
    }
    block_argmax(v, i, sv, si);
    if (threadIdx.x == 0) { pv[blockIdx.x * gridDim.y + blockIdx.y] = v; pi[blockIdx.x * gridDim.y + blockIdx.y] = i; }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                          int* __restrict__ out, int nchunks) {
    float v = -INFINITY;
    int i = 0x7fffffff;
    for (int c = threadIdx.x; c < nchunks; c += 64) argmax_combine(v, i, pv[blockIdx.x * nchunks + c], pi[blockIdx.x * nchunks + c]);
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o, LI_WAVE);
        const int oi = __shfl_xor(i, o, LI_WAVE);
        argmax_combine(v, i, ov, oi);
    }
    if (threadIdx.x == 0) out[blockIdx.x] = i;
}

// scratch_v, scratch_i: n * ARGMAX_CHUNKS floats / ints
extern "C" int li_argmax_rows(const float* logits, int* out, float* scratch_v, int* scratch_i, int n, int V,
                              hipStream_t stream) {
    if (n <= 0 || V <= 0) return LI_ERR_SIZE;
    int nchunks = (V + 4095) / 4096;
    if (nchunks > ARGMAX_CHUNKS) nchunks = ARGMAX_CHUNKS;
    const int chunk = (V + nchunks - 1) / nchunks;
    argmax_partial_kernel<<<dim3(n, nchunks), SMP_NT, 0, stream>>>(logits, scratch_v, scratch_i, V, chunk);
    argmax_final_kernel<<<n, 64, 0, stream>>>(scratch_v, scratch_i, out, nchunks);
    return li_launch_status();
}

// ------------------------------------------------- argmax that allocates nothing
// The same two kernels with their partial results in a file-scope device array instead of
// buffers that the caller brings: for callers that cannot allocate (li_noalloc.h).  Every
// GPU holds its own copy of the array at its own address; host code must use the address
// that hipGetSymbolAddress gives for the current device, never the array's name.
static __device__ __align__(256) unsigned char scratch[LI_ARGMAX_NOALLOC_MAX_ROWS * ARGMAX_CHUNKS * 8];

#define LI_NOALLOC_MAX_DEVICES 64
static void* g_scratch_ptr[LI_NOALLOC_MAX_DEVICES];       // the array's address on each device, once asked for
static std::mutex g_scratch_mutex;
static thread_local char g_noalloc_error[200];

static int noalloc_fail(int code, const char* what, hipError_t e) {
    if (e != hipSuccess) snprintf(g_noalloc_error, sizeof g_noalloc_error, "%s: %s", what, hipGetErrorString(e));
    else snprintf(g_noalloc_error, sizeof g_noalloc_error, "%s", what);
    return code;
}

// The scratch array's address on the current device (asked for once per device).
static int noalloc_scratch(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return noalloc_fail(LI_ERR_LAUNCH, "li_argmax_rows_noalloc: hipGetDevice", e);
    if (dev < 0 || dev >= LI_NOALLOC_MAX_DEVICES)
        return noalloc_fail(LI_ERR_SIZE, "li_argmax_rows_noalloc: device number beyond the table of scratch addresses", hipSuccess);
    std::lock_guard<std::mutex> hold(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return noalloc_fail(LI_ERR_LAUNCH, "li_argmax_rows_noalloc: hipGetSymbolAddress(scratch)", e);
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return LI_OK;
}

extern "C" int li_argmax_rows_noalloc_init(void) {
    void* p;
    return noalloc_scratch(&p);
}

extern "C" int li_argmax_rows_noalloc_max_rows(void) { return LI_ARGMAX_NOALLOC_MAX_ROWS; }

extern "C" const char* li_argmax_rows_noalloc_error(void) { return g_noalloc_error; }

extern "C" int li_argmax_rows_noalloc(const float* logits, int* out, int n, int V, hipStream_t stream) {
    g_noalloc_error[0] = 0;
    if (n <= 0 || V <= 0) return noalloc_fail(LI_ERR_SIZE, "li_argmax_rows_noalloc: rows and vocabulary must be positive", hipSuccess);
    if (n > LI_ARGMAX_NOALLOC_MAX_ROWS) {
        snprintf(g_noalloc_error, sizeof g_noalloc_error,
                 "li_argmax_rows_noalloc: %d rows are more than the %d that the scratch array holds; "
                 "use li_argmax_rows with buffers of the caller", n, LI_ARGMAX_NOALLOC_MAX_ROWS);
        return LI_ERR_SIZE;
    }
    void* base = nullptr;
    const int rc = noalloc_scratch(&base);
    if (rc != LI_OK) return rc;
    // partial maxima first, their indices behind them; stage 1 writes every place that stage 2
    // reads, so nothing of an earlier call's contents has to be cleared
    float* pv = reinterpret_cast<float*>(base);
    int* pi = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + (size_t)LI_ARGMAX_NOALLOC_MAX_ROWS * ARGMAX_CHUNKS * 4);
    int nchunks = (V + 4095) / 4096;
    if (nchunks > ARGMAX_CHUNKS) nchunks = ARGMAX_CHUNKS;
    const int chunk = (V + nchunks - 1) / nchunks;
    argmax_partial_kernel<<<dim3(n, nchunks), SMP_NT, 0, stream>>>(logits, pv, pi, V, chunk);
    argmax_final_kernel<<<n, 64, 0, stream>>>(pv, pi, out, nchunks);
    if (li_launch_status() != LI_OK) return noalloc_fail(LI_ERR_LAUNCH, "li_argmax_rows_noalloc: launch failed", hipSuccess);
    return LI_OK;
}

// ---------------------------------------------------------------- sampling
// The candidates are ordered by (value descending, index ascending); top-k keeps the first k, top-p
// then the shortest prefix whose softmax mass (among the top-k survivors) reaches p; the survivors'
// softmax is sampled by inverse CDF over ASCENDING ids with the given uniform number.
// Two kernels.  The first has a block for every tile of SMP_TILE ids of every row, so that a few
// rows still use many compute units: a tile's maximum, and for rows without top-k and top-p its
// softmax sum, for greedy rows its argmax.  The second has one block per row.  It reads the row in
// the same tiles (thread t the 8 consecutive ids t * 8 ... of a tile: whole lines), in as few
// passes as it can: the thresholds of top-k and top-p are found four bits a pass over the
// order-preserving integer image of the floats (16 counts or 16 masses a thread and pass).  Every
// count and every mass is added in a fixed order, so the same inputs always give the same token.
constexpr int SMP_TILE = SMP_NT * 8;
constexpr int SMP_WAVES = SMP_NT / LI_WAVE;

__device__ __forceinline__ uint32_t sort_key(float z) {
    const uint32_t b = __float_as_uint(z);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ bool sample_unfiltered(int k, float p, int V) { return !(k > 0 && k < V) && !(p > 0.f && p < 1.f); }

__device__ __forceinline__ int block_sum_int(int v, int* smem) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LI_WAVE);
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < SMP_WAVES; ++i) t += smem[i];
    return t;
}

__device__ __forceinline__ float block_max_f(float v, float* smem) {
    v = wave_max(v);
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float t = smem[0];
#pragma unroll
    for (int i = 1; i < SMP_WAVES; ++i) t = fmaxf(t, smem[i]);
    return t;
}

__device__ __forceinline__ int block_min_int(int v, int* smem) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, LI_WAVE));
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    int t = smem[0];
#pragma unroll
    for (int i = 1; i < SMP_WAVES; ++i) t = min(t, smem[i]);
    return t;
}

// The 16 sums of a pass over the whole block, left in tot[0..15] for every thread to read.  Within a
// wave the lanes halve what they hold step by step (a lane keeps one half of its sums and gets the
// other lane's part of that half: 8 + 4 + 2 + 1 exchanges), until each lane holds one sum of its 16
// lanes, then the four groups of 16 lanes are added: 17 exchanges instead of 96; then the waves in
// their order.  The order of the additions is fixed.  work: SMP_WAVES * 16 values.
template <typename T>
__device__ __forceinline__ void block_sum16(T (&c)[16], T* work, T* tot) {
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
#define LI_HALVE(H, MASK)                                                         \
    {                                                                             \
        const bool upper = (lane & (MASK)) != 0;                                  \
        _Pragma("unroll") for (int i = 0; i < (H); ++i) {                         \
            const T give = upper ? c[i] : c[i + (H)];                             \
            const T keep = upper ? c[i + (H)] : c[i];                             \
            c[i] = keep + __shfl_xor(give, (MASK), LI_WAVE);                      \
        }                                                                         \
    }
    LI_HALVE(8, 1)
    LI_HALVE(4, 2)
    LI_HALVE(2, 4)
    LI_HALVE(1, 8)
#undef LI_HALVE
    c[0] += __shfl_xor(c[0], 16, LI_WAVE);
    c[0] += __shfl_xor(c[0], 32, LI_WAVE);
    // lane l < 16 now holds the wave's sum number 8 (l & 1) + 4 (l >> 1 & 1) + 2 (l >> 2 & 1) + (l >> 3 & 1)
    __syncthreads();                                 // (the last pass's totals have been read)
    if (lane < 16) work[w * 16 + 8 * (lane & 1) + 4 * ((lane >> 1) & 1) + 2 * ((lane >> 2) & 1) + ((lane >> 3) & 1)] = c[0];
    __syncthreads();
    if (threadIdx.x < 16) {
        T t = 0;
        for (int i = 0; i < SMP_WAVES; ++i) t += work[i * 16 + threadIdx.x];
        tot[threadIdx.x] = t;
    }
    __syncthreads();
}

// Sum of v over the threads before this one, in thread order.  work: SMP_WAVES values.
template <typename T>
__device__ __forceinline__ T block_sum_before(T v, T* work) {
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    T inc = v;
#pragma unroll
    for (int o = 1; o < LI_WAVE; o <<= 1) {
        const T t = __shfl_up(inc, o, LI_WAVE);
        if (lane >= o) inc += t;
    }
    T before = __shfl_up(inc, 1, LI_WAVE);
    if (lane == 0) before = 0;
    __syncthreads();
    if (lane == LI_WAVE - 1) work[w] = inc;
    __syncthreads();
    T base = 0;
    for (int i = 0; i < w; ++i) base += work[i];
    return base + before;
}

// A thread's 8 ids of a tile as z = logit / T (whole 16-byte loads where the row allows them)
__device__ __forceinline__ void load_ids8(const float* __restrict__ row, int j0, int V, float T, bool vec, float (&z)[8]) {
    if (vec && j0 + 8 <= V) {
        const float4 a = *reinterpret_cast<const float4*>(row + j0), b = *reinterpret_cast<const float4*>(row + j0 + 4);
        z[0] = a.x / T; z[1] = a.y / T; z[2] = a.z / T; z[3] = a.w / T;
        z[4] = b.x / T; z[5] = b.y / T; z[6] = b.z / T; z[7] = b.w / T;
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) z[e] = (j0 + e < V) ? row[j0 + e] / T : -INFINITY;
    }
}

// f(z, id) for this thread's ids of all tiles, ascending
template <typename F>
__device__ __forceinline__ void each_id(const float* __restrict__ row, int V, float T, bool vec, int ntiles, F&& f) {
    for (int tile = 0; tile < ntiles; ++tile) {
        const int j0 = tile * SMP_TILE + (int)threadIdx.x * 8;
        if (j0 >= V) break;
        float z[8];
        load_ids8(row, j0, V, T, vec, z);
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (j0 + e < V) f(z[e], j0 + e);
    }
}

// tau = the kk-th largest key among the z that `each` hands out (to all threads of the block together),
// need (>= 1) = how many of the keys equal to tau are among the kk largest.  Four bits a pass: counts of
// the 16 values of the next digit among the keys that agree with the digits found so far.
template <typename Each>
__device__ __forceinline__ void radix_kth(Each&& each, int kk, uint32_t& tau, int& need, int* work_i, int* tot_i) {
    tau = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
        int cnt[16];
#pragma unroll
        for (int b = 0; b < 16; ++b) cnt[b] = 0;
        each([&](float z) {
            const uint32_t key = sort_key(z);
            if (shift == 28 || (key >> (shift + 4)) == (tau >> (shift + 4))) {
                const int d = (key >> shift) & 15;
#pragma unroll
                for (int b = 0; b < 16; ++b) cnt[b] += (d == b);
            }
        });
        block_sum16(cnt, work_i, tot_i);
        int above = 0, d = 15;
        for (; d > 0; --d) {
            if (above + tot_i[d] >= kk) break;
            above += tot_i[d];
        }
        kk -= above;
        tau |= (uint32_t)d << shift;
    }
    need = kk;
}

// Top-p among the survivors of top-k (cut: the keys above tau, and `ties` keys equal to tau with
// e_ties = their mass together; not cut: all keys): tp = the largest key c with mass(keys >= c) >=
// `remaining`, four bits a pass (masses by the next digit); on return `remaining` is what the keys
// equal to tp have to bring.  m: the maximum that masses are taken against.
template <typename Each>
__device__ __forceinline__ void radix_mass(Each&& each, bool cut, uint32_t tau, int ties, float e_ties, float m,
                                           float& remaining, uint32_t& tp, float* work_f, float* tot_f) {
    tp = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
        float mass[16];
#pragma unroll
        for (int b = 0; b < 16; ++b) mass[b] = 0.f;
        each([&](float z) {
            const uint32_t key = sort_key(z);
            if ((!cut || key > tau) && (shift == 28 || (key >> (shift + 4)) == (tp >> (shift + 4)))) {
                const int d = (key >> shift) & 15;
                const float e = expf(z - m);
#pragma unroll
                for (int b = 0; b < 16; ++b) mass[b] += (d == b) ? e : 0.f;
            }
        });
        block_sum16(mass, work_f, tot_f);
        const bool ties_here = cut && ties > 0 && (shift == 28 || (tau >> (shift + 4)) == (tp >> (shift + 4)));
        const int d_ties = (tau >> shift) & 15;
        float above = 0.f;
        int d = 15, lowest = -1;
        bool reached = false;
        for (; d >= 0; --d) {
            const float t = tot_f[d] + ((ties_here && d == d_ties) ? e_ties : 0.f);
            if (t > 0.f) lowest = d;
            if (t > 0.f && above + t >= remaining) { reached = true; break; }
            above += t;
        }
        if (!reached) {                       // rounding left the target just above the sum: the lowest digit with mass
            d = lowest < 0 ? 0 : lowest;
            above = 0.f;
            for (int b = 15; b > d; --b) above += tot_f[b] + ((ties_here && b == d_ties) ? e_ties : 0.f);
        }
        remaining -= above;
        tp |= (uint32_t)d << shift;
    }
}

// how many of the keys equal to tp count, from what they have to bring
__device__ __forceinline__ int ties_needed(float remaining, uint32_t tp, float m) {
    const float e_tp = expf(key_value(tp) - m);
    if (!(e_tp > 0.f)) return 0x7fffffff;     // ties without mass: all of them
    const float q = ceilf(remaining / e_tp);
    return q < 1.f ? 1 : (q > 2.0e9f ? 0x7fffffff : (int)q);
}

// Rows with top-k or top-p: the first kernel hands the second one, per tile, the tile's SMP_KC
// or fewer largest ids (in the order (value descending, id ascending)), so that the second kernel
// searches among ntiles * kc candidates in registers instead of reading the row pass after pass.
// With top-k <= SMP_KC the candidates hold all survivors (kc = k).  With top-p alone kc = SMP_KC_P
// and the second kernel checks that the prefix ends above the kc-th largest id of the row, whose
// betters are all among the candidates; otherwise it reads the row.  0: no candidates.
constexpr int SMP_KC = 256, SMP_KC_P = 128, SMP_CAND_PER_THREAD = 8;
__device__ __forceinline__ int sample_candidates(int k, float p, int V, int ntiles) {
    if (sample_unfiltered(k, p, V)) return 0;
    const int kc = (k > 0 && k < V) ? k : SMP_KC_P;
    return (kc <= SMP_KC && (long)kc * ntiles <= (long)SMP_NT * SMP_CAND_PER_THREAD) ? kc : 0;
}

__global__ __launch_bounds__(SMP_NT) void sample_tiles_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, float* __restrict__ tile_m, float* __restrict__ tile_s,
    int* __restrict__ tile_i, float* __restrict__ cand_z, int* __restrict__ cand_id, int V) {
    __shared__ float sf[SMP_WAVES];
    __shared__ int si[SMP_WAVES];
    __shared__ int work_i[SMP_WAVES * 16], tot_i[16];
    const int tile = blockIdx.x, ntiles = gridDim.x, r = blockIdx.y, tid = threadIdx.x;
    const float* row = logits + (size_t)r * V;
    const float T = temperature[r];
    const int j0 = tile * SMP_TILE + tid * 8;
    const size_t slot = (size_t)r * ntiles + tile;
    if (!(T > 0.f)) {                                          // greedy: the tile's (maximum, lowest index)
        float v = -INFINITY;
        int i = 0x7fffffff;
        for (int e = 0; e < 8 && j0 + e < V; ++e) {
            const float x = row[j0 + e];
            if (x > v || i == 0x7fffffff) { v = x; i = j0 + e; }
        }
        block_argmax(v, i, sf, si);
        if (tid == 0) { tile_m[slot] = v; tile_i[slot] = i; }
        return;
    }
    float z[8], m = -INFINITY;
    load_ids8(row, j0, V, T, (reinterpret_cast<uintptr_t>(row) & 15) == 0, z);
#pragma unroll
    for (int e = 0; e < 8; ++e) m = fmaxf(m, z[e]);
    m = block_max_f(m, sf);
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += (j0 + e < V && m > -INFINITY) ? expf(z[e] - m) : 0.f;       // (a tile of -inf alone has no mass)
    sum = block_sum<SMP_NT>(sum, sf);
    if (tid == 0) { tile_m[slot] = m; tile_s[slot] = sum; }
    const int kc = sample_candidates(top_k[r], top_p[r], V, ntiles);
    if (kc == 0) return;
    // the tile's kc largest ids, written in id order
    const int in_tile = min(SMP_TILE, V - tile * SMP_TILE);
    const bool all = in_tile <= kc;
    uint32_t tau = 0u;
    int need = 0x7fffffff;
    if (!all)
        radix_kth([&](auto f) {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (j0 + e < V) f(z[e]);
        }, kc, tau, need, work_i, tot_i);
    int eq = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) eq += (j0 + e < V) && sort_key(z[e]) == tau;
    int rank = all ? 0 : block_sum_before(eq, si);
    bool in[8];
    int mine = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const uint32_t key = sort_key(z[e]);
        in[e] = (j0 + e < V) && (all || key > tau || (key == tau && rank++ < need));
        mine += in[e];
    }
    int pos = block_sum_before(mine, si);
    const size_t base = slot * SMP_KC;
#pragma unroll
    for (int e = 0; e < 8; ++e)
        if (in[e]) {
            cand_z[base + pos] = z[e];
            cand_id[base + pos] = j0 + e;
            ++pos;
        }
}

// tile_m, tile_s, tile_i, cand_z, cand_id: what sample_tiles_kernel left for the row's ntiles tiles (ntiles <= SMP_NT)
__global__ __launch_bounds__(SMP_NT) void sample_rows_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ uniform, int* __restrict__ out, int V,
    const float* __restrict__ tile_m, const float* __restrict__ tile_s, const int* __restrict__ tile_i,
    const float* __restrict__ cand_z, const int* __restrict__ cand_id, int ntiles) {
    __shared__ float sf[SMP_WAVES];
    __shared__ int si[SMP_WAVES];
    __shared__ float tile_sum[SMP_NT];               // the survivors' mass of every tile
    __shared__ int ties_before[SMP_NT];              // ids at the threshold before every tile
    __shared__ float work_f[SMP_WAVES * 16], tot_f[16];
    __shared__ int work_i[SMP_WAVES * 16], tot_i[16];
    __shared__ float pick_f[3];
    __shared__ int pick_i[1];
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * V;
    const float T = temperature[r];
    tile_m += (size_t)r * ntiles;
    tile_s += (size_t)r * ntiles;
    tile_i += (size_t)r * ntiles;
    if (!(T > 0.f)) {                                          // greedy: the tiles' maxima, ties to the lower id
        float v = -INFINITY;
        int i = 0x7fffffff;
        for (int t = tid; t < ntiles; t += SMP_NT) argmax_combine(v, i, tile_m[t], tile_i[t]);
        block_argmax(v, i, sf, si);
        if (tid == 0) out[r] = i;
        return;
    }
    const bool vec = (reinterpret_cast<uintptr_t>(row) & 15) == 0;
    const int k = top_k[r];
    const float p = top_p[r];
    const bool filtered = !sample_unfiltered(k, p, V);
    const bool by_k = k > 0 && k < V, by_p = p > 0.f && p < 1.f;

    // The survivors are the ids with key > tau and the first `need` (in id order) of those with key == tau.
    bool cut = false;
    uint32_t tau = 0u;
    int need = 0x7fffffff;
    float m = -INFINITY;                              // the maximum that masses are taken against
    if (filtered)
        for (int t = 0; t < ntiles; ++t) m = fmaxf(m, tile_m[t]);

    const int kc = sample_candidates(k, p, V, ntiles);
    if (kc > 0) {
        // ---- among the candidates: slot s = tile * kc + place, ascending ids; thread t has the slots t * C ...
        const int slots = ntiles * kc, C = (slots + SMP_NT - 1) / SMP_NT;
        float cz[SMP_CAND_PER_THREAD];
        int cid[SMP_CAND_PER_THREAD];
        bool have[SMP_CAND_PER_THREAD];
        int total = 0;                                // candidates in all
        for (int t = 0; t < ntiles; ++t) total += min(kc, V - t * SMP_TILE);
#pragma unroll
        for (int c = 0; c < SMP_CAND_PER_THREAD; ++c) {
            const int s = tid * C + c;
            have[c] = false;
            cz[c] = -INFINITY;
            cid[c] = 0;
            if (c < C && s < slots) {
                const int t = s / kc, i = s % kc;
                if (i < min(kc, V - t * SMP_TILE)) {
                    const size_t at = ((size_t)r * ntiles + t) * SMP_KC + i;
                    have[c] = true;
                    cz[c] = cand_z[at];
                    cid[c] = cand_id[at];
                }
            }
        }
        auto each = [&](auto f) {
#pragma unroll
            for (int c = 0; c < SMP_CAND_PER_THREAD; ++c)
                if (have[c]) f(cz[c]);
        };
        // the k-th largest (top-k), or the kc-th: above it the candidates are all there is
        uint32_t tau_c;
        int need_c;
        radix_kth(each, min(by_k ? k : kc, total), tau_c, need_c, work_i, tot_i);
        bool exact = true;
        if (by_k) { cut = true; tau = tau_c; need = need_c; }
        if (by_p) {
            float zk = 0.f;
            int eq = 0;
            each([&](float z) {
                const uint32_t key = sort_key(z);
                if (!cut || key > tau) zk += expf(z - m);
                else if (key == tau) ++eq;
            });
            zk = block_sum<SMP_NT>(zk, sf);
            const int ties = cut ? min(need, block_sum_int(eq, si)) : 0;
            const float e_ties = cut ? (float)ties * expf(key_value(tau) - m) : 0.f;
            if (!cut && total < V) {                  // the mass of all ids, from the tiles' sums
                zk = 0.f;
                for (int t = 0; t < ntiles; ++t) zk += tile_s[t] * expf(tile_m[t] - m);
            }
            float remaining = p * (zk + e_ties);
            uint32_t tp;
            radix_mass(each, cut, tau, ties, e_ties, m, remaining, tp, work_f, tot_f);
            if (!by_k && total < V && !(tp > tau_c)) exact = false;       // the prefix may go on beyond the candidates
            const int need_p = ties_needed(remaining, tp, m);
            need = (cut && tp == tau) ? min(need, need_p) : need_p;
            tau = tp;
            cut = true;
        }
        if (exact) {
            // inverse CDF over the surviving candidates in id order
            int eq = 0;
            each([&](float z) { eq += sort_key(z) == tau; });
            const bool ranked = block_sum_int(eq, si) > need;
            const int rank0 = ranked ? block_sum_before(eq, work_i) : 0;
            float mine = 0.f;
            bool any = false;
            {
                int rank = rank0;
#pragma unroll
                for (int c = 0; c < SMP_CAND_PER_THREAD; ++c) {
                    if (!have[c]) continue;
                    const uint32_t key = sort_key(cz[c]);
                    if (key > tau || (key == tau && (!ranked || rank++ < need))) { mine += expf(cz[c] - m); any = true; }
                }
            }
            const float run0 = block_sum_before(mine, work_f);
            if (tid == SMP_NT - 1) pick_f[0] = uniform[r] * (run0 + mine);
            __syncthreads();
            const float target = pick_f[0];
            int chosen = block_min_int((any && run0 + mine >= target) ? tid : 0x7fffffff, si);
            if (chosen == 0x7fffffff) chosen = -block_min_int(any ? -tid : 1, si);
            if (tid == chosen) {
                float run = run0;
                int rank = rank0, pick = cid[0];
#pragma unroll
                for (int c = 0; c < SMP_CAND_PER_THREAD; ++c) {
                    if (!have[c]) continue;
                    const uint32_t key = sort_key(cz[c]);
                    if (!(key > tau || (key == tau && (!ranked || rank++ < need)))) continue;
                    pick = cid[c];
                    run += expf(cz[c] - m);
                    if (run >= target) break;
                }
                out[r] = pick;
            }
            return;
        }
        cut = false;                                  // from the row itself, then
        tau = 0u;
        need = 0x7fffffff;
    }

    int tile = 0;                                     // the tile that holds the target,
    float before = 0.f, target = 0.f;                 // the mass before it and the target, in units of exp(z - m)
    auto each_of_row = [&](auto f) { each_id(row, V, T, vec, ntiles, [&](float z, int) { f(z); }); };
    if (filtered) {
        if (by_k) {
            cut = true;
            radix_kth(each_of_row, k, tau, need, work_i, tot_i);
        }
        if (by_p) {
            // mass of the top-k survivors, and how many ids sit at tau
            float zk = 0.f;
            int eq = 0;
            each_of_row([&](float z) {
                const uint32_t key = sort_key(z);
                if (!cut || key > tau) zk += expf(z - m);
                else if (key == tau) ++eq;
            });
            zk = block_sum<SMP_NT>(zk, sf);
            const int ties = cut ? min(need, block_sum_int(eq, si)) : 0;
            const float e_ties = cut ? (float)ties * expf(key_value(tau) - m) : 0.f;
            float remaining = p * (zk + e_ties);      // mass that the prefix has to reach
            uint32_t tp;
            radix_mass(each_of_row, cut, tau, ties, e_ties, m, remaining, tp, work_f, tot_f);
            const int need_p = ties_needed(remaining, tp, m);
            need = (cut && tp == tau) ? min(need, need_p) : need_p;
            tau = tp;
            cut = true;
        }
    }

    // ---- inverse CDF over ascending ids among the survivors
    // Are there more ids at tau than count?  Then an id's place among them decides (ties_before).
    bool ranked = false;
    if (cut) {
        int eq = 0;
        each_of_row([&](float z) { eq += sort_key(z) == tau; });
        ranked = block_sum_int(eq, si) > need;
        if (ranked) {
            int running = 0;
            for (int t = 0; t < ntiles; ++t) {
                const int j0 = t * SMP_TILE + tid * 8;
                float z[8];
                int c = 0;
                if (j0 < V) {
                    load_ids8(row, j0, V, T, vec, z);
#pragma unroll
                    for (int e = 0; e < 8; ++e) c += (j0 + e < V) && sort_key(z[e]) == tau;
                }
                c = block_sum_int(c, si);
                if (tid == 0) ties_before[t] = running;
                running += c;
            }
            __syncthreads();
        }
    }
    // this thread's ids of a tile: their mass (sum in id order), whether any survives, and the place
    // among the ids at tau of its first one
    auto mine_of = [&](int t, bool& any, int& rank0) {
        const int j0 = t * SMP_TILE + tid * 8;
        float z[8];
        any = false;
        rank0 = 0;
        if (j0 < V) load_ids8(row, j0, V, T, vec, z);
        if (ranked) {
            int c = 0;
            if (j0 < V) {
#pragma unroll
                for (int e = 0; e < 8; ++e) c += (j0 + e < V) && sort_key(z[e]) == tau;
            }
            rank0 = ties_before[t] + block_sum_before(c, work_i);
        }
        float sum = 0.f;
        if (j0 < V) {
            int rank = rank0;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (j0 + e >= V) continue;
                const uint32_t key = sort_key(z[e]);
                const bool in = !cut || key > tau || (key == tau && (!ranked || rank++ < need));
                if (in) { sum += expf(z[e] - m); any = true; }
            }
        }
        return sum;
    };
    if (!filtered) {
        // The tiles' sums are there, each against its tile's own maximum: brought to the row's maximum
        // they give the tile that holds the target; within it the search goes on in the tile's own scale.
        if (tid == 0) {
            float top = -INFINITY;
            for (int t = 0; t < ntiles; ++t) top = fmaxf(top, tile_m[t]);
            float total = 0.f;
            for (int t = 0; t < ntiles; ++t) total += tile_s[t] * expf(tile_m[t] - top);
            const float want = uniform[r] * total;
            float run = 0.f;
            int pick = -1, last = 0;                 // (a tile far below the maximum has no mass at all in float32)
            for (int t = 0; t < ntiles; ++t) {
                const float w = tile_s[t] * expf(tile_m[t] - top);
                if (w > 0.f) last = t;
                if (w > 0.f && run + w >= want) { pick = t; break; }
                run += w;
            }
            const bool past = pick < 0;              // rounding left the target just above the total:
            if (past) pick = last;                   // the last id with mass (no sum reaches infinity below)
            pick_i[0] = pick;
            pick_f[0] = 0.f;
            pick_f[1] = past ? INFINITY : (want - run) / expf(tile_m[pick] - top);
            pick_f[2] = tile_m[pick];
        }
        __syncthreads();
        m = pick_f[2];
    } else {
        for (int t = 0; t < ntiles; ++t) {
            bool any;
            int rank0;
            const float ts = block_sum<SMP_NT>(mine_of(t, any, rank0), sf);
            if (tid == 0) tile_sum[t] = ts;
        }
        __syncthreads();
        if (tid == 0) {
            float total = 0.f;
            for (int t = 0; t < ntiles; ++t) total += tile_sum[t];
            const float want = uniform[r] * total;
            float run = 0.f;
            int pick = -1, last = 0;
            for (int t = 0; t < ntiles; ++t) {
                if (tile_sum[t] > 0.f) last = t;
                if (tile_sum[t] > 0.f && run + tile_sum[t] >= want) { pick = t; break; }
                run += tile_sum[t];
            }
            const bool past = pick < 0;
            if (past) pick = last;
            pick_i[0] = pick;
            pick_f[0] = past ? 0.f : run;
            pick_f[1] = past ? INFINITY : want;
        }
        __syncthreads();
    }
    tile = pick_i[0];
    before = pick_f[0];
    target = pick_f[1];
    // within the tile: the first thread whose ids bring the running sum to the target, else the last one with a survivor
    bool any;
    int rank0;
    const float mine = mine_of(tile, any, rank0);
    const float run0 = before + block_sum_before(mine, work_f);
    int chosen = block_min_int((any && run0 + mine >= target) ? tid : 0x7fffffff, si);
    if (chosen == 0x7fffffff) chosen = -block_min_int(any ? -tid : 1, si);     // (the tile has a survivor: its sum is above zero)
    if (tid == chosen) {
        const int j0 = tile * SMP_TILE + tid * 8;
        float z[8];
        load_ids8(row, j0, V, T, vec, z);
        float run = run0;
        int rank = rank0, pick = j0;
        for (int e = 0; e < 8 && j0 + e < V; ++e) {
            const uint32_t key = sort_key(z[e]);
            const bool in = !cut || key > tau || (key == tau && (!ranked || rank++ < need));
            if (!in) continue;
            pick = j0 + e;
            run += expf(z[e] - m);
            if (run >= target) break;
        }
        out[r] = pick;
    }
}

// ------------------------------------------------- sampling state of the live requests, on the device
// One row of eight 32-bit words for every state slot of the cache: {temperature, top_p (float bits), top_k,
// seed low, seed high, draws so far, 0, 0}.  The host writes a row when a request is bound to its slot and
// never again; the device counts the draws.  (The reference keeps the same per sequence on the host:
// src/llaisys/models/qwen2.hpp:100-110.)
//
// li_sample_prepare turns the rows of a step, given as slot | flags << 24 (flag 1: this row is greedy
// whatever its slot says, e.g. a request's first token), into the per-row arrays that li_sample_rows takes:
// temperature, top_k, top_p and the uniform number of the slot's next draw, the draws-th number of the
// stream `seed`: a splitmix64 hash of both, its upper 24 bits as a value in [0, 1).  A row that samples
// (temperature > 0) advances its slot's count.  A slot outside the table gives a greedy row.
#define SAMPLE_SLOT_WORDS 8
__device__ __forceinline__ float stream_uniform(unsigned long long seed, unsigned long long counter) {
    unsigned long long z = seed * 0x9E3779B97F4A7C15ull + (counter + 1ull) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

__global__ void sample_prepare_kernel(const int* __restrict__ rows, int n, int* __restrict__ table, int nslots,
                                      float* __restrict__ temperature, int* __restrict__ top_k,
                                      float* __restrict__ top_p, float* __restrict__ uniform) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int slot = rows[i] & 0xffffff, flags = (rows[i] >> 24) & 0x7f;
    float T = 0.f, P = 1.f, U = 0.f;
    int K = 0;
    if (slot < nslots && !(flags & 1)) {
        int* row = table + (size_t)slot * SAMPLE_SLOT_WORDS;
        T = __int_as_float(row[0]);
        P = __int_as_float(row[1]);
        K = row[2];
        if (T > 0.f) {
            const unsigned long long seed = (unsigned long long)(unsigned)row[3] | ((unsigned long long)(unsigned)row[4] << 32);
            const int draws = row[5];
            U = stream_uniform(seed, (unsigned long long)(unsigned)draws);
            row[5] = draws + 1;                      // (a slot stands once in a step's rows: no two threads write it)
        } else {
            T = 0.f;
        }
    }
    temperature[i] = T; top_k[i] = K; top_p[i] = P; uniform[i] = U;
}

extern "C" int li_sample_prepare(const int* rows, int n, int* table, int nslots, float* temperature, int* top_k,
                                 float* top_p, float* uniform, hipStream_t stream) {
    if (n <= 0 || nslots <= 0 || !rows || !table) return LI_ERR_SIZE;
    sample_prepare_kernel<<<(n + 255) / 256, 256, 0, stream>>>(rows, n, table, nslots, temperature, top_k, top_p, uniform);
    return li_launch_status();
}

// Floats of scratch memory that li_sample_rows needs for n rows of V logits.
extern "C" long li_sample_rows_scratch_floats(int n, int V) {
    if (n <= 0 || V <= 0) return 0;
    const long ntiles = (V + SMP_TILE - 1) / SMP_TILE;
    return (3 + 2 * (long)SMP_KC) * n * ntiles;
}

// tiles: scratch of li_sample_rows_scratch_floats(n, V) floats, in which the first kernel leaves every tile's part.
extern "C" int li_sample_rows(const float* logits, const float* temperature, const int* top_k,
                              const float* top_p, const float* uniform, int* out, int n, int V,
                              float* tiles, long tiles_floats, hipStream_t stream) {
    if (n <= 0 || n > 65535 || V <= 0) return LI_ERR_SIZE;
    const int ntiles = (V + SMP_TILE - 1) / SMP_TILE;
    if (ntiles > SMP_NT || !tiles || tiles_floats < li_sample_rows_scratch_floats(n, V)) return LI_ERR_SIZE;
    const size_t per = (size_t)n * ntiles;
    float* tm = tiles;
    float* ts = tiles + per;
    int* ti = reinterpret_cast<int*>(tiles + 2 * per);
    float* cz = tiles + 3 * per;
    int* ci = reinterpret_cast<int*>(tiles + (3 + (size_t)SMP_KC) * per);
    sample_tiles_kernel<<<dim3(ntiles, n), SMP_NT, 0, stream>>>(logits, temperature, top_k, top_p, tm, ts, ti, cz, ci, V);
    sample_rows_kernel<<<n, SMP_NT, 0, stream>>>(logits, temperature, top_k, top_p, uniform, out, V, tm, ts, ti, cz, ci, ntiles);
    return li_launch_status();
}
