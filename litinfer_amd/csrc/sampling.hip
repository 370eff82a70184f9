// Choosing the next token from float32 logits: argmax (lowest index on ties)
// and temperature / top-k / top-p sampling by inverse CDF with a uniform
// number that the host derives from the request's own counter-based stream.
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
// One block per row.  The candidates are ordered by (value descending, index
// ascending); top-k keeps the first k, top-p then the shortest prefix whose
// softmax mass (among the top-k survivors) reaches p; the survivors' softmax is
// sampled by inverse CDF over ASCENDING ids with the given uniform number.
// Thresholds are found by a bitwise search over the order-preserving integer
// image of the floats, every count and mass being a block reduction in a fixed
// order, so the same inputs always give the same token.
__device__ __forceinline__ uint32_t sort_key(float z) {
    const uint32_t b = __float_as_uint(z);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

__device__ __forceinline__ int block_sum_int(int v, int* smem) {
#pragma unroll
    for (int o = LI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LI_WAVE);
    const int lane = threadIdx.x & (LI_WAVE - 1), w = threadIdx.x / LI_WAVE;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    int t = 0;
#pragma unroll
    for (int i = 0; i < SMP_NT / LI_WAVE; ++i) t += smem[i];
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
    for (int i = 1; i < SMP_NT / LI_WAVE; ++i) t = fmaxf(t, smem[i]);
    return t;
}

__global__ __launch_bounds__(SMP_NT) void sample_rows_kernel(
    const float* __restrict__ logits, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p,
    const float* __restrict__ uniform, int* __restrict__ out, int V) {
    __shared__ float sf[SMP_NT / LI_WAVE];
    __shared__ int si[SMP_NT / LI_WAVE];
    __shared__ float part_f[SMP_NT];
    __shared__ int part_i[SMP_NT];
    __shared__ int chosen_thread;
    const int r = blockIdx.x, tid = threadIdx.x;
    const float* row = logits + (size_t)r * V;
    const float T = temperature[r];
    if (!(T > 0.f)) {                                          // greedy
        float v = -INFINITY;
        int i = 0x7fffffff;
        for (int j = tid; j < V; j += SMP_NT) {
            const float x = row[j];
            if (x > v || i == 0x7fffffff) { v = x; i = j; }
        }
        block_argmax(v, i, sf, si);
        if (tid == 0) out[r] = i;
        return;
    }
    {
        // Temperature alone (no top-k, no top-p: every id survives), the common case: no thresholds
        // to search for and no ties to count, so the row is read three times in whole lines.
        // Ids are taken in tiles of SMP_NT * 8: thread t holds the 8 consecutive ids t * 8 .. of a
        // tile.  The inverse CDF runs over ascending ids: tile by tile (sums of whole tiles, each a
        // block sum in its fixed order), then thread by thread within the tile that holds the
        // target, then id by id within that thread.
        const int kk = top_k[r];
        const float pp = top_p[r];
        constexpr int TILE = SMP_NT * 8;
        const int ntiles = (V + TILE - 1) / TILE;
        if (!(kk > 0 && kk < V) && !(pp > 0.f && pp < 1.f) && ntiles <= SMP_NT) {
            float m = -INFINITY;
            for (int j = tid; j < V; j += SMP_NT) m = fmaxf(m, row[j] / T);
            m = block_max_f(m, sf);
            auto mine_of = [&](int tile) {               // this thread's 8 ids of a tile, in id order
                const int j0 = tile * TILE + tid * 8;
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) s += (j0 + e < V) ? expf(row[j0 + e] / T - m) : 0.f;
                return s;
            };
            for (int tile = 0; tile < ntiles; ++tile) {
                const float ts = block_sum<SMP_NT>(mine_of(tile), sf);
                if (tid == 0) part_f[tile] = ts;         // (ntiles <= SMP_NT places)
            }
            __syncthreads();
            if (tid == 0) {
                float total = 0.f;
                for (int t = 0; t < ntiles; ++t) total += part_f[t];
                const float target = uniform[r] * total;
                float run = 0.f;
                int pick = ntiles - 1;                   // rounding may leave the target just above the total
                for (int t = 0; t < ntiles; ++t) {
                    if (run + part_f[t] >= target) { pick = t; break; }
                    run += part_f[t];
                }
                si[0] = pick;
                sf[0] = run;
                sf[1] = target;
            }
            __syncthreads();
            const int tile = si[0];
            const float before_tile = sf[0], target = sf[1];
            __syncthreads();
            part_f[tid] = mine_of(tile);
            __syncthreads();
            if (tid == 0) {
                float run = before_tile;
                int pick = -1, last = 0;
                for (int t = 0; t < SMP_NT; ++t) {
                    if (tile * TILE + t * 8 < V) last = t;
                    if (pick < 0 && tile * TILE + t * 8 < V && run + part_f[t] >= target) pick = t;
                    if (pick < 0) run += part_f[t];
                }
                if (pick < 0) { pick = last; run -= part_f[last]; }
                chosen_thread = pick;
                sf[0] = run;
            }
            __syncthreads();
            if (tid == chosen_thread) {
                float run = sf[0];
                const int j0 = tile * TILE + tid * 8;
                int pick = j0;
                for (int e = 0; e < 8 && j0 + e < V; ++e) {
                    pick = j0 + e;
                    run += expf(row[j0 + e] / T - m);
                    if (run >= target) break;
                }
                out[r] = pick;
            }
            return;
        }
    }
    // contiguous chunk of ids per thread, so that block scans run in id order
    const int chunk = (V + SMP_NT - 1) / SMP_NT;
    const int c0 = min(tid * chunk, V), c1 = min(c0 + chunk, V);

    float m = -INFINITY;
    for (int j = c0; j < c1; ++j) m = fmaxf(m, row[j] / T);
    m = block_max_f(m, sf);

    // ---- top-k: tau_k = k-th largest key, need_k = how many of its ties count
    uint32_t tau = 0u;
    int need = 0x7fffffff;
    const int k = top_k[r];
    if (k > 0 && k < V) {
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tau | (1u << bit);
            int c = 0;
            for (int j = c0; j < c1; ++j) c += sort_key(row[j] / T) >= cand;
            if (block_sum_int(c, si) >= k) tau = cand;
        }
        int c = 0;
        for (int j = c0; j < c1; ++j) c += sort_key(row[j] / T) > tau;
        need = k - block_sum_int(c, si);
    }
    // ---- top-p among the top-k survivors
    const float p = top_p[r];
    if (p > 0.f && p < 1.f) {
        // Z_k: mass of the top-k survivors (ties at tau in id order, `need` of them)
        int eq = 0;
        for (int j = c0; j < c1; ++j) eq += sort_key(row[j] / T) == tau;
        part_i[tid] = eq;
        __syncthreads();
        int before = 0;
        for (int t = 0; t < tid; ++t) before += part_i[t];
        float zk = 0.f;
        {
            int rank = before;
            for (int j = c0; j < c1; ++j) {
                const float z = row[j] / T;
                const uint32_t key = sort_key(z);
                if (key > tau || (key == tau && rank++ < need)) zk += expf(z - m);
            }
        }
        zk = block_sum<SMP_NT>(zk, sf);
        const float target = p * zk;
        // tp = the largest c with f(c) >= target, where f(c) = Z_k for c <= tau (the top-k
        // survivors as a whole) and the mass of the keys >= c above it; f does not increase
        uint32_t tp = 0u;
        for (int bit = 31; bit >= 0; --bit) {
            const uint32_t cand = tp | (1u << bit);
            if (cand <= tau) { tp = cand; continue; }
            float s = 0.f;
            for (int j = c0; j < c1; ++j) {
                const float z = row[j] / T;
                if (sort_key(z) >= cand) s += expf(z - m);
            }
            if (block_sum<SMP_NT>(s, sf) >= target) tp = cand;
        }
        float s = 0.f;
        for (int j = c0; j < c1; ++j) {
            const float z = row[j] / T;
            if (sort_key(z) > tp) s += expf(z - m);
        }
        const float mass_gt = block_sum<SMP_NT>(s, sf);
        const float e_tau = expf(key_value(tp) - m);
        int need_p = 0x7fffffff;                               // ties without mass: all of them
        if (e_tau > 0.f) {
            const float q = ceilf((target - mass_gt) / e_tau);
            need_p = q < 1.f ? 1 : (q > 2.0e9f ? 0x7fffffff : (int)q);
        }
        need = (tp == tau) ? min(need, need_p) : need_p;
        tau = tp;
    }
    // ---- inverse CDF over ascending ids among the survivors
    int eq = 0;
    for (int j = c0; j < c1; ++j) eq += sort_key(row[j] / T) == tau;
    __syncthreads();
    part_i[tid] = eq;
    __syncthreads();
    int before = 0;
    for (int t = 0; t < tid; ++t) before += part_i[t];
    __syncthreads();                 // part_i is written again below
    float mine = 0.f;
    int last_in = -1;
    {
        int rank = before;
        for (int j = c0; j < c1; ++j) {
            const float z = row[j] / T;
            const uint32_t key = sort_key(z);
            if (key > tau || (key == tau && rank++ < need)) { mine += expf(z - m); last_in = j; }
        }
    }
    part_f[tid] = mine;
    part_i[tid] = last_in;           // (the tie counts are no longer needed: `before` is in a register)
    if (tid == 0) chosen_thread = -1;
    __syncthreads();
    if (tid == 0) {                  // sequential scan in id order: 1024 additions, fixed order
        float total = 0.f;
        for (int t = 0; t < SMP_NT; ++t) total += part_f[t];
        const float target = uniform[r] * total;
        float run = 0.f;
        int pick = -1, last_nonempty = -1;
        for (int t = 0; t < SMP_NT; ++t) {
            if (part_i[t] >= 0) last_nonempty = t;
            if (pick < 0 && part_i[t] >= 0 && run + part_f[t] >= target) pick = t;
            if (pick < 0) run += part_f[t];
        }
        if (pick < 0) pick = last_nonempty;               // rounding left the target just above the total
        chosen_thread = pick;
        sf[0] = run;                                       // mass before the chosen thread's chunk
        sf[1] = target;
    }
    __syncthreads();
    if (tid == chosen_thread) {
        float run = sf[0];
        const float target = sf[1];
        int rank = before, pick = last_in;
        for (int j = c0; j < c1; ++j) {
            const float z = row[j] / T;
            const uint32_t key = sort_key(z);
            if (key > tau || (key == tau && rank++ < need)) {
                run += expf(z - m);
                if (run >= target) { pick = j; break; }
            }
        }
        out[r] = pick;
    }
}

extern "C" int li_sample_rows(const float* logits, const float* temperature, const int* top_k,
                              const float* top_p, const float* uniform, int* out, int n, int V,
                              hipStream_t stream) {
    if (n <= 0 || V <= 0) return LI_ERR_SIZE;
    sample_rows_kernel<<<n, SMP_NT, 0, stream>>>(logits, temperature, top_k, top_p, uniform, out, V);
    return li_launch_status();
}
