// Row-wise and element-wise kernels: embedding gather, RMSNorm, row gather,
// casts, SwiGLU, rotary tables and rotation, and the write of keys and values
// into their pages.  Arithmetic is float32 throughout; bfloat16 is a storage
// format that is widened on load and rounded once on store.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = float(table[id(t), :])  (row copy, no scaling), with id(t) = ids[t], or, where
// id_src is given and id_src[t] >= 0, feedback[id_src[t]]: a token that an earlier kernel on the
// stream chose and the host has not seen yet.
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const int* __restrict__ id_src,
                                 const int* __restrict__ feedback, const T* __restrict__ table,
                                 float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id_src) {
        const int src = id_src[t];
        if (src >= 0) id = feedback[src];
    }
    float* o = out + (size_t)t * H;
    if (id < 0 || id >= V) {                       // the host has checked what it knows; never read outside:
        for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = 0.f;      // a row of zeros, not what an earlier step left
        return;
    }
    const T* row = table + (size_t)id * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) o[j] = load_as_float(row + j);
}

extern "C" int li_embedding(const int* ids, const int* id_src, const int* feedback, const void* table,
                            int table_dtype, float* out, int T, int H, int V, hipStream_t stream) {
    if (T <= 0 || H <= 0 || (id_src && !feedback)) return LI_ERR_SIZE;
    if (table_dtype == LI_F32)
        embedding_kernel<float><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const float*)table, out, H, V);
    else if (table_dtype == LI_BF16)
        embedding_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, id_src, feedback, (const bf16_t*)table, out, H, V);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ------------------------------------------------------------------ rmsnorm
// y = w * x * rsqrt(mean(x^2) + eps), eps inside the root; one block per row.  The row is
// read once and kept in registers (up to RN_PER elements a thread); longer rows are read again.
// Few rows (a decoding step): 1024 threads a row, so that the one row is read with the least
// latency; many rows (a prompt): 256 threads a row, less of a block's time goes into meeting.
template <typename TI, typename TO, int NT, int PER>
__global__ __launch_bounds__(NT) void rmsnorm_kernel(const TI* __restrict__ x, const float* __restrict__ w,
                                                      float eps, TO* __restrict__ out, int H) {
    __shared__ float red[NT / LI_WAVE];
    const TI* row = x + (size_t)blockIdx.x * H;
    TO* o = out + (size_t)blockIdx.x * H;
    float v[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        v[i] = (j < H) ? load_as_float(row + j) : 0.f;
        ss += v[i] * v[i];
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT) { const float t = load_as_float(row + j); ss += t * t; }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        if (j < H) store_from_float(o + j, w[j] * v[i] * inv);
    }
    for (int j = threadIdx.x + PER * NT; j < H; j += NT)
        store_from_float(o + j, w[j] * load_as_float(row + j) * inv);
}

// Many rows of float32 whose length is a multiple of 4 (a prompt's residual rows): 16 bytes a lane.
template <typename TO, int NT, int PER>
__global__ __launch_bounds__(NT) void rmsnorm_vec_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                          float eps, TO* __restrict__ out, int H) {
    __shared__ float red[NT / LI_WAVE];
    const float4* row = reinterpret_cast<const float4*>(x + (size_t)blockIdx.x * H);
    const float4* w4 = reinterpret_cast<const float4*>(w);
    TO* o = out + (size_t)blockIdx.x * H;
    const int n4 = H / 4;
    float4 v[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        v[i] = (j < n4) ? row[j] : float4{0.f, 0.f, 0.f, 0.f};
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int j = threadIdx.x + i * NT;
        if (j < n4) {
            const float4 g = w4[j];
            const float y0 = g.x * v[i].x * inv, y1 = g.y * v[i].y * inv, y2 = g.z * v[i].z * inv, y3 = g.w * v[i].w * inv;
            if constexpr (sizeof(TO) == 2) {
                *reinterpret_cast<uint2*>(o + 4 * j) = uint2{pack2_bf16(y0, y1), pack2_bf16(y2, y3)};
            } else {
                *reinterpret_cast<float4*>(o + 4 * j) = float4{y0, y1, y2, y3};
            }
        }
    }
}

extern "C" int li_rmsnorm(const void* x, int x_dtype, const float* w, float eps, void* out,
                          int out_dtype, int T, int H, hipStream_t stream) {
    if (T <= 0 || H <= 0) return LI_ERR_SIZE;
#define LI_NORM(TI, TO)                                                                                        \
    {                                                                                                          \
        if (T >= 256) rmsnorm_kernel<TI, TO, 256, 16><<<T, 256, 0, stream>>>((const TI*)x, w, eps, (TO*)out, H); \
        else rmsnorm_kernel<TI, TO, 1024, 8><<<T, 1024, 0, stream>>>((const TI*)x, w, eps, (TO*)out, H);        \
    }
    if (x_dtype == LI_F32 && T >= 256 && H % 4 == 0 && H <= 4 * 256 * 8 && ((uintptr_t)x | (uintptr_t)w | (uintptr_t)out) % 16 == 0) {
        if (out_dtype == LI_F32) rmsnorm_vec_kernel<float, 256, 8><<<T, 256, 0, stream>>>((const float*)x, w, eps, (float*)out, H);
        else if (out_dtype == LI_BF16) rmsnorm_vec_kernel<bf16_t, 256, 8><<<T, 256, 0, stream>>>((const float*)x, w, eps, (bf16_t*)out, H);
        else return LI_ERR_DTYPE;
        return li_launch_status();
    }
    if (x_dtype == LI_F32 && out_dtype == LI_F32) LI_NORM(float, float)
    else if (x_dtype == LI_F32 && out_dtype == LI_BF16) LI_NORM(float, bf16_t)
    else if (x_dtype == LI_BF16 && out_dtype == LI_BF16) LI_NORM(bf16_t, bf16_t)
    else if (x_dtype == LI_BF16 && out_dtype == LI_F32) LI_NORM(bf16_t, float)
    else return LI_ERR_DTYPE;
#undef LI_NORM
    return li_launch_status();
}

// -------------------------------------------------------------- gather rows
__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                   float* __restrict__ out, int H) {
    const float* src = x + (size_t)rows[blockIdx.x] * H;
    float* dst = out + (size_t)blockIdx.x * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) dst[j] = src[j];
}

extern "C" int li_gather_rows(const float* x, const int* rows, float* out, int n, int H,
                              hipStream_t stream) {
    if (n <= 0 || H <= 0) return LI_ERR_SIZE;
    gather_rows_kernel<<<n, 256, 0, stream>>>(x, rows, out, H);
    return li_launch_status();
}

// --------------------------------------------------------------------- cast
template <typename TI, typename TO>
__global__ void cast_kernel(const TI* __restrict__ src, TO* __restrict__ dst, long n) {
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        store_from_float(dst + i, load_as_float(src + i));
}

extern "C" int li_cast(const void* src, int sdt, void* dst, int ddt, long n, hipStream_t stream) {
    if (n <= 0) return LI_ERR_SIZE;
    long blocks = (n + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    if (sdt == LI_F32 && ddt == LI_BF16) cast_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>((const float*)src, (bf16_t*)dst, n);
    else if (sdt == LI_BF16 && ddt == LI_F32) cast_kernel<bf16_t, float><<<blocks, 256, 0, stream>>>((const bf16_t*)src, (float*)dst, n);
    else if (sdt == LI_F32 && ddt == LI_F32) cast_kernel<float, float><<<blocks, 256, 0, stream>>>((const float*)src, (float*)dst, n);
    else if (sdt == LI_BF16 && ddt == LI_BF16) cast_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)src, (bf16_t*)dst, n);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ------------------------------------------------------------------- swiglu
// out[t, i] = up * gate / (1 + exp(-gate)), gate = gu[t, i], up = gu[t, I + i]
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
    const T* g = gu + (size_t)blockIdx.y * 2 * I;
    T* o = out + (size_t)blockIdx.y * I;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < I) {
        const float gv = load_as_float(g + i), uv = load_as_float(g + I + i);
        store_from_float(o + i, uv * (gv / (1.0f + expf(-gv))));
    }
}

extern "C" int li_swiglu(const void* gu, void* out, int dtype, int T, int I, hipStream_t stream) {
    if (T <= 0 || I <= 0 || T > 65535 * 32) return LI_ERR_SIZE;
    // grid.y is limited to 65535: walk the rows in slabs
    for (int t0 = 0; t0 < T; t0 += 65535) {
        const int rows = (T - t0 < 65535) ? T - t0 : 65535;
        dim3 grid((I + 255) / 256, rows);
        if (dtype == LI_F32)
            swiglu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu + (size_t)t0 * 2 * I, (float*)out + (size_t)t0 * I, I);
        else if (dtype == LI_BF16)
            swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu + (size_t)t0 * 2 * I, (bf16_t*)out + (size_t)t0 * I, I);
        else return LI_ERR_DTYPE;
    }
    return li_launch_status();
}

// --------------------------------------------------------------------- rope
// angle = float(pos) / powf(theta, float(2j) / rotary_dim); cos and sin in float32
__global__ void rope_table_kernel(const int* __restrict__ pos, float theta, int rotary_dim,
                                  float* __restrict__ cosv, float* __restrict__ sinv, int T) {
    const int half = rotary_dim / 2;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (long)T * half) return;
    const int t = (int)(idx / half), j = (int)(idx % half);
    const float ang = (float)pos[t] / powf(theta, (float)(2 * j) / (float)rotary_dim);
    cosv[idx] = cosf(ang);
    sinv[idx] = sinf(ang);
}

extern "C" int li_rope_table(const int* pos, float theta, int rotary_dim, float* cosv, float* sinv,
                             int T, hipStream_t stream) {
    if (T <= 0 || rotary_dim <= 0 || (rotary_dim & 1)) return LI_ERR_SIZE;
    const long n = (long)T * (rotary_dim / 2);
    rope_table_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(pos, theta, rotary_dim, cosv, sinv, T);
    return li_launch_status();
}

// y[j] = a cos - b sin; y[j + half] = b cos + a sin with a = x[j], b = x[j + half]
// One rotation, with its roundings spelled out (one product rounded, the other fused into the sum),
// so that every kernel here gives the same bits whatever the compiler would contract.
__device__ __forceinline__ void rotate_values(float a, float b, float c, float s, float& ra, float& rb) {
    ra = __builtin_fmaf(a, c, -__fmul_rn(b, s));
    rb = __builtin_fmaf(b, c, __fmul_rn(a, s));
}

template <typename T>
__device__ __forceinline__ void rotate_pair(T* head, int j, int half, float c, float s, T* dst) {
    const float a = load_as_float(head + j), b = load_as_float(head + j + half);
    float ra, rb;
    rotate_values(a, b, c, s, ra, rb);
    store_from_float(dst + j, ra);
    store_from_float(dst + j + half, rb);
}

template <typename T>
__global__ void rope_apply_kernel(T* __restrict__ qkv, int row_stride, int head_dim, int rotary_dim,
                                  const float* __restrict__ cosv, const float* __restrict__ sinv) {
    const int t = blockIdx.x, h = blockIdx.y, half = rotary_dim / 2;
    T* head = qkv + (size_t)t * row_stride + (size_t)h * head_dim;
    for (int j = threadIdx.x; j < half; j += blockDim.x)
        rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], head);
}

extern "C" int li_rope_apply(void* qkv, int dtype, int row_stride, int n_heads, int head_dim,
                             int rotary_dim, const float* cosv, const float* sinv, int T,
                             hipStream_t stream) {
    if (T <= 0 || n_heads <= 0 || n_heads > 65535 || rotary_dim > head_dim || (rotary_dim & 1)) return LI_ERR_SIZE;
    dim3 grid(T, n_heads);
    if (dtype == LI_F32) rope_apply_kernel<float><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, head_dim, rotary_dim, cosv, sinv);
    else if (dtype == LI_BF16) rope_apply_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, head_dim, rotary_dim, cosv, sinv);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// ----------------------------------------------------------------- kv store
// Cache layout per layer: [pages, kv_heads, page_size, head_dim]; the slot of
// a token is page * page_size + offset.
template <typename T>
__device__ __forceinline__ T* cache_row(T* base, int slot, int page_size, int nkv, int kvh, int dh) {
    const int page = slot / page_size, off = slot - page * page_size;
    return base + (((size_t)page * nkv + kvh) * page_size + off) * dh;
}

// grid (T, nh + 2 nkv) when ROTATE (query heads rotated in place, key heads
// rotated into the cache, value heads copied), grid (T, 2 nkv) otherwise
template <typename T, bool ROTATE>
__global__ void kv_store_kernel(T* __restrict__ qkv, int row_stride, int nh, int nkv, int dh,
                                int rotary_dim, const float* __restrict__ cosv,
                                const float* __restrict__ sinv, const int* __restrict__ slot_map,
                                T* __restrict__ kc, T* __restrict__ vc, int page_size, int num_pages) {
    const int t = blockIdx.x;
    int hh = blockIdx.y + (ROTATE ? 0 : nh);
    T* head = qkv + (size_t)t * row_stride + (size_t)hh * dh;
    const int half = rotary_dim / 2;
    if (hh < nh) {                                               // query head: rotate in place
        for (int j = threadIdx.x; j < half; j += blockDim.x)
            rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], head);
        return;
    }
    const int slot = slot_map[t];
    if (slot < 0 || slot >= num_pages * page_size) return;       // never write outside the pool
    if (hh < nh + nkv) {
        T* dst = cache_row(kc, slot, page_size, nkv, hh - nh, dh);
        if (ROTATE) {
            for (int j = threadIdx.x; j < half; j += blockDim.x)
                rotate_pair(head, j, half, cosv[(size_t)t * half + j], sinv[(size_t)t * half + j], dst);
            for (int j = rotary_dim + threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
        } else {
            for (int j = threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
        }
    } else {
        T* dst = cache_row(vc, slot, page_size, nkv, hh - nh - nkv, dh);
        for (int j = threadIdx.x; j < dh; j += blockDim.x) dst[j] = head[j];
    }
}

// The same with 16 bytes a lane, for whole-head rotation (rotary_dim == dh) or none, where a half
// head is a whole number of 16-byte pieces and rows start on 16 bytes: thread (t, head, c) takes
// the pieces c of the head's two halves, i.e. E pairs when it rotates.
template <typename T, bool ROTATE>
__global__ __launch_bounds__(256) void kv_store_vec_kernel(T* __restrict__ qkv, int row_stride, int nh, int nkv, int dh,
                                                            const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                            const int* __restrict__ slot_map, T* __restrict__ kc,
                                                            T* __restrict__ vc, int page_size, int num_pages, long total) {
    constexpr int E = 16 / (int)sizeof(T);
    struct __attribute__((aligned(16))) piece { T e[E]; };
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int half = dh / 2, cph = half / E;                     // pieces in half a head
    const int nheads = ROTATE ? nh + 2 * nkv : 2 * nkv;
    const int c = (int)(i % cph);
    const int hh = (int)((i / cph) % nheads) + (ROTATE ? 0 : nh);
    const int t = (int)(i / ((long)cph * nheads));
    T* head = qkv + (size_t)t * row_stride + (size_t)hh * dh;
    T* dst = head;                                               // query heads: rotated in place
    if (hh >= nh) {
        const int slot = slot_map[t];
        if (slot < 0 || slot >= num_pages * page_size) return;   // never write outside the pool
        dst = hh < nh + nkv ? cache_row(kc, slot, page_size, nkv, hh - nh, dh)
                            : cache_row(vc, slot, page_size, nkv, hh - nh - nkv, dh);
    }
    piece a = *reinterpret_cast<const piece*>(head + E * c), b = *reinterpret_cast<const piece*>(head + half + E * c);
    if (ROTATE && hh < nh + nkv) {
        const float* cs = cosv + (size_t)t * half + E * c;
        const float* sn = sinv + (size_t)t * half + E * c;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float ra, rb;
            rotate_values(load_as_float(&a.e[e]), load_as_float(&b.e[e]), cs[e], sn[e], ra, rb);
            store_from_float(&a.e[e], ra);
            store_from_float(&b.e[e], rb);
        }
    } else if (dst == head) {
        return;                                                  // (cannot happen: an unrotated head is a cache head)
    }
    *reinterpret_cast<piece*>(dst + E * c) = a;
    *reinterpret_cast<piece*>(dst + half + E * c) = b;
}

template <typename T, bool ROTATE>
static bool kv_store_vec(T* qkv, int row_stride, int nh, int nkv, int dh, int rotary_dim, const float* cosv,
                         const float* sinv, const int* slot_map, T* kc, T* vc, int page_size, int num_pages, int Tn,
                         hipStream_t stream) {
    constexpr int E = 16 / (int)sizeof(T);
    if ((ROTATE && rotary_dim != dh) || dh % (2 * E) || row_stride % E || ((uintptr_t)qkv | (uintptr_t)kc | (uintptr_t)vc) % 16 ||
        (ROTATE && (((uintptr_t)cosv | (uintptr_t)sinv) % 16)))
        return false;
    const long total = (long)Tn * (ROTATE ? nh + 2 * nkv : 2 * nkv) * (dh / 2 / E);
    const long blocks = (total + 255) / 256;
    if (blocks > 0x7fffffffL) return false;
    kv_store_vec_kernel<T, ROTATE><<<(unsigned)blocks, 256, 0, stream>>>(qkv, row_stride, nh, nkv, dh, cosv, sinv, slot_map, kc, vc,
                                                                        page_size, num_pages, total);
    return true;
}

extern "C" int li_kv_store(void* qkv, int dtype, int row_stride, int nh, int nkv, int dh,
                           const int* slot_map, void* kc, void* vc, int page_size, int num_pages,
                           int T, hipStream_t stream) {
    if (T <= 0 || nkv <= 0 || 2 * nkv > 65535 || page_size <= 0) return LI_ERR_SIZE;
    dim3 grid(T, 2 * nkv);
    if (dtype == LI_F32 && kv_store_vec<float, false>((float*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (float*)kc, (float*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_BF16 && kv_store_vec<bf16_t, false>((bf16_t*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_F32) kv_store_kernel<float, false><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (float*)kc, (float*)vc, page_size, num_pages);
    else if (dtype == LI_BF16) kv_store_kernel<bf16_t, false><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, nh, nkv, dh, 0, nullptr, nullptr, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

extern "C" int li_rope_kv_store(void* qkv, int dtype, int row_stride, int nh, int nkv, int dh,
                                int rotary_dim, const float* cosv, const float* sinv,
                                const int* slot_map, void* kc, void* vc, int page_size,
                                int num_pages, int T, hipStream_t stream) {
    if (T <= 0 || nh + 2 * nkv > 65535 || page_size <= 0 || rotary_dim > dh || (rotary_dim & 1)) return LI_ERR_SIZE;
    dim3 grid(T, nh + 2 * nkv);
    if (dtype == LI_F32 && kv_store_vec<float, true>((float*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (float*)kc, (float*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_BF16 && kv_store_vec<bf16_t, true>((bf16_t*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages, T, stream)) return li_launch_status();
    if (dtype == LI_F32) kv_store_kernel<float, true><<<grid, 64, 0, stream>>>((float*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (float*)kc, (float*)vc, page_size, num_pages);
    else if (dtype == LI_BF16) kv_store_kernel<bf16_t, true><<<grid, 64, 0, stream>>>((bf16_t*)qkv, row_stride, nh, nkv, dh, rotary_dim, cosv, sinv, slot_map, (bf16_t*)kc, (bf16_t*)vc, page_size, num_pages);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}
