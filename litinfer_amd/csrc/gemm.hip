// out[M, N] = x[M, K] w[N, K]^T (+ bias[N]) (+ out), float32 accumulation.
//
// float32 operands: an LDS-tiled FMA kernel (true 32-bit, no reduced-precision
// matrix mode).  bfloat16 operands: MFMA tiles for 64-wide waves.  For each
// output element the sum over K runs in an order that depends on K alone, not
// on M or on the element's place, so a row's result does not depend on which
// other rows are in the batch.
#include "common.h"
#include <algorithm>
#include <type_traits>
#include <utility>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <typename TO>
__device__ __forceinline__ void epilogue_store(TO* out, size_t idx, float acc, const float* bias,
                                               int col, bool accumulate) {
    if (bias) acc += bias[col];
    if (accumulate) acc += load_as_float(out + idx);
    store_from_float(out + idx, acc);
}

// ------------------------------------------------------------ float32 tiles
// 64 x 64 tile per block of 256 threads, 4 x 4 outputs per thread, K in steps of 16.
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ x,
                                                        const float* __restrict__ w,
                                                        const float* __restrict__ bias,
                                                        float* __restrict__ out, int M, int N, int K,
                                                        int accumulate) {
    __shared__ float As[F32_BK][F32_BM + 4];
    __shared__ float Bs[F32_BK][F32_BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
    const int ty = tid / 16, tx = tid % 16;
    const int lrow = tid / 4, lk = (tid % 4) * 4;            // this thread's 4 consecutive k of one row
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += F32_BK) {
        float a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = k0 + lk + i;
            a[i] = (m0 + lrow < M && k < K) ? x[(size_t)(m0 + lrow) * K + k] : 0.f;
            b[i] = (n0 + lrow < N && k < K) ? w[(size_t)(n0 + lrow) * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) { As[lk + i][lrow] = a[i]; Bs[lk + i][lrow] = b[i]; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < F32_BK; ++k) {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { av[i] = As[k][ty * 4 + i]; bv[i] = Bs[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = m0 + ty * 4 + i;
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + tx * 4 + j;
            if (col < N) epilogue_store(out, (size_t)row * N + col, acc[i][j], bias, col, accumulate);
        }
    }
}

// The same product in tiles of 128 x 128 with 8 x 8 outputs a thread, for many rows and columns:
// a step reads 16 floats from LDS for 64 multiply-adds (the small tile reads 8 for 16), so the
// FMA units and not LDS bound it.  Every output element still adds its products up in ascending
// k, one fused multiply-add after the other: the results are those of the small tile bit for bit.
#define F32B_BM 128
#define F32B_BN 128
#define F32B_BK 8

__global__ __launch_bounds__(256) void gemm_f32_big_kernel(const float* __restrict__ x,
                                                            const float* __restrict__ w,
                                                            const float* __restrict__ bias,
                                                            float* __restrict__ out, int M, int N, int K,
                                                            int accumulate) {
    __shared__ __attribute__((aligned(16))) float As[2][F32B_BK][F32B_BM + 4];
    __shared__ __attribute__((aligned(16))) float Bs[2][F32B_BK][F32B_BN + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * F32B_BM, n0 = blockIdx.x * F32B_BN;
    const int ty = tid / 16, tx = tid % 16;                  // outputs rows 4 ty .. +3 and 64 + 4 ty .., columns likewise
    const int lrow = tid / 2, lk = (tid % 2) * 4;            // this thread's 4 consecutive k of one row of each operand
    const bool vec = (K % 4) == 0;
    const float* arow = x + (size_t)(m0 + lrow < M ? m0 + lrow : M - 1) * K;
    const float* brow = w + (size_t)(n0 + lrow < N ? n0 + lrow : N - 1) * K;
    float acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
    float a[4], b[4];
    auto fetch = [&](int k0) {
        if (vec && k0 + lk + 4 <= K) {
            const floatx4 av = *reinterpret_cast<const floatx4*>(arow + k0 + lk);
            const floatx4 bv = *reinterpret_cast<const floatx4*>(brow + k0 + lk);
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = av[i]; b[i] = bv[i]; }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = k0 + lk + i;
                a[i] = k < K ? arow[k] : 0.f;
                b[i] = k < K ? brow[k] : 0.f;
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) { As[buf][lk + i][lrow] = a[i]; Bs[buf][lk + i][lrow] = b[i]; }
    };
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += F32B_BK) {
        const bool more = k0 + F32B_BK < K;
        if (more) fetch(k0 + F32B_BK);                       // on its way while this step is multiplied
#pragma unroll
        for (int k = 0; k < F32B_BK; ++k) {
            const floatx4 a0 = *reinterpret_cast<const floatx4*>(&As[buf][k][4 * ty]);
            const floatx4 a1 = *reinterpret_cast<const floatx4*>(&As[buf][k][64 + 4 * ty]);
            const floatx4 b0 = *reinterpret_cast<const floatx4*>(&Bs[buf][k][4 * tx]);
            const floatx4 b1 = *reinterpret_cast<const floatx4*>(&Bs[buf][k][64 + 4 * tx]);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float av = i < 4 ? a0[i] : a1[i - 4];
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(av, j < 4 ? b0[j] : b1[j - 4], acc[i][j]);
            }
        }
        if (more) {
            stash(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int row = m0 + (i < 4 ? 4 * ty + i : 64 + 4 * ty + i - 4);
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int col = n0 + (j < 4 ? 4 * tx + j : 64 + 4 * tx + j - 4);
            if (col < N) epilogue_store(out, (size_t)row * N + col, acc[i][j], bias, col, accumulate);
        }
    }
}

// ------------------------------------------------------ float32 on the matrix cores
// v_mfma_f32_32x32x2_f32 multiplies and adds in float32 (no operand is rounded to a shorter format: this
// is not one of the reduced-precision matrix modes), at twice the rate of the vector ALU's FMA and without
// the operands' way through registers that an 8 x 8 tile a lane needs.  Block tile 128 x 128, four waves
// two by two, each 64 x 64 = 2 x 2 MFMA tiles; K in steps of 16 (eight MFMAs of two k-values a tile).
// A stage holds x and w transposed, [k][row] with rows of 128 + 4 floats: lane (row, k) of an MFMA operand
// reads consecutive words, and the transposing writes of the 16-byte global loads (lane = row / k-quarter)
// meet no bank twice.  Two stages: the next step's global loads are in registers while this step is
// multiplied.  K a multiple of 4; rows and columns past the end repeat the last and are not stored.
#define F32M_BM 128
#define F32M_BN 128
#define F32M_BK 16
#define F32M_LD (F32M_BM + 4)
__global__ __launch_bounds__(256) void gemm_f32_mfma_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                             const float* __restrict__ bias, float* __restrict__ out,
                                                             int M, int N, int K, int accumulate) {
    __shared__ float As[2][F32M_BK * F32M_LD];
    __shared__ float Bs[2][F32M_BK * F32M_LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * F32M_BM, n0 = blockIdx.x * F32M_BN;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    // global loads: thread t takes the k-quarter t % 4 of rows t / 4 and t / 4 + 64 of both tiles
    const int lrow = tid >> 2, lkq = tid & 3;
    const float* xa[2];
    const float* wb[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int ra = m0 + lrow + 64 * h, rb = n0 + lrow + 64 * h;
        xa[h] = x + (size_t)(ra < M ? ra : M - 1) * K + 4 * lkq;
        wb[h] = w + (size_t)(rb < N ? rb : N - 1) * K + 4 * lkq;
    }
    floatx4 ga[2], gb[2];
    // WHOLE: the step's 16 k-values lie inside K; nothing is then chosen or replaced (a value chosen between what
    // was loaded and zero is waited for at once: the loads of the next step then did not run under this step's MFMAs)
    auto fetch = [&](int k0, auto whole_tag) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
        const bool ok = WHOLE || k0 + 4 * lkq < K;         // (K % 4 == 0: a 16-byte piece is inside the row or past its end)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            ga[h] = *reinterpret_cast<const floatx4*>(xa[h] + (ok ? k0 : 0));
            gb[h] = *reinterpret_cast<const floatx4*>(wb[h] + (ok ? k0 : 0));
            if constexpr (!WHOLE) { if (!ok) { ga[h] = floatx4{0.f, 0.f, 0.f, 0.f}; gb[h] = floatx4{0.f, 0.f, 0.f, 0.f}; } }
        }
    };
    auto stash = [&](int st) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                As[st][(4 * lkq + e) * F32M_LD + lrow + 64 * h] = ga[h][e];
                Bs[st][(4 * lkq + e) * F32M_LD + lrow + 64 * h] = gb[h][e];
            }
    };
    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int frow = lane & 31, fk = lane >> 5;
    auto multiply = [&](int st) {
#pragma unroll
        for (int s2 = 0; s2 < F32M_BK / 2; ++s2) {
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = As[st][(2 * s2 + fk) * F32M_LD + wm + 32 * i + frow];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = Bs[st][(2 * s2 + fk) * F32M_LD + wn + 32 * j + frow];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    };
    if (K >= F32M_BK) fetch(0, std::true_type{}); else fetch(0, std::false_type{});
    stash(0);
    __syncthreads();
    int st = 0, k0 = 0;
    // while the step after this one is whole, its loads are neither conditional nor chosen from ...
    for (; k0 + 2 * F32M_BK <= K; k0 += F32M_BK) {
        fetch(k0 + F32M_BK, std::true_type{});
        __builtin_amdgcn_sched_barrier(0);                 // (left to itself the compiler moves the loads down to where their values are stored)
        multiply(st);
        stash(st ^ 1);                                     // (the other stage: its readers passed the barrier a step ago)
        __syncthreads();
        st ^= 1;
    }
    // ... then the last whole step and, where K is no multiple of the step, the one behind it
    for (; k0 < K; k0 += F32M_BK) {
        const bool more = k0 + F32M_BK < K;
        if (more) fetch(k0 + F32M_BK, std::false_type{});
        multiply(st);
        if (more) stash(st ^ 1);
        __syncthreads();
        st ^= 1;
    }
    // register r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4, column l % 32 of a 32 x 32 tile
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn + 32 * j + frow;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm + 32 * i + 8 * (r >> 2) + 4 * fk + (r & 3);
                if (row < M && col < N) epilogue_store(out, (size_t)row * N + col, acc[i][j][r], bias, col, accumulate != 0);
            }
        }
}

// ------------------------------------------------------ float32, few rows (decode)
// The product streams w once, on the matrix cores in float32 (v_mfma_f32_16x16x4_f32: operands, products and sums
// are float32, nothing is rounded to a shorter format).  A block owns up to 16 columns a tile and 16 rows a tile;
// its eight waves split K in pieces of 32 k-values (a row's whole 128-byte line), wave v taking the pieces
// v, v + 8, ...  Lane (c, q) = (lane % 16, lane / 16) loads the four values k0 + 4 q .. + 3 of column c of w
// and of row c of x with one 16-byte load each; the MFMA e of a piece multiplies the e-th of them, i.e. its
// four k-slots are the k-values k0 + e, k0 + 4 + e, k0 + 8 + e, k0 + 12 + e (the order within a piece does
// not matter for a sum; it is the same for every row and column).  No vector arithmetic and few registers,
// so a wave keeps many loads in flight: the FMA form held 8 x 8 sums a lane and one piece in flight, and
// streamed w at 3.2 TB/s.  The eight waves' sums are added in wave order: an order that depends on K alone.
#define F32RM_WAVES 8
template <int AHEAD, int TILES, int RT, bool SWIGLU>
__global__ __launch_bounds__(F32RM_WAVES * 64) void gemm_f32_rows_mfma_kernel(const float* __restrict__ x,
                                                                              const float* __restrict__ w,
                                                                              const float* __restrict__ bias,
                                                                              float* __restrict__ out, int M, int N, int K,
                                                                              int accumulate, int cols) {
    // TILES: MFMA tiles of 16 columns side by side in a block (`cols` <= 16 TILES): they share the block's
    // loads of x, which come through the same path as w (a matrix of many columns has blocks enough).
    // RT: tiles of 16 rows one above the other (M <= 16 RT): they share the block's loads of w, which is
    // read from memory once whatever the rows.
    // SWIGLU: w is [gate; up] of N rows each, the tiles come in pairs (the gate columns n0 + 16 p .. and the
    // up columns of the same outputs), `cols` <= 8 TILES outputs a block, and out [M, N] gets
    // up * gate / (1 + exp(-gate)) from the float32 sums: the 2 N columns never go to memory.
    static_assert(!SWIGLU || TILES % 2 == 0, "gate and up tiles in pairs");
    __shared__ float part[F32RM_WAVES][RT * TILES * 256];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // (the same for a wave's lanes: its branches are scalar)
    const int c = lane & 15, q = lane >> 4;
    const int n0 = blockIdx.x * cols;
    const int nend = n0 + cols < N ? n0 + cols : N;
    const float* wrow[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const int col = SWIGLU ? n0 + 16 * (t / 2) + c : n0 + 16 * t + c;
        wrow[t] = w + ((size_t)(col < nend ? col : nend - 1) + (SWIGLU && (t & 1) ? (size_t)N : 0)) * K + 4 * q;
    }
    const float* xrow[RT];
#pragma unroll
    for (int i = 0; i < RT; ++i) xrow[i] = x + (size_t)(16 * i + c < M ? 16 * i + c : M - 1) * K + 4 * q;
    floatx4 acc[RT][TILES][2];                                // two chains of MFMAs a tile (each waits for its own last result only)
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int t = 0; t < TILES; ++t) acc[i][t][0] = acc[i][t][1] = floatx4{0.f, 0.f, 0.f, 0.f};
    const int last = K - 4;                                   // (K is a multiple of 4: the last whole 16-byte piece of a row)
    // A trip is AHEAD pieces of 32 k-values a wave: all their loads at once, never conditional (a piece past
    // the end reads the row's last 16 bytes and multiplies by zero); the next trip's loads are issued before
    // this trip is multiplied, into the other set of registers.  (Loads that pass the caches by, `nontemporal`,
    // were 10 % slower here, as for the bfloat16 products.)
    floatx4 wv[2][AHEAD][2][TILES], xv[2][AHEAD][2][RT];
    constexpr int PIECE = 32 * F32RM_WAVES, TRIP = PIECE * AHEAD;
    // WHOLE: every piece of the trip lies inside K; nothing is then chosen or replaced (a value chosen between what
    // was loaded and zero is waited for at once, and so is the next use of any load behind a conditional one).
    auto fetch = [&](int buf, int k0, auto whole_tag) {
        constexpr bool WHOLE = decltype(whole_tag)::value;
#pragma unroll
        for (int a = 0; a < AHEAD; ++a)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int k = k0 + PIECE * a + 16 * u;                    // + 4 q is in the row pointers
                const bool ok = WHOLE || k + 4 * q < K;
                const int at = ok ? k : last - 4 * q;
#pragma unroll
                for (int t = 0; t < TILES; ++t) wv[buf][a][u][t] = *reinterpret_cast<const floatx4*>(wrow[t] + at);
#pragma unroll
                for (int i = 0; i < RT; ++i) {
                    xv[buf][a][u][i] = *reinterpret_cast<const floatx4*>(xrow[i] + at);
                    if constexpr (!WHOLE) { if (!ok) xv[buf][a][u][i] = floatx4{0.f, 0.f, 0.f, 0.f}; }
                }
            }
    };
    auto whole = [&](int k0) { return k0 + PIECE * (AHEAD - 1) + 32 <= K; };    // (the same for a wave's lanes)
    auto fetch_any = [&](int buf, int k0) {
        if (whole(k0)) fetch(buf, k0, std::true_type{}); else fetch(buf, k0, std::false_type{});
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int a = 0; a < AHEAD; ++a)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < RT; ++i)
#pragma unroll
                        for (int t = 0; t < TILES; ++t)
                            acc[i][t][e & 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[buf][a][u][i][e], wv[buf][a][u][t][e],
                                                                                    acc[i][t][e & 1], 0, 0, 0);
    };
    int k0 = 32 * wave;
    if (k0 < K) fetch_any(0, k0);
    // while the two trips after this one are whole, nothing about the loads is conditional (where a path with
    // loads and one without meet, the compiler's count of the loads in flight is the smaller one, and the
    // next wait is for all of them) ...
    for (; whole(k0 + 2 * TRIP); k0 += 2 * TRIP) {
        fetch(1, k0 + TRIP, std::true_type{});
        multiply(0);
        fetch(0, k0 + 2 * TRIP, std::true_type{});
        multiply(1);
    }
    // ... and the trips that are left
    for (; k0 < K; k0 += 2 * TRIP) {
        if (k0 + TRIP < K) fetch_any(1, k0 + TRIP);
        multiply(0);
        if (k0 + TRIP >= K) break;
        if (k0 + 2 * TRIP < K) fetch_any(0, k0 + 2 * TRIP);
        multiply(1);
    }
    // acc[i][t][.][r] = the sum for row 16 i + 4 q + r, column c of tile t, of this wave's share of K (its even and
    // its odd k-values)
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) part[wave][256 * (TILES * i + t) + (4 * q + r) * 16 + c] = acc[i][t][0][r] + acc[i][t][1][r];
    __syncthreads();
    constexpr int OT = SWIGLU ? TILES / 2 : TILES;            // tiles of outputs
    for (int e = threadIdx.x; e < RT * OT * 256; e += F32RM_WAVES * 64) {
        const int i = e / (OT * 256), t = (e >> 8) % OT, row = 16 * i + ((e >> 4) & 15), j = 16 * t + (e & 15);
        if (row >= M || n0 + j >= nend) continue;
        const int at = 256 * (TILES * i + (SWIGLU ? 2 * t : t)) + (e & 255);
        float v = part[0][at];
#pragma unroll
        for (int v2 = 1; v2 < F32RM_WAVES; ++v2) v += part[v2][at];
        if constexpr (SWIGLU) {
            float up = part[0][at + 256];
#pragma unroll
            for (int v2 = 1; v2 < F32RM_WAVES; ++v2) up += part[v2][at + 256];
            out[(size_t)row * N + n0 + j] = up * (v / (1.0f + expf(-v)));
        } else {
            epilogue_store(out, (size_t)row * N + n0 + j, v, bias, n0 + j, accumulate != 0);
        }
    }
}

#define F32_ROWS_MAX 64          // up to this many rows the row kernel is taken (K a multiple of 4)

static int compute_units();

// swiglu: w is [gate; up] of N rows each and out [M, N] gets the activation (no bias, no accumulation)
static int launch_f32_rows(const float* x, const float* w, const float* bias, float* out, int M, int N, int K,
                           int accumulate, hipStream_t stream, bool swiglu = false) {
    // as many blocks as a whole number of rounds over the compute units, each with the same share of the columns;
    // two MFMA tiles side by side where 16 columns a block would not fit one round (they share the loads of x:
    // the 7B's gate/up matrix at 8 rows 136 -> 130 us)
    const int cu = compute_units();
    const int rt = M <= 16 ? 1 : M <= 32 ? 2 : 4;
    // (four tiles side by side were slower than two: the 7B's gate/up matrix at 8 rows 148 against 130 us)
    int tiles = N > 16 * cu ? 2 : 1;                          // tiles of 16 outputs
    if (swiglu) tiles = 1;                                    // (a pair of gate and up tiles: two tiles of w already)
    const int most = 16 * tiles;
    const int rounds = (N + cu * most - 1) / (cu * most);
    int cols = (N + cu * rounds - 1) / (cu * rounds);
    if (cols < 1) cols = 1;
    const long groups = (N + cols - 1) / cols;
    if (groups > 0x7fffffffL) return LI_ERR_SIZE;
    const unsigned grid = (unsigned)groups;
    // pieces a trip: a long K keeps four a wave in flight, a short one two (measured: 3,584 columns 136 against
    // 156 us for the 7B's gate/up matrix, 18,944 columns 68.6 against 74.0 us for its way back), a tiny one, and
    // many rows (whose registers hold the rows' pieces too), one
#define LI_F32RM(AH, TL, RTV, SW) gemm_f32_rows_mfma_kernel<AH, TL, RTV, SW><<<grid, F32RM_WAVES * 64, 0, stream>>>(x, w, bias, out, M, N, K, accumulate, cols)
    const int ahead = rt == 4 ? 1 : K >= 8192 && rt == 1 ? 4 : K >= 32 * F32RM_WAVES * 4 ? 2 : 1;
    if (swiglu) {
        if (rt == 1) { if (ahead == 4) LI_F32RM(4, 2, 1, true); else if (ahead == 2) LI_F32RM(2, 2, 1, true); else LI_F32RM(1, 2, 1, true); }
        else if (rt == 2) { if (ahead >= 2) LI_F32RM(2, 2, 2, true); else LI_F32RM(1, 2, 2, true); }
        else LI_F32RM(1, 2, 4, true);
        return li_launch_status();
    }
    if (rt == 1) {
        if (tiles == 2) { if (ahead == 4) LI_F32RM(4, 2, 1, false); else if (ahead == 2) LI_F32RM(2, 2, 1, false); else LI_F32RM(1, 2, 1, false); }
        else { if (ahead == 4) LI_F32RM(4, 1, 1, false); else if (ahead == 2) LI_F32RM(2, 1, 1, false); else LI_F32RM(1, 1, 1, false); }
    } else if (rt == 2) {
        if (tiles == 2) { if (ahead >= 2) LI_F32RM(2, 2, 2, false); else LI_F32RM(1, 2, 2, false); }
        else { if (ahead >= 2) LI_F32RM(2, 1, 2, false); else LI_F32RM(1, 1, 2, false); }
    } else {
        if (tiles == 2) LI_F32RM(1, 2, 4, false); else LI_F32RM(1, 1, 4, false);
    }
#undef LI_F32RM
    return li_launch_status();
}

// ----------------------------------------------------------- bfloat16 MFMA
// Block tile 128 x 128, K in steps of 32, 4 waves in a 2 x 2 grid, each wave a
// 64 x 64 tile made of 2 x 2 MFMA 32x32x16 tiles.  Operand layout of
// v_mfma_f32_32x32x16_bf16: lane l holds 8 consecutive k of row (l % 32),
// starting at k = 8 * (l / 32), for A and for B alike; the result's register r
// of lane l is row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
#define BF_BM 128
#define BF_BN 128
#define BF_BK 32
#define BF_LDS_STRIDE (BF_BK + 8)           // in elements; the pad spreads rows over banks

struct __attribute__((aligned(16))) chunk16 { uint32_t w[4]; };

template <bool ALIGNED>
__device__ __forceinline__ chunk16 load_chunk(const bf16_t* __restrict__ base, int row, int rows,
                                              int k, int K) {
    chunk16 c = {{0u, 0u, 0u, 0u}};
    if (row >= rows || k >= K) return c;
    const bf16_t* p = base + (size_t)row * K + k;
    if (ALIGNED) {                                   // K % 8 == 0: the chunk is whole and 16-byte aligned
        c = *reinterpret_cast<const chunk16*>(p);
    } else {
        uint16_t e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = (k + i < K) ? p[i].bits : (uint16_t)0;
#pragma unroll
        for (int i = 0; i < 4; ++i) c.w[i] = (uint32_t)e[2 * i] | ((uint32_t)e[2 * i + 1] << 16);
    }
    return c;
}

template <typename TO, bool ALIGNED>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const bf16_t* __restrict__ x,
                                                         const bf16_t* __restrict__ w,
                                                         const float* __restrict__ bias,
                                                         TO* __restrict__ out, int M, int N, int K,
                                                         int accumulate) {
    __shared__ __attribute__((aligned(16))) uint16_t As[BF_BM * BF_LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[BF_BN * BF_LDS_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    const int m0 = blockIdx.y * BF_BM, n0 = blockIdx.x * BF_BN;
    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // each thread moves two 16-byte chunks of A and two of B per K step
    const int crow0 = tid >> 2, ck = (tid & 3) * 8;
    chunk16 ra[2], rb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        ra[i] = load_chunk<ALIGNED>(x, m0 + crow0 + 64 * i, M, ck, K);
        rb[i] = load_chunk<ALIGNED>(w, n0 + crow0 + 64 * i, N, ck, K);
    }
    const int frow = lane & 31, fk = (lane >> 5) * 8;
    for (int k0 = 0; k0 < K; k0 += BF_BK) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<chunk16*>(&As[(crow0 + 64 * i) * BF_LDS_STRIDE + ck]) = ra[i];
            *reinterpret_cast<chunk16*>(&Bs[(crow0 + 64 * i) * BF_LDS_STRIDE + ck]) = rb[i];
        }
        __syncthreads();
        if (k0 + BF_BK < K) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                ra[i] = load_chunk<ALIGNED>(x, m0 + crow0 + 64 * i, M, k0 + BF_BK + ck, K);
                rb[i] = load_chunk<ALIGNED>(w, n0 + crow0 + 64 * i, N, k0 + BF_BK + ck, K);
            }
        }
#pragma unroll
        for (int ks = 0; ks < BF_BK; ks += 16) {
            bf16x8 af[2], bfr[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                af[i] = *reinterpret_cast<const bf16x8*>(&As[(wm + 32 * i + frow) * BF_LDS_STRIDE + ks + fk]);
                bfr[i] = *reinterpret_cast<const bf16x8*>(&Bs[(wn + 32 * i + frow) * BF_LDS_STRIDE + ks + fk]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
    }
    const int ccol = lane & 31, crow = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wn + 32 * j + ccol;
            if (col >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm + 32 * i + 8 * (r >> 2) + crow + (r & 3);
                if (row < M) epilogue_store(out, (size_t)row * N + col, acc[i][j][r], bias, col, accumulate);
            }
        }
}

// ---------------------------------------------- bfloat16, many rows (prompts)
// With many rows the product is bound by the matrix cores and, before them, by
// how often an operand byte has to be read from LDS: a wave's tile of WM x WN
// needs (WM + WN) * BK operand elements for WM * WN * BK multiply-adds, so the
// tiles are made large.  Block tile BM x BN, 4 waves as 2 x 2, wave tile
// BM/2 x BN/2 made of MFMA 32x32x16 tiles, K in steps of 64.  Two LDS stages:
// the global loads of the next K step are in flight (in registers) while this
// step is multiplied from LDS, then written to the other stage; one barrier a
// step.  A row of a stage is 64 elements = 128 bytes = 8 chunks of 16 bytes;
// chunk c of row r lies at position c ^ ((r >> 1) & 7), which spreads the 16
// rows that one fragment read touches over all banks.
// Blocks go to the 8 XCDs in turn (block b runs on XCD b % 8), and each XCD has an L2 of its
// own.  The tiles are put in one sequence: patches of up to 8 row panels x 4 or more column panels
// (32 tiles, what an XCD runs at one time; smaller at the matrix's edges), patches along the rows
// first, then along the columns; what a patch reads from beyond its L2 is (8 + 4) panels for 32
// tiles.  Each XCD takes one eighth of the sequence in one piece: a run of neighbouring column
// panels of W, which no other XCD reads but for the two panels at its ends.  Every block has a
// tile, but for the last few of the last XCD, and no XCD has more than one tile more than another:
// blocks that return at once in the middle of the queue, and XCDs with a column panel more than
// others, made a matrix of fewer tiles than compute units take two rounds.
struct TileOrder {
    int pm, gn;                                      // row panels and column panels of a patch
    __host__ __device__ TileOrder(int mtiles) {
        pm = mtiles < 8 ? mtiles : 8;
        gn = 32 / pm;
    }
    __host__ static long blocks(long mtiles, long ntiles, long nsplit = 1) {      // grid size: the same number of blocks on each XCD
        return (mtiles * ntiles * nsplit + 7) / 8 * 8;
    }
    // With K in nsplit parts: where the tiles divide by 8 every XCD takes its eighth of them in every
    // part (the same rows of w, all of K).  Otherwise the sequence is that of the tiles nsplit times
    // over, part after part, and the XCDs share the whole of it: dealt part by part, the last XCD's
    // few tiles fewer would come nsplit times over and the other XCDs would hold more blocks than they
    // have compute units (36 tiles in 7 parts: 35 blocks on each of seven XCDs, 7 on the last).
    // (All of it in 32 bits: the launch has checked that the blocks fit.)
    __device__ bool tile(unsigned block, int mtiles, int ntiles, int nsplit, int& mt, int& nt, int& split) const {
        const unsigned tiles = (unsigned)mtiles * (unsigned)ntiles, total = tiles * (unsigned)nsplit;
        unsigned t;
        if (nsplit > 1 && (tiles & 7) == 0) {
            split = (int)(block / tiles);
            const unsigned b = block - (unsigned)split * tiles;
            t = (b & 7) * (tiles >> 3) + (b >> 3);
        } else {
            const unsigned per = (total + 7) / 8, s = (block & 7) * per + (block >> 3);
            if (s >= total) return false;
            split = (int)(s / tiles);
            t = s - (unsigned)split * tiles;
        }
        const int group = mtiles * gn;               // tiles of gn column panels
        const int cg = (int)(t / group), r = (int)(t % group);
        const int gc = ntiles - cg * gn < gn ? ntiles - cg * gn : gn;        // column panels of this group
        const int rg = r / (pm * gc), r2 = r % (pm * gc);
        const int rows_in = mtiles - rg * pm < pm ? mtiles - rg * pm : pm;  // row panels of this patch
        mt = rg * pm + r2 % rows_in;
        nt = cg * gn + r2 / rows_in;
        return true;
    }
};

template <int BM, int BN, int BK, typename TO>
__global__ __launch_bounds__(256) void gemm_bf16_big_kernel(const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ w,
                                                             const float* __restrict__ bias,
                                                             TO* __restrict__ out, int M, int N, int K,
                                                             int accumulate) {
    constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
    constexpr int CPR = BK / 8;                                   // 16-byte chunks in a row of a stage
    constexpr int WRAP = 128 / BK;                                // rows that fill all 64 banks once
    constexpr int CA = BM * CPR / 256, CB = BN * CPR / 256;       // chunks per thread and stage
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    uint16_t* As = lds;                                           // [2][BM][BK]
    uint16_t* Bs = lds + 2 * BM * BK;                             // [2][BN][BK]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;
    const int mtiles = (M + BM - 1) / BM, ntiles = (N + BN - 1) / BN;
    int mt, nt, split;
    if (!TileOrder(mtiles).tile(blockIdx.x, mtiles, ntiles, 1, mt, nt, split)) return;
    const int m0 = mt * BM, n0 = nt * BN;
    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    auto slot = [](int row, int c) { return row * BK + ((c ^ ((row / WRAP) & (CPR - 1))) << 3); };
    // Global loads carry no branches: a row past the end is read as the last row (its products
    // land in output rows that are not stored), and only a K step that reaches past K is
    // masked, chunk by chunk.
    bf16x8 ra[CA], rb[CB];
    size_t oa[CA], ob[CB];
#pragma unroll
    for (int i = 0; i < CA; ++i) {
        const int qd = tid + 256 * i, row = qd / CPR, c = qd % CPR;
        oa[i] = (size_t)((m0 + row < M) ? m0 + row : M - 1) * K + 8 * c;
    }
#pragma unroll
    for (int i = 0; i < CB; ++i) {
        const int qd = tid + 256 * i, row = qd / CPR, c = qd % CPR;
        ob[i] = (size_t)((n0 + row < N) ? n0 + row : N - 1) * K + 8 * c;
    }
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#define LI_GLOAD(k0)                                                                                      \
    {                                                                                                     \
        const bool full_ = (k0) + BK <= K;                                                                \
        _Pragma("unroll") for (int i = 0; i < CA; ++i)                                                    \
            ra[i] = (full_ || (k0) + 8 * ((tid + 256 * i) % CPR) < K)                                     \
                        ? *reinterpret_cast<const bf16x8*>(x + oa[i] + (k0)) : zero8;                     \
        _Pragma("unroll") for (int i = 0; i < CB; ++i)                                                    \
            rb[i] = (full_ || (k0) + 8 * ((tid + 256 * i) % CPR) < K)                                     \
                        ? *reinterpret_cast<const bf16x8*>(w + ob[i] + (k0)) : zero8;                     \
    }
#define LI_LSTORE(stage)                                                                                  \
    {                                                                                                     \
        _Pragma("unroll") for (int i = 0; i < CA; ++i) {                                                  \
            const int qd = tid + 256 * i, row = qd / CPR, c = qd % CPR;                                   \
            *reinterpret_cast<bf16x8*>(&As[(stage) * BM * BK + slot(row, c)]) = ra[i];                    \
        }                                                                                                 \
        _Pragma("unroll") for (int i = 0; i < CB; ++i) {                                                  \
            const int qd = tid + 256 * i, row = qd / CPR, c = qd % CPR;                                   \
            *reinterpret_cast<bf16x8*>(&Bs[(stage) * BN * BK + slot(row, c)]) = rb[i];                    \
        }                                                                                                 \
    }
    const int frow = lane & 31, fh = lane >> 5;
    const int nk = (K + BK - 1) / BK;
    // fragments of K sub-step ks + 1 are read from LDS before the MFMAs of sub-step ks are
    // issued, so the reads' latency passes while the matrix cores work
    bf16x8 af[2][TM], bfr[2][TN];
#define LI_FREAD(stage, ks, buf)                                                                          \
    {                                                                                                     \
        const int c_ = 2 * (ks) + fh;                                                                     \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                    \
            af[buf][i] = *reinterpret_cast<const bf16x8*>(&As[(stage) * BM * BK + slot(wm + 32 * i + frow, c_)]); \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                    \
            bfr[buf][j] = *reinterpret_cast<const bf16x8*>(&Bs[(stage) * BN * BK + slot(wn + 32 * j + frow, c_)]); \
    }
    LI_GLOAD(0)
    LI_LSTORE(0)
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int stage = kt & 1;
        if (kt + 1 < nk) LI_GLOAD((kt + 1) * BK)
        LI_FREAD(stage, 0, 0)
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            if (ks + 1 < BK / 16) LI_FREAD(stage, ks + 1, (ks + 1) & 1)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bfr[ks & 1][j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) LI_LSTORE(stage ^ 1)
        __syncthreads();
    }
#undef LI_FREAD
#undef LI_GLOAD
#undef LI_LSTORE
    // Epilogue through LDS: a wave puts a band of 32 rows of its tile into a piece of LDS of its
    // own and takes it out again row by row, 8 consecutive columns a lane, so that the stores
    // (and the loads of what is added to) are whole 16-byte pieces, 16 lanes to a row.
    __syncthreads();                               // the main loop's LDS is free now
    constexpr int ESTRIDE = WN + 4;                // floats per row of a band (pad against bank conflicts)
    float* band = reinterpret_cast<float*>(lds) + wave * 32 * ESTRIDE;
    const int ccol = lane & 31, crow = (lane >> 5) * 4;
    constexpr int LPR = WN / 8;                    // lanes that take one row of the band out (8 columns each)
    constexpr int RPP = 64 / LPR;                  // rows per pass of the wave
    const int erow = lane / LPR, ecol = (lane % LPR) * 8;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                band[(8 * (r >> 2) + crow + (r & 3)) * ESTRIDE + 32 * j + ccol] = acc[i][j][r];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int pass = 0; pass < 32 / RPP; ++pass) {
            const int row = m0 + wm + 32 * i + RPP * pass + erow;
            if (row >= M) continue;
            {
                const int col = n0 + wn + ecol;
                if (col >= N) continue;
                const float* src = &band[(RPP * pass + erow) * ESTRIDE + ecol];
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = src[e];
                const size_t idx = (size_t)row * N + col;
                if (col + 8 <= N && (N % 8) == 0) {               // whole pieces: wide loads and stores
                    if (bias) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] += bias[col + e];
                    }
                    if constexpr (sizeof(TO) == 4) {
                        float4* o = reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + idx);
                        if (accumulate) {
                            const float4 a0 = o[0], a1 = o[1];
                            v[0] += a0.x; v[1] += a0.y; v[2] += a0.z; v[3] += a0.w;
                            v[4] += a1.x; v[5] += a1.y; v[6] += a1.z; v[7] += a1.w;
                        }
                        o[0] = float4{v[0], v[1], v[2], v[3]};
                        o[1] = float4{v[4], v[5], v[6], v[7]};
                    } else {
                        chunk16 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            o.w[e] = pack2_bf16(v[2 * e], v[2 * e + 1]);
                        *reinterpret_cast<chunk16*>(reinterpret_cast<uint16_t*>(out) + idx) = o;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (col + e < N) epilogue_store(out, idx + e, v[e], bias, col + e, accumulate);
                }
            }
        }
    }
}

// ------------------------------- bfloat16, many rows, loads straight into LDS
// The same tiling with the global loads going straight into LDS
// (global_load_lds_dwordx4: lane i's 16 bytes land at the wave's LDS base + 16 i),
// which needs no staging registers, so all stages but the one being multiplied are
// in flight: the latency of a load is long against a step.  The
// compiler does not track these loads' completion; `s_waitcnt vmcnt(n)` is
// placed by hand: a wave's loads retire in order, so allowing the loads of the
// younger steps to stay outstanding waits exactly for the oldest step, and the
// barrier after it makes that true for the loads of all four waves.
// Needs K to be a multiple of the step (a load cannot be masked to zeros).  A step is 64
// columns, so that a row of a stage is one whole 128-byte line of the caches.  Tiles: 256 x 256
// with two stages, 256 x 128 with three, 128 x 128 with four (what fits the 160 KB of LDS).
#define LI_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)
#define LI_LOAD_TO_LDS(gptr, lptr)                                                                        \
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr),              \
                                     (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)

// up * gate / (1 + exp(-gate)) for a result that is rounded to bfloat16: the exponential and the reciprocal are
// the instructions' own (v_exp_f32, v_rcp_f32: an ulp each), 5 instructions where expf and the division are some
// 25; a tile of 256 x 256 makes 128 of them a thread, 7 % of the tile's time.  (A gate far below zero: the
// exponential overflows to infinity, the reciprocal is 0 and so is the result, as it should be.)  The 32-bit
// path keeps expf and the division.
__device__ __forceinline__ float swiglu_bf16(float gate, float up) {
    const float e = __builtin_amdgcn_exp2f(-1.44269504088896341f * gate);
    return up * (gate * __builtin_amdgcn_rcpf(1.0f + e));
}

// f(std::integral_constant<int, 0>) ... f(std::integral_constant<int, N - 1>)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// The same load with its address as (scalar base) + (32-bit offset of the lane): no address
// arithmetic in vector registers.  M0 carries the LDS address, as in the compiler's own form.
#define LI_LOAD_TO_LDS_AT(base, voff, lptr)                                                              \
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"                          \
                 :: "s"((uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(lptr)), "v"(voff), "s"(base) : "memory", "m0")

template <int BM, int BN, int BK, int NSTAGE, bool SWIGLU, typename TO, int WLM = 2>
__global__ __launch_bounds__(256) void gemm_bf16_dma_kernel(const bf16_t* __restrict__ x,
                                                             const bf16_t* __restrict__ w,
                                                             const float* __restrict__ bias,
                                                             TO* __restrict__ out, int M, int N, int K,
                                                             int accumulate, int nsplit,
                                                             const float* __restrict__ row_parts, int nparts, float eps) {
    // row_parts (SwiGLU tiles of 64 rows, up to 32 rows of x): x is the xg of li_linear_residual_norm and these
    // are its sq_parts; every row's sums are scaled by 1 / sqrt(sum of the row's parts / K + eps) before the
    // activation, which makes the result that of the RMS norm (the factor of a row does not depend on k).
    // nsplit > 1: a block multiplies one of nsplit parts of K, the y-th, and writes its sums to the y-th
    // [M, N] matrix behind `out` (float, no bias, no accumulation); splitk_reduce_kernel adds them
    // WLM: waves along the rows of the tile, 2 (two by two) or 4 (each wave 32-row bands over all columns:
    // BN may then be any multiple of 32, for matrices whose columns no other tile divides into 256 tiles)
    constexpr int WLN = 4 / WLM;
    constexpr int WM = BM / WLM, WN = BN / WLN, TM = WM / 32, TN = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0 && (WLM == 2 || WLM == 4), "a wave's part of the tile is made of 32 x 32 tiles");
    constexpr bool SWSPLIT = SWIGLU && (TN % 2 == 1);        // gates and ups in different waves (see the rows of w below)
    static_assert(!SWSPLIT || WLN == 2, "gates in one wave, ups in the wave beside it");
    static_assert(BM % 32 == 0 && BN % 32 == 0 && (BM / 4) % (64 / (BK / 8)) == 0 && (BN / 4) % (64 / (BK / 8)) == 0, "whole load instructions a wave");
    constexpr int CPR = BK / 8, WRAP = 128 / BK;                 // chunks in a row; rows that fill all banks once
    constexpr int RPI = 64 / CPR;                                // rows one load instruction of a wave covers
    constexpr int IA = BM / 4 / RPI, IB = BN / 4 / RPI;          // load instructions per wave and step for A and B
    constexpr int STAGE = (BM + BN) * BK;                        // elements of a stage: A rows then B rows
    constexpr int LPW = IA + IB;                                 // loads a wave issues per step
    extern __shared__ __attribute__((aligned(16))) uint16_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave / WLN) * WM, wn = (wave % WLN) * WN;
    const int mtiles = (M + BM - 1) / BM, ntiles = (N + BN - 1) / BN;
    int mt, nt, split;
    if (!TileOrder(mtiles).tile(blockIdx.x, mtiles, ntiles, nsplit, mt, nt, split)) return;
    const int m0 = mt * BM, n0 = nt * BN;
    constexpr bool ROWSCALE = SWIGLU && BM == 64;
    // The shares of the rows' sums of squares are asked for now, all at once and never conditional (a share
    // past the last reads the last and is not added), before the first loads of the main loop: a wave's loads
    // retire in order, so they have arrived when the first stage has, and the waits placed by hand below
    // still count the main loop's loads only.  They are added up behind the main loop.
    constexpr int RS_PER = ROWSCALE ? 64 : 1;          // shares a thread adds: 512 at most, 16 or 8 threads a row
    [[maybe_unused]] float rs_part[RS_PER];
    [[maybe_unused]] const int rs_rows = M <= 16 ? 16 : 32;      // rows the shares are kept for (as the product before the norm wrote them)
    [[maybe_unused]] const int rs_groups = 256 / rs_rows;
    if constexpr (ROWSCALE) {
        if (row_parts) {
            const int r = threadIdx.x % rs_rows, g = threadIdx.x / rs_rows;
#pragma unroll
            for (int i = 0; i < RS_PER; ++i) {
                const int p = g + rs_groups * i;
                rs_part[i] = 0.f;
                if (rs_groups * i < nparts) rs_part[i] = row_parts[(size_t)(p < nparts ? p : nparts - 1) * rs_rows + r];      // (the same for all lanes)
            }
        }
    }
    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    // chunk c of row r lies at position c ^ ((r / WRAP) % CPR) of the row's CPR positions
    auto slot = [](int row, int c) { return row * BK + ((c ^ ((row / WRAP) & (CPR - 1))) << 3); };
    // this lane's part of a step: a wave takes BM / 4 rows of A and BN / 4 rows of B; one
    // instruction covers RPI rows, lane -> row lane / CPR, position lane % CPR
    // Addresses: a base that is the same for the whole wave (scalar registers, moved on by a step's
    // columns) plus this lane's 32-bit byte offset within the tile's rows, which never changes.
    uint32_t ga[IA], gb[IB];
    const bf16_t* abase = x + (size_t)m0 * K;
    const bf16_t* bbase = w + (size_t)(SWIGLU ? n0 / 2 : n0) * K;
#pragma unroll
    for (int i = 0; i < IA; ++i) {
        const int row = (BM / 4) * wave + RPI * i + lane / CPR, c = (lane % CPR) ^ ((row / WRAP) & (CPR - 1));
        ga[i] = (uint32_t)(((size_t)((m0 + row < M) ? row : M - 1 - m0) * K + 8 * c) * 2);       // rows past the end: the last row
    }
#pragma unroll
    for (int i = 0; i < IB; ++i) {
        const int row = (BN / 4) * wave + RPI * i + lane / CPR, c = (lane % CPR) ^ ((row / WRAP) & (CPR - 1));
        size_t rel = (n0 + row < N) ? row : N - 1 - n0;            // row of w relative to the tile's first
        if constexpr (SWIGLU && !SWSPLIT) {
            // w is [gate; up] with N / 2 rows each.  The tile's rows alternate in blocks of 32: 32
            // gate rows, the 32 up rows of the same outputs, the next 32 gate rows, ..., so that an
            // accumulator tile and its neighbour hold the two factors of one output tile.
            const int half = N / 2, blk = row / 32;
            const int o = n0 / 2 + (blk / 2) * 32 + row % 32;
            rel = (size_t)((o < half ? o : half - 1) - n0 / 2) + (size_t)(blk & 1) * half;
        } else if constexpr (SWSPLIT) {
            // (a wave's part of the tile is an odd number of blocks of 32 columns: the tile's first half
            // are gate rows, its second half the up rows of the same outputs, so that of two waves side
            // by side one holds the gates and the other the ups; they meet in the epilogue's LDS)
            const int half = N / 2;
            const int o = n0 / 2 + row % (BN / 2);
            rel = (size_t)((o < half ? o : half - 1) - n0 / 2) + (size_t)(row / (BN / 2)) * half;
        }
        gb[i] = (uint32_t)((rel * K + 8 * c) * 2);
    }
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    // load `idx` of a wave's LPW loads of step kt: first its rows of A, then its rows of B
    auto issue_one = [&](int kt, int idx) {
        uint16_t* st = lds + (kt % NSTAGE) * STAGE;
        if (idx < IA) LI_LOAD_TO_LDS_AT(abase + (size_t)kt * BK, ga[idx], st + ((BM / 4) * uwave + RPI * idx) * BK);
        else LI_LOAD_TO_LDS_AT(bbase + (size_t)kt * BK, gb[idx - IA], st + BM * BK + ((BN / 4) * uwave + RPI * (idx - IA)) * BK);
    };
    auto issue = [&](int kt) {
#pragma unroll
        for (int i = 0; i < LPW; ++i) issue_one(kt, i);
    };
    const int frow = lane & 31, fh = lane >> 5;
    // (the parts' steps: equal shares, the first parts one more where they do not divide)
    const int ksteps = K / BK, kshare = ksteps / nsplit, kmore = ksteps - kshare * nsplit;
    const int kt_first = split * kshare + (split < kmore ? split : kmore);
    const int nk = kshare + (split < kmore ? 1 : 0);
    out += (size_t)split * M * (SWIGLU ? N / 2 : N);
    abase += (size_t)kt_first * BK;
    bbase += (size_t)kt_first * BK;
    constexpr int KS = BK / 16;                    // MFMA groups of a step: 16 columns each
    constexpr int GM = TM * TN, GD = TM + TN;      // MFMAs and fragment reads of a group
    // Order of a step.  A wave issues in order and is alone on its SIMD, and the CU's address unit
    // takes a 16-byte-per-lane load of one wave every 16 cycles, i.e. one of each of the four waves
    // every 64 = two MFMAs: loads issued back to back hold the wave, and with it the SIMD's
    // MFMAs, until the unit has taken them.  So the loads of step kt + NSTAGE - 1 (into the stage
    // that the barrier of step kt - 1 freed) are issued one by one between the MFMAs of the first
    // groups of step kt, at most one per two MFMAs.  Each group's MFMAs run while the fragments
    // of the next 16 columns are read; in the middle of the LAST group the wave waits for the
    // loads of step kt + 1, meets the others at the barrier (stage kt + 1 is there for all, stage kt
    // is read by all) and reads the first fragments of step kt + 1, so that the barrier and the
    // latency of LDS fall under the remaining MFMAs.
    // With 64 rows of x a step has few MFMAs and the product waits for w from memory: there the
    // loads of step kt + NSTAGE are issued all at once, right after the barrier of step kt, so that as
    // many bytes as possible are on their way.
    constexpr bool SPREAD = BM >= 128;
    constexpr int AHEAD = SPREAD ? NSTAGE - 1 : NSTAGE;                // steps loaded before the first is multiplied
    constexpr int PER0 = GM / 2 > 0 ? GM / 2 : 1, PER1 = (LPW + KS - 2) / (KS - 1);
    constexpr int PER = PER0 > PER1 ? PER0 : PER1;                     // loads of one group
#pragma unroll
    for (int p = 0; p < AHEAD; ++p)
        if (p < nk) issue(p);
    bf16x8 af[2][TM], bfr[2][TN];
#define LI_FREAD(stage_, ks, buf)                                                                          \
    {                                                                                                     \
        const uint16_t* As_ = lds + (stage_) * STAGE;                                                     \
        const uint16_t* Bs_ = As_ + BM * BK;                                                              \
        const int c_ = 2 * (ks) + fh;                                                                     \
        _Pragma("unroll") for (int i = 0; i < TM; ++i)                                                    \
            af[buf][i] = *reinterpret_cast<const bf16x8*>(&As_[slot(wm + 32 * i + frow, c_)]);            \
        _Pragma("unroll") for (int j = 0; j < TN; ++j)                                                    \
            bfr[buf][j] = *reinterpret_cast<const bf16x8*>(&Bs_[slot(wn + 32 * j + frow, c_)]);           \
    }
#define LI_WAIT_YOUNGER(y)                                                                                 \
    { if ((y) >= 3) LI_VMCNT(3 * LPW); else if ((y) == 2) LI_VMCNT(2 * LPW); else if ((y) == 1) LI_VMCNT(LPW); else LI_VMCNT(0); }
    {
        const int inflight = nk < AHEAD ? nk : AHEAD;
        LI_WAIT_YOUNGER(inflight - 1)
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        LI_FREAD(0, 0, 0)
    }
    // one step; LOADS: the loads of step kt + NSTAGE - 1 are issued between its MFMAs
    auto step = [&](int kt, auto loads_tag) {
        constexpr bool LOADS = decltype(loads_tag)::value;
        const int stage = kt % NSTAGE;
        static_for<KS - 1>([&](auto ks_tag) {
            constexpr int ks = decltype(ks_tag)::value;
            constexpr int l0 = ks * PER < LPW ? ks * PER : LPW, l1 = (ks + 1) * PER < LPW ? (ks + 1) * PER : LPW;
            constexpr int NL = LOADS && SPREAD ? l1 - l0 : 0;
            const uint16_t* As_ = lds + stage * STAGE;
            const uint16_t* Bs_ = As_ + BM * BK;
            const int c_ = 2 * (ks + 1) + fh;
            // written in the order it is to run, and kept so: before MFMA m the m-th fragment read of
            // the next 16 columns (the earlier MFMAs the more, where there are more reads than MFMAs:
            // the group's remaining MFMAs are what covers the latency of LDS), after it the loads that
            // fall to it
            static_for<GM>([&](auto m_tag) {
                constexpr int m = decltype(m_tag)::value;
                constexpr int r0 = GD > GM ? GD - ((GM - m) * GD) / GM : (m < GD ? m : GD);
                constexpr int r1 = GD > GM ? GD - ((GM - m - 1) * GD) / GM : (m < GD ? m + 1 : GD);
#pragma unroll
                for (int r = r0; r < r1; ++r) {
                    if (r < TM) af[(ks + 1) & 1][r] = *reinterpret_cast<const bf16x8*>(&As_[slot(wm + 32 * r + frow, c_)]);
                    else bfr[(ks + 1) & 1][r - TM] = *reinterpret_cast<const bf16x8*>(&Bs_[slot(wn + 32 * (r - TM) + frow, c_)]);
                }
                acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][m / TN], bfr[ks & 1][m % TN], acc[m / TN][m % TN], 0, 0, 0);
#pragma unroll
                for (int l = l0 + (m * NL) / GM; l < l0 + ((m + 1) * NL) / GM; ++l) issue_one(kt + NSTAGE - 1, l);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        constexpr int BL = (KS - 1) & 1;           // the buffer with the fragments of the last 16 columns
        constexpr int HALF = (TM / 2) * TN > 0 ? (TM / 2) * TN : GM / 2;       // MFMAs of the last group before the wait
#pragma unroll
        for (int m = 0; m < HALF; ++m)
            acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[BL][m / TN], bfr[BL][m % TN], acc[m / TN][m % TN], 0, 0, 0);
        if (kt + 1 < nk) {
            // loads of later steps that may stay in flight: steps kt + 2 .. kt + NSTAGE - 1, where they exist
            const int younger = LOADS ? NSTAGE - 2 : (nk - 2 - kt < NSTAGE - 2 ? nk - 2 - kt : NSTAGE - 2);
            LI_WAIT_YOUNGER(younger)
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if constexpr (!SPREAD) {
                if (kt + NSTAGE < nk) issue(kt + NSTAGE);              // into the stage of step kt
            }
            LI_FREAD((kt + 1) % NSTAGE, 0, 0)
        }
#pragma unroll
        for (int m = HALF; m < GM; ++m)
            acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[BL][m / TN], bfr[BL][m % TN], acc[m / TN][m % TN], 0, 0, 0);
    };
    int kt = 0;
    if constexpr (SPREAD)
        for (; kt + NSTAGE - 1 < nk; ++kt) step(kt, std::true_type{});
    for (; kt < nk; ++kt) step(kt, std::false_type{});
#undef LI_FREAD
#undef LI_WAIT_YOUNGER
    __syncthreads();                               // the main loop's LDS is free now
    [[maybe_unused]] float* row_inv = nullptr;
    if constexpr (ROWSCALE) {
        // the rows' factors, in the order of additions of the few-row kernel with four waves: thread t adds the
        // shares t / R, t / R + 256 / R, ... of row t % R (R = 16 rows, or 32), thread r < R the sums of row r
        __shared__ float inv_s[32], part_s[256];
        row_inv = inv_s;
        if (row_parts) {
            const int r = threadIdx.x % rs_rows, g = threadIdx.x / rs_rows;
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < RS_PER; ++i) mine += (g + rs_groups * i < nparts) ? rs_part[i] : 0.f;
            part_s[g * rs_rows + r] = mine;
            __syncthreads();
            if ((int)threadIdx.x < rs_rows) {
                float sq = part_s[threadIdx.x];
                for (int q = 1; q < rs_groups; ++q) sq += part_s[q * rs_rows + threadIdx.x];
                inv_s[threadIdx.x] = 1.0f / sqrtf(sq / (float)K + eps);
            }
            __syncthreads();
        }
    }
    if constexpr (SWSPLIT) {
        // every wave leaves its sums in its band; of two waves side by side the first then takes rows 0 .. 15
        // of the 32 and the second rows 16 .. 31: gates from the first wave's band, ups from the second's
        constexpr int ES = WN + 4;
        static_assert(4 * 32 * ES * 4 <= NSTAGE * STAGE * 2, "the waves' bands fit the main loop's LDS");
        float* bands = reinterpret_cast<float*>(lds);
        float* band = bands + wave * 32 * ES;
        const float* gband = bands + (wave & ~1) * 32 * ES;
        const float* uband = bands + (wave | 1) * 32 * ES;
        const int ccol = lane & 31, crow = (lane >> 5) * 4;
        constexpr int LPR = WN / 8, RPP = 64 / LPR;
        const int erow = lane / LPR, ecol = (lane % LPR) * 8;
        const int NO = N / 2;
        const int col = n0 / 2 + ecol;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            if (i > 0) __syncthreads();              // (the bands have been read)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    band[(8 * (r >> 2) + crow + (r & 3)) * ES + 32 * j + ccol] = acc[i][j][r];
            __syncthreads();
#pragma unroll
            for (int pass = 0; pass < (16 + RPP - 1) / RPP; ++pass) {
                const int rr = RPP * pass + erow;
                const int row = m0 + wm + 32 * i + 16 * (wave & 1) + rr;
                if (erow >= RPP || rr >= 16 || row >= M || col >= NO) continue;
                const float* gs = &gband[(16 * (wave & 1) + rr) * ES + ecol];
                const float* us = &uband[(16 * (wave & 1) + rr) * ES + ecol];
                float v[8];
                float f = 1.0f;
                if constexpr (ROWSCALE) f = row_parts ? row_inv[row & 31] : 1.0f;      // (row_parts: M <= 32, so row < 32 here)
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = swiglu_bf16(gs[e] * f, us[e] * f);
                const size_t o_idx = (size_t)row * NO + col;
                if (col + 8 <= NO && (NO % 8) == 0) {
                    chunk16 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o.w[e] = pack2_bf16(v[2 * e], v[2 * e + 1]);
                    *reinterpret_cast<chunk16*>(reinterpret_cast<uint16_t*>(out) + o_idx) = o;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (col + e < NO) epilogue_store(out, o_idx + e, v[e], nullptr, col + e, 0);
                }
            }
        }
        return;
    }
    constexpr int EW = SWIGLU ? WN / 2 : WN;        // output columns of a wave
    constexpr int ESTRIDE = EW + 4;
    static_assert(4 * 32 * ESTRIDE * 4 <= NSTAGE * STAGE * 2, "the waves' bands fit the main loop's LDS");
    float* band = reinterpret_cast<float*>(lds) + wave * 32 * ESTRIDE;
    const int ccol = lane & 31, crow = (lane >> 5) * 4;
    constexpr int LPR = EW / 8, RPP = 64 / LPR;     // lanes a row of the band takes; rows a pass of the wave covers
    const int erow = lane / LPR, ecol = (lane % LPR) * 8;      // (where 64 is no multiple of LPR the last lanes idle)
    const int NO = SWIGLU ? N / 2 : N;             // columns of out
    const int col = (SWIGLU ? (n0 + wn) / 2 : n0 + wn) + ecol;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        __builtin_amdgcn_wave_barrier();
        if constexpr (SWIGLU) {
#pragma unroll
            for (int j = 0; j < TN; j += 2)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float gv = acc[i][j][r], uv = acc[i][j + 1][r];
                    if constexpr (ROWSCALE) {
                        if (row_parts) {                 // (M <= 32: only the tile's first 32 rows are written)
                            const float f = row_inv[(wm + 32 * i + 8 * (r >> 2) + crow + (r & 3)) & 31];
                            gv *= f;
                            uv *= f;
                        }
                    }
                    band[(8 * (r >> 2) + crow + (r & 3)) * ESTRIDE + 16 * j + ccol] = swiglu_bf16(gv, uv);
                }
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    band[(8 * (r >> 2) + crow + (r & 3)) * ESTRIDE + 32 * j + ccol] = acc[i][j][r];
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int pass = 0; pass < (32 + RPP - 1) / RPP; ++pass) {
            const int row = m0 + wm + 32 * i + RPP * pass + erow;
            if (erow >= RPP || RPP * pass + erow >= 32 || row >= M || col >= NO) continue;
            const float* src = &band[(RPP * pass + erow) * ESTRIDE + ecol];
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = src[e];
            const size_t o_idx = (size_t)row * NO + col;
            if (col + 8 <= NO && (NO % 8) == 0) {
                if (bias) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += bias[col + e];
                }
                if constexpr (sizeof(TO) == 4) {
                    float4* o = reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + o_idx);
                    if (accumulate) {
                        const float4 a0 = o[0], a1 = o[1];
                        v[0] += a0.x; v[1] += a0.y; v[2] += a0.z; v[3] += a0.w;
                        v[4] += a1.x; v[5] += a1.y; v[6] += a1.z; v[7] += a1.w;
                    }
                    o[0] = float4{v[0], v[1], v[2], v[3]};
                    o[1] = float4{v[4], v[5], v[6], v[7]};
                } else {
                    chunk16 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o.w[e] = pack2_bf16(v[2 * e], v[2 * e + 1]);
                    *reinterpret_cast<chunk16*>(reinterpret_cast<uint16_t*>(out) + o_idx) = o;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (col + e < NO) epilogue_store(out, o_idx + e, v[e], bias, col + e, accumulate);
            }
        }
    }
}

template <int BM, int BN, int BK, int NSTAGE, bool SWIGLU, typename TO, int WLM = 2>
static int launch_dma(const bf16_t* x, const bf16_t* w, const float* bias, TO* out, int M, int N, int K,
                      int accumulate, hipStream_t stream, int nsplit = 1, const float* row_parts = nullptr,
                      int nparts = 0, float eps = 0.f) {
    if (row_parts && !(SWIGLU && BM == 64 && M <= 32 && nparts > 0)) return LI_ERR_SIZE;
    const long mtiles = (M + BM - 1) / BM, ntiles = (N + BN - 1) / BN;
    if (nsplit < 1 || nsplit > 65535 || nsplit > K / BK) return LI_ERR_SIZE;
    const long blocks = TileOrder::blocks(mtiles, ntiles, nsplit);
    if (blocks > 0x7fffffffL) return LI_ERR_SIZE;
    // a lane's byte offset from its tile's first row is kept in 32 bits (the gate and up rows of a
    // SwiGLU tile lie N / 2 rows apart)
    const unsigned long long span_rows = SWIGLU ? (unsigned long long)N / 2 + BN : (unsigned long long)(BM > BN ? BM : BN);
    if (span_rows * (unsigned long long)K * 2ull >= (1ull << 32)) return LI_ERR_SIZE;
    constexpr int lds_bytes = NSTAGE * (BM + BN) * BK * 2;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)gemm_bf16_dma_kernel<BM, BN, BK, NSTAGE, SWIGLU, TO, WLM>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
            return LI_ERR_LAUNCH;
        configured = true;
    }
    gemm_bf16_dma_kernel<BM, BN, BK, NSTAGE, SWIGLU, TO, WLM><<<(unsigned)blocks, 256, lds_bytes, stream>>>(x, w, bias, out, M, N, K, accumulate, nsplit, row_parts, nparts, eps);
    return li_launch_status();
}

// out (+)= sum over the parts, in the order of the parts, + bias
template <typename TO>
__global__ void splitk_reduce_kernel(const float* __restrict__ part, int nsplit, size_t mn, int N,
                                     const float* __restrict__ bias, TO* __restrict__ out, int accumulate) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= mn) return;
    float v = part[i];
    for (int s = 1; s < nsplit; ++s) v += part[(size_t)s * mn + i];
    epilogue_store(out, i, v, bias, (int)(i % N), accumulate);
}

// The same for the residual sum, one block a row, with the RMS norm of the new sum as a second
// result: out[m, :] += sum of the parts + bias (float32), xn[m, :] = gamma * out[m, :] /
// sqrt(mean(out[m, :]^2) + eps).  A row is kept in registers (N <= NT * PER).
template <typename TN, int NT, int PER>
__global__ __launch_bounds__(NT) void splitk_reduce_norm_kernel(const float* __restrict__ part, int nsplit, size_t mn, int N,
                                                                 const float* __restrict__ bias, float* __restrict__ out,
                                                                 const float* __restrict__ gamma, float eps,
                                                                 TN* __restrict__ xn) {
    __shared__ float red[NT / LI_WAVE];
    const size_t row = (size_t)blockIdx.x * N;
    float v[PER];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int n = threadIdx.x + i * NT;
        v[i] = 0.f;
        if (n < N) {
            // all loads at once (a part past the last reads the first and is not added): the block is
            // one of few and must not wait for memory part after part
            float a[8];
#pragma unroll
            for (int sp = 0; sp < 8; ++sp) a[sp] = part[(size_t)(sp < nsplit ? sp : 0) * mn + row + n];
            const float o = out[row + n];
            float t = a[0];
#pragma unroll
            for (int sp = 1; sp < 8; ++sp) t += sp < nsplit ? a[sp] : 0.f;
            if (bias) t += bias[n];
            t += o;
            out[row + n] = t;
            v[i] = t;
        }
        ss += v[i] * v[i];
    }
    ss = block_sum<NT>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)N + eps);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int n = threadIdx.x + i * NT;
        if (n < N) store_from_float(xn + row + n, gamma[n] * v[i] * inv);
    }
}
#define REDUCE_NORM_NT 1024
#define REDUCE_NORM_PER 8

template <int BM, int BN, int BK, typename TO>
static int launch_big(const bf16_t* x, const bf16_t* w, const float* bias, TO* out, int M, int N, int K,
                      int accumulate, hipStream_t stream) {
    const long mtiles = (M + BM - 1) / BM, ntiles = (N + BN - 1) / BN;
    const long per_xcd = TileOrder::blocks(mtiles, ntiles) / 8;
    if (per_xcd * 8 > 0x7fffffffL) return LI_ERR_SIZE;
    dim3 grid((unsigned)(per_xcd * 8));
    constexpr int lds_bytes = 2 * (BM + BN) * BK * 2;
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)gemm_bf16_big_kernel<BM, BN, BK, TO>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess)
            return LI_ERR_LAUNCH;
        configured = true;
    }
    gemm_bf16_big_kernel<BM, BN, BK, TO><<<grid, 256, lds_bytes, stream>>>(x, w, bias, out, M, N, K, accumulate);
    return li_launch_status();
}

// ------------------------------------------------- bfloat16, few rows (decode)
// With M <= 64 the product is bound by streaming W once from HBM, and the
// bandwidth reached is (bytes in flight) / (memory latency): the kernel is
// built to keep many independent 16-byte loads outstanding.  A block owns NT
// tiles of 16 rows of W (16 output columns each); its WAVES waves split K
// between them in chunks of 128 and add their partial sums through LDS in wave
// order.  The loads of a wave's next chunk are in flight while one chunk is
// multiplied.  Per chunk a lane loads four 16-byte pieces of one row of W per
// tile (the four lanes of a row together 64 contiguous bytes an instruction)
// and the matching pieces of x;
// v_mfma_f32_16x16x32_bf16 takes W as the row operand and x as the column
// operand (lane l: row/column l % 16, 8 k-values of k-group l / 16; any
// assignment of real k to (k-group, slot) is right as long as both operands
// share it).  The result's register r of lane l is row 4 * (l / 16) + r (an
// output column n), column l % 16 (an x row m).
//
// SWIGLU: W is [gate; up] with N rows each: tile 0 takes gate rows, tile 1 the
// up rows of the same columns, and out[m, n] = up * gate / (1 + exp(-gate)).
//
// ROPE (one tile of rows and of columns): W is the packed [q; k; v] projection.  A block takes,
// of one head, the 8 columns 8 i .. and their partners of the half-split rotation, dh / 2
// further on, so that lane l and lane l ^ 32 hold the two members of a pair; the epilogue adds
// the bias, rotates query and key heads by the row's angles (float32 tables), writes the
// queries to out and keys and values straight into their page slots (and to out as well).
#define SK_CHUNK 128

struct SkinnyArgs {
    const bf16_t* x;        // [M, K]
    const bf16_t* w;        // [N, K], or [2 N, K] with SWIGLU
    const float* bias;      // [N] or null
    void* out;              // [M, N]
    int M, N, K, accumulate;
    // ROPE (the packed q/k/v projection of a decoding step): rotary tables [M, dh / 2], the page
    // slot of each row, the cache layer's keys and values [pages, nkv, page_size, dh]
    const float* cos;
    const float* sin;
    const int* slot_map;
    bf16_t* kc;
    bf16_t* vc;
    int nh, nkv, dh, page_size, num_pages;
    // An RMS norm between two products of up to 32 rows, without a pass of its own.  The product
    // BEFORE it (float out with accumulate: the residual sum) also writes xg[m, n] = bf16(gamma[n] *
    // out[m, n]) and, per block, the sums of squares of its columns of out to sq_parts[block * R + m],
    // R = 16 up to 16 rows and 32 above.
    const float* gamma;
    bf16_t* xg;
    float* sq_parts;
    // The product AFTER it takes such an xg as its x and scales row m's sums by
    // 1 / sqrt(sum_p row_parts[p * R + m] / K + eps): the factor of a row does not depend on k.
    const float* row_parts;
    int nparts;
    float eps;
    // Columns a block takes (with ROPE: rotation pairs a block takes); 0: as many as its tiles hold.
    // Fewer than the tiles hold where that spreads a matrix of few columns evenly over the compute units.
    int cols;
};
#define SK_MAX_PARTS 512            // blocks of a producing product whose sums one consumer adds up

template <int MT, int NT, int WAVES, bool SWIGLU, typename TO, bool ROPE = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_bf16_skinny_kernel(SkinnyArgs a) {
    static_assert(!ROPE || (MT <= 2 && !SWIGLU), "the rotary epilogue takes one or two tiles of rows");
    static_assert(MT <= WAVES, "wave mt writes the results of row tile mt");
    __shared__ floatx4 red[WAVES][MT * NT][64];
    __shared__ float part_sums[WAVES * 64];          // [group of threads][row]: the rows' sums of squares, a share a group
    // rows that the shares of the sums of squares are kept for, a block and a step: 16 up to 16 rows, else 32
    // (the products on both sides of a norm see the same M)
    constexpr int RP = MT <= 1 ? 16 : 32;
    const int M = a.M, N = a.N, K = a.K;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);      // (the same for a wave's lanes: its branches are scalar)
    const int g = lane >> 4, r16 = lane & 15;
    const int per_block = a.cols > 0 ? a.cols : (ROPE ? 8 : 16) * (SWIGLU ? 1 : NT);
    const int n0 = blockIdx.x * per_block;                  // first column (with ROPE: first pair) of this block
    const int half = a.dh / 2;
    const int total = ROPE ? (a.nh + 2 * a.nkv) * half : N;
    const int nend = n0 + per_block < total ? n0 + per_block : total;     // one past its last
    const bf16_t* wrow[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        int row;
        if (SWIGLU) row = ((n0 + r16 < nend) ? n0 + r16 : nend - 1) + nt * N;      // gate row, up row
        else if (ROPE) {                                    // rows 0..7 of a tile: first members of 8 pairs, 8..15: their partners
            int p = n0 + 8 * nt + (r16 & 7);
            p = p < nend ? p : nend - 1;
            row = (p / half) * a.dh + p % half + (r16 < 8 ? 0 : half);
        } else row = (n0 + 16 * nt + r16 < nend) ? n0 + 16 * nt + r16 : nend - 1;    // rows past the end repeat the last
        wrow[nt] = a.w + (size_t)row * K;
    }
    // x is read with whole rows of a chunk contiguous over 16 lanes (lane l: row l / 16 + 4 i,
    // piece l % 16), which costs the load path a quarter of what reading it in the MFMA's
    // operand order would, and is turned into that order through a piece of LDS of the wave's own.
    // (With 64 rows that piece of LDS would be too large; then x is read in operand order.)
    constexpr bool XLDS = MT <= 2;
    constexpr int XR = MT * 4;                      // 16-byte pieces of x per lane and chunk
    __shared__ __attribute__((aligned(16))) uint16_t xs_all[XLDS ? WAVES : 1][XLDS ? MT * 16 * 128 : 8];
    uint16_t* xs = xs_all[XLDS ? wave : 0];
    const int xl_row = lane >> 4, xl_piece = lane & 15;
    // piece p of row r lies at position p ^ (r % 16): the 16 rows a fragment read touches fall
    // into 16 different positions, so into all banks
    auto xslot = [](int row, int piece) { return row * 128 + ((piece ^ (row & 15)) << 3); };
    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int nchunks = (K + SK_CHUNK - 1) / SK_CHUNK;
    const int nfull = K / SK_CHUNK;                    // whole chunks

    // What the epilogue adds to or multiplies with the sums (bias, the residual sum, a norm's
    // weights, the rotation's cosines and sines, the page slot) is asked for now, by the wave
    // that will write the results: the answers arrive with the first chunk, and the epilogue
    // waits for no memory.  Never conditional per lane: a place past the end reads the last one.
    constexpr bool PRE = MT <= 2 && !SWIGLU;        // (wave mt writes row tile mt: thread t of the epilogue is lane t % 64 of wave t / 64)
    float pre_bias[NT][4], pre_res[NT][4], pre_gamma[NT][4], pre_cos[NT][4], pre_sin[NT][4];
    int pre_slot = 0;
    if constexpr (PRE) {
        if (wave < MT) {
            const int m = 16 * wave + (lane & 15) < M ? 16 * wave + (lane & 15) : M - 1;
            if constexpr (ROPE) {
                const bool second = (lane >> 4) >= 2;
                pre_slot = a.slot_map[m];
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        int p = n0 + 8 * nt + 4 * ((lane >> 4) & 1) + r;
                        p = p < nend ? p : nend - 1;
                        const int head = p / half, j = p % half;
                        pre_bias[nt][r] = a.bias ? a.bias[head * a.dh + (second ? half + j : j)] : 0.f;
                        pre_cos[nt][r] = a.cos[(size_t)m * half + j];
                        pre_sin[nt][r] = a.sin[(size_t)m * half + j];
                    }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int n = n0 + 16 * nt + 4 * (lane >> 4) + r;
                        const int nc = n < nend ? n : nend - 1;
                        pre_bias[nt][r] = a.bias ? a.bias[nc] : 0.f;
                        pre_gamma[nt][r] = a.gamma ? a.gamma[nc] : 0.f;
                        if constexpr (sizeof(TO) == 4)
                            pre_res[nt][r] = a.accumulate ? reinterpret_cast<const float*>(a.out)[(size_t)m * N + nc] : 0.f;
                        else pre_res[nt][r] = 0.f;
                    }
            }
        }
    }

    // The memory counter of a wave retires loads in the order they were issued, so waiting for
    // a chunk's x pieces also waits for every load issued before them.  All loads of a chunk (W
    // and x) are therefore issued together, one chunk ahead of their use: when chunk c is
    // multiplied, exactly the loads of chunk c + WAVES are still in flight.  (With 64 rows the x
    // pieces do not fit a second buffer; then a chunk is loaded and used in one go and the other
    // waves of the compute unit cover the latency.)
    constexpr bool AHEAD = MT <= 2;
    constexpr int NBUF = AHEAD ? 2 : 1;
    bf16x8 wbuf[NBUF][NT][4], xbuf[NBUF][XR];
    // No load of a whole chunk is conditional, and none is replaced by zeros: a load under a branch makes the
    // compiler wait for every load in flight at the next use of any (found in this kernel's code: s_waitcnt
    // vmcnt(0) before each multiplication, right behind the loads of the chunk after it, so that nothing was in
    // flight while a wave multiplied), and a value chosen between what was loaded and zero is waited for at once.
    // A row of x past the last is read from the last row (its sums are not written).  Only the last chunk of a K
    // that is no multiple of the chunk has k-values to leave out: it is taken by itself, behind the loop (TAIL).
    auto load_chunk = [&](int c, bf16x8 (*wd)[4], bf16x8* xd, auto tail_tag) {
        constexpr bool TAIL = decltype(tail_tag)::value;
        const int kb = c * SK_CHUNK;
#pragma unroll
        for (int i = 0; i < XR; ++i) {
            int m, kk;
            if constexpr (XLDS) { m = xl_row + 4 * i; kk = kb + 8 * xl_piece; }
            else { m = 16 * (i >> 2) + r16; kk = kb + 8 * g + 32 * (i & 3); }       // operand order: row 16 mt + r16, pieces g + 4 j
            const bf16_t* row = a.x + (size_t)(m < M ? m : M - 1) * K;
            if constexpr (TAIL) xd[i] = kk < K ? *reinterpret_cast<const bf16x8*>(row + kk) : zero;
            else xd[i] = *reinterpret_cast<const bf16x8*>(row + kk);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int kk = kb + 8 * g + 32 * j;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if constexpr (TAIL) wd[nt][j] = kk < K ? *reinterpret_cast<const bf16x8*>(wrow[nt] + kk) : zero;
                else wd[nt][j] = *reinterpret_cast<const bf16x8*>(wrow[nt] + kk);
            }
        }
    };
    auto multiply = [&](bf16x8 (*wa)[4], bf16x8* xd) {
        if constexpr (XLDS) {
            __builtin_amdgcn_wave_barrier();        // a wave's LDS operations run in order; keep the compiler's too
#pragma unroll
            for (int i = 0; i < XR; ++i)
                *reinterpret_cast<bf16x8*>(&xs[xslot(xl_row + 4 * i, xl_piece)]) = xd[i];
            __builtin_amdgcn_wave_barrier();
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            bf16x8 xa[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (XLDS) xa[j] = *reinterpret_cast<const bf16x8*>(&xs[xslot(16 * mt + r16, g + 4 * j)]);
                else xa[j] = xd[4 * mt + j];
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[nt][j], xa[j], acc[mt][nt], 0, 0, 0);
        }
        __builtin_amdgcn_wave_barrier();
    };
    if constexpr (AHEAD) {
        if (wave < nfull) load_chunk(wave, wbuf[0], xbuf[0], std::false_type{});
        // the rows' sums of squares: thread t adds the parts t / 16, t / 16 + G, ... of row t % 16 in
        // that order; the epilogue adds the G sums in theirs.  The loads are issued together, behind
        // those of the first chunk, only as many rounds as there are parts, and never conditional
        // within a round (a part past the end reads the last one).  They are added up behind the
        // loads of the second chunk: the wait for them is the wait the first multiplication has anyway.
        constexpr int G = WAVES * 64 / RP, PER = SK_MAX_PARTS / G;
        float part[PER];
        if (a.row_parts) {
            const int m = threadIdx.x % RP, q = threadIdx.x / RP;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                part[i] = 0.f;
                if (i * G < a.nparts) {
                    const int p = q + i * G;
                    part[i] = a.row_parts[(size_t)(p < a.nparts ? p : a.nparts - 1) * RP + m];
                }
            }
        }
        if (wave + WAVES < nfull) load_chunk(wave + WAVES, wbuf[1], xbuf[1], std::false_type{});
        if (a.row_parts) {
            const int m = threadIdx.x % RP, q = threadIdx.x / RP;
            float mine = 0.f;
#pragma unroll
            for (int i = 0; i < PER; ++i) mine += (q + i * G < a.nparts) ? part[i] : 0.f;
            part_sums[q * RP + m] = mine;
        }
        // (the first turn is written out: its loads of the second chunk stand above, before the parts are added up)
        if (wave < nfull) multiply(wbuf[0], xbuf[0]);
        if (wave + WAVES < nfull) {
            if (wave + 2 * WAVES < nfull) load_chunk(wave + 2 * WAVES, wbuf[0], xbuf[0], std::false_type{});
            multiply(wbuf[1], xbuf[1]);
            // Two chunks a turn (buffer numbers are constants).  Inside the loop nothing about the loads is
            // conditional: where a path with loads and one without meet, the compiler's count of the loads in
            // flight is the smaller one, and the next wait is for all of them.  So the loop runs while both of
            // a turn's loads exist, and the one or two chunks that are left are taken behind it.
            int c = wave + 2 * WAVES;
            for (; c + 2 * WAVES < nfull; c += 2 * WAVES) {
                load_chunk(c + WAVES, wbuf[1], xbuf[1], std::false_type{});
                multiply(wbuf[0], xbuf[0]);
                load_chunk(c + 2 * WAVES, wbuf[0], xbuf[0], std::false_type{});
                multiply(wbuf[1], xbuf[1]);
            }
            if (c < nfull) {
                const bool more = c + WAVES < nfull;
                if (more) load_chunk(c + WAVES, wbuf[1], xbuf[1], std::false_type{});
                multiply(wbuf[0], xbuf[0]);
                if (more) multiply(wbuf[1], xbuf[1]);
            }
        }
    } else {
        for (int c = wave; c < nfull; c += WAVES) {
            load_chunk(c, wbuf[0], xbuf[0], std::false_type{});
            multiply(wbuf[0], xbuf[0]);
        }
    }
    if (nfull < nchunks && wave == nfull % WAVES) {     // the chunk that K ends in
        load_chunk(nfull, wbuf[0], xbuf[0], std::true_type{});
        multiply(wbuf[0], xbuf[0]);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) red[wave][mt * NT + nt][lane] = acc[mt][nt];
    __syncthreads();
    TO* out = (TO*)a.out;
    for (int t = threadIdx.x; t < MT * 64; t += WAVES * 64) {
        const int mt = t >> 6, l = t & 63;
        const int m = 16 * mt + (l & 15);
        if (m >= M) continue;                       // (with ROPE lanes l and l ^ 32 share m: both stay or both go)
        floatx4 s[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            s[nt] = red[0][mt * NT + nt][l];
#pragma unroll
            for (int wv = 1; wv < WAVES; ++wv) {
                const floatx4 o = red[wv][mt * NT + nt][l];
                s[nt][0] += o[0]; s[nt][1] += o[1]; s[nt][2] += o[2]; s[nt][3] += o[3];
            }
        }
        if (AHEAD && a.row_parts) {
            float sq = part_sums[m % RP];
#pragma unroll
            for (int q = 1; q < WAVES * 64 / RP; ++q) sq += part_sums[q * RP + m % RP];
            const float inv = 1.0f / sqrtf(sq / (float)K + a.eps);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) { s[nt][0] *= inv; s[nt][1] *= inv; s[nt][2] *= inv; s[nt][3] *= inv; }
        }
        if constexpr (ROPE) {
            const int dh = a.dh;
            const bool second = (l >> 4) >= 2;                       // this lane holds the pairs' second members
            const int slot = pre_slot;                               // (thread t is lane l of wave mt, which asked for these)
            const int page = slot / a.page_size, in_page = slot - page * a.page_size;
            const bool page_ok = page >= 0 && page < a.num_pages;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int p = n0 + 8 * nt + 4 * ((l >> 4) & 1) + r;  // the pair's number among all heads' pairs
                    float own = s[nt][r] + pre_bias[nt][r];
                    const float other = __shfl_xor(own, 32, 64);
                    if (p >= nend) continue;                         // (lanes l and l ^ 32 share p: the exchange above is done by both)
                    const int head = p / half, j = p - head * half;
                    const int d = second ? half + j : j;
                    const int col = head * dh + d;
                    float v = own;
                    if (head < a.nh + a.nkv) {
                        const float c = pre_cos[nt][r], sn = pre_sin[nt][r];
                        v = second ? own * c + other * sn : own * c - other * sn;
                    }
                    const uint16_t bits = float_to_bf16(v);
                    reinterpret_cast<bf16_t*>(out)[(size_t)m * N + col].bits = bits;
                    if (head >= a.nh && page_ok) {
                        const bool is_k = head < a.nh + a.nkv;
                        const int kvh = is_k ? head - a.nh : head - a.nh - a.nkv;
                        bf16_t* dst = (is_k ? a.kc : a.vc) + (((size_t)page * a.nkv + kvh) * a.page_size + in_page) * dh + d;
                        dst->bits = bits;
                    }
                }
        } else if constexpr (SWIGLU) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int n = n0 + 4 * (l >> 4) + r;
                if (n < nend) {
                    const float gv = s[0][r], uv = s[NT - 1][r];
                    store_from_float(out + (size_t)m * N + n, swiglu_bf16(gv, uv));
                }
            }
        } else {
            if constexpr (sizeof(TO) == 4 && MT <= 2) {
                if (a.xg) {                          // the sum goes out three ways (see SkinnyArgs)
                    float sq = 0.f;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const int n = n0 + 16 * nt + 4 * (l >> 4) + r;
                            if (n < nend) {
                                const size_t idx = (size_t)m * N + n;
                                const float v = (s[nt][r] + pre_bias[nt][r]) + pre_res[nt][r];
                                reinterpret_cast<float*>(out)[idx] = v;
                                a.xg[idx].bits = float_to_bf16(pre_gamma[nt][r] * v);
                                sq += v * v;
                            }
                        }
                    // the four lanes of a row (l, l ^ 16, l ^ 32, l ^ 48: all of them are here, or none)
                    sq += __shfl_xor(sq, 16, 64);
                    sq += __shfl_xor(sq, 32, 64);
                    if ((l >> 4) == 0) a.sq_parts[(size_t)blockIdx.x * RP + m] = sq;
                    continue;
                }
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int n = n0 + 16 * nt + 4 * (l >> 4) + r;
                    if (n >= nend) continue;
                    if constexpr (PRE) store_from_float(out + (size_t)m * N + n, (s[nt][r] + pre_bias[nt][r]) + pre_res[nt][r]);
                    else epilogue_store(out, (size_t)m * N + n, s[nt][r], a.bias, n, a.accumulate);
                }
        }
    }
}

// Compute units of the current device (256 where it cannot be asked).
static int compute_units() {
    static int units[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) { (void)hipGetLastError(); return 256; }
    if (!units[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) { (void)hipGetLastError(); n = 256; }
        units[dev] = n;
    }
    return units[dev];
}

// Up to 16 rows against a matrix of few columns (or rotation pairs: `unit` is 16 columns or 8 pairs a
// tile): a compute unit takes in what its blocks ask for at a rate of its own, far below its share of
// the memory's rate times the number of units, so the time of such a product is that of the unit with the
// most blocks.  Every unit therefore gets one block and every block the same number of columns (at
// most two tiles' worth, at least half a tile's), not whole tiles.
static int balanced_per_block(int total, int unit) {
    const int cu = compute_units();
    int per = (total + cu - 1) / cu;
    per = per < unit / 2 ? unit / 2 : per;
    return per > 2 * unit ? 0 : per;
}

// Many columns in tiles of `unit`: the blocks of a product go round the compute units several times, and
// the units with one block more than the others set the time when the matrix is small.  The columns a
// block takes are therefore cut down until the last round is as full as the others: as many rounds as
// whole tiles would need, and equal shares of the columns within them (at least half a tile's).
static int balanced_round_cols(int total, int unit) {
    const long cu = compute_units();
    const long rounds = (total + unit * cu - 1) / (unit * cu);
    long per = (total + rounds * cu - 1) / (rounds * cu);
    per = per < unit / 2 ? unit / 2 : per;
    return (int)(per > unit ? unit : per);
}

template <bool SWIGLU, typename TO>
static void launch_skinny(SkinnyArgs a, hipStream_t stream) {
    const int M = a.M, N = a.N;
#define LI_SK(MT, NT, WV) gemm_bf16_skinny_kernel<MT, NT, WV, SWIGLU, TO><<<(N + 16 * (SWIGLU ? 1 : NT) - 1) / (16 * (SWIGLU ? 1 : NT)), WV * 64, 0, stream>>>(a)
    if constexpr (SWIGLU) {
        a.cols = balanced_round_cols(N, 16);
        const int blocks = (N + a.cols - 1) / a.cols;
        if (M <= 16) gemm_bf16_skinny_kernel<1, 2, 4, true, TO><<<blocks, 4 * 64, 0, stream>>>(a);
        else if (M <= 32) gemm_bf16_skinny_kernel<2, 2, 4, true, TO><<<blocks, 4 * 64, 0, stream>>>(a);
        else gemm_bf16_skinny_kernel<4, 2, 8, true, TO><<<blocks, 8 * 64, 0, stream>>>(a);
    } else if (N >= 8192) {                                 // many columns: many blocks, two tiles share each piece of x
        if (M <= 16) LI_SK(1, 2, 4); else if (M <= 32) LI_SK(2, 2, 4); else LI_SK(4, 2, 8);
    } else if (M <= 16) {                                   // few columns: a block a compute unit, eight waves split K
        a.cols = balanced_per_block(N, 16);
        const int per = a.cols ? a.cols : 16, blocks = (N + per - 1) / per;
        if (per > 16) gemm_bf16_skinny_kernel<1, 2, 8, false, TO><<<blocks, 8 * 64, 0, stream>>>(a);
        else gemm_bf16_skinny_kernel<1, 1, 8, false, TO><<<blocks, 8 * 64, 0, stream>>>(a);
    } else if (M <= 32) {
        a.cols = balanced_per_block(N, 16);
        const int per = a.cols ? a.cols : 16, blocks = (N + per - 1) / per;
        if (per > 16) gemm_bf16_skinny_kernel<2, 2, 4, false, TO><<<blocks, 4 * 64, 0, stream>>>(a);
        else gemm_bf16_skinny_kernel<2, 1, 4, false, TO><<<blocks, 4 * 64, 0, stream>>>(a);
    } else {
        LI_SK(4, 2, 8);
    }
#undef LI_SK
}

// Few rows (M <= 64), bfloat16, K a multiple of 8.  swiglu: w has 2 N rows ([gate; up]).
extern "C" int li_linear_skinny(const void* x, const void* w, const float* bias, void* out, int M, int N,
                                int K, int out_dtype, int accumulate, int swiglu, hipStream_t stream) {
    if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K % 8)) return LI_ERR_SIZE;
    if (accumulate && out_dtype != LI_F32) return LI_ERR_DTYPE;
    if (swiglu && (bias || accumulate || out_dtype != LI_BF16)) return LI_ERR_DTYPE;
    SkinnyArgs a{(const bf16_t*)x, (const bf16_t*)w, bias, out, M, N, K, accumulate,
                 nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr, nullptr, 0, 0.f};
    if (swiglu) launch_skinny<true, bf16_t>(a, stream);
    else if (out_dtype == LI_BF16) launch_skinny<false, bf16_t>(a, stream);
    else if (out_dtype == LI_F32) launch_skinny<false, float>(a, stream);
    else return LI_ERR_DTYPE;
    return li_launch_status();
}

// The product before an RMS norm that is fused into its neighbours (see SkinnyArgs): out += x w^T + bias
// in float32, xg = bf16(gamma * out), sq_parts[block * R + m] = the block's share of row m's sum of
// squares (R = 16 up to 16 rows, 32 above).  Up to 32 rows.  li_residual_norm_parts(N) is the number of
// blocks, i.e. of parts.
extern "C" int li_residual_norm_parts(int N) {
    int per = 32;                                      // as launch_skinny tiles the columns of few rows
    if (N < 8192) { per = balanced_per_block(N, 16); per = per ? per : 16; }
    return (N + per - 1) / per;
}

extern "C" int li_linear_residual_norm(const void* x, const void* w, const float* bias, float* out, int M, int N,
                                       int K, const float* gamma, void* xg, float* sq_parts, hipStream_t stream) {
    if (M <= 0 || M > 32 || N <= 0 || K <= 0 || (K % 8) || !gamma || !xg || !sq_parts) return LI_ERR_SIZE;
    if (li_residual_norm_parts(N) > SK_MAX_PARTS) return LI_ERR_SIZE;
    SkinnyArgs a{(const bf16_t*)x, (const bf16_t*)w, bias, out, M, N, K, 1,
                 nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, gamma, (bf16_t*)xg, sq_parts, nullptr, 0, 0.f};
    launch_skinny<false, float>(a, stream);
    return li_launch_status();
}

// Between 13 and 64 rows (a large decoding batch) the product is still bound by streaming W, but
// x is too large to be read again by every block of a few columns (every block of the few-row
// kernel reads all of x, and what a compute unit can take in then bounds the product): tiles of
// 64 rows with the loads straight into LDS, and, where the matrix has too few such tiles to fill
// the chip, K cut into parts whose sums go to `work` and are added up in a fixed order, by kernels
// that also do what follows the product (the norm of the new residual sum, the rotary encoding
// and the page write), which the few-row kernel does in its epilogue for up to 16 rows only.
// Measured on the 7B layer sizes, a decode step of 17 / 24 / 32 requests: 4.57 / 4.95 / 5.33 ms
// against 4.90 / 5.33 / 5.84 ms with the few-row kernel up to 32 rows.  Returns -1 when it does
// not take the call.
// The few-row kernel takes up to 16 rows with its fused epilogues.  Up to 12 rows it is the faster one for
// every product but the largest gate/up matrices (li_linear_swiglu); at 13 to 16 rows the tiles with K in
// parts are faster where the matrix is large (at 13 rows the 7B's way back from the feed-forward, 136 MB:
// 29.8 us with its adding-up kernel against 33.5 us; its q/k/v, 33 MB: 11.8 against 9.2 us; the whole step
// of 16 requests at the 7B sizes 4.28 against 4.43 ms, at the 1.5B sizes 2.22 against 1.94 ms).
#define FEW_ROWS_FUSED 12
#define FEW_ROWS_LARGE_BYTES (100l << 20)
// 17 to 32 rows (two tiles of rows a block, the fused epilogues as with one): every block reads all of x, 32
// rows of it now, so the few-row kernel wins only against small matrices, and of those with long rows only
// against the smallest.  Alone, tiles with their adding-up kernel against the few-row kernel at 24 rows: the
// 7B's q/k/v (33 MB) 12.4 / 8.7 us and o 12.3 / 8.5; the 1.5B's q/k/v 11.6 / 6.4, o 11.8 / 6.6, gate/up (55 MB)
// 16.8 / 15.7, down (27 MB, rows of 8,960) 14.2 / 12.9; the 3B's down (45 MB, rows of 11,008) 17.6 / 19.0; the
// 14B's q/k/v (73 MB) 19.7 / 19.5 and o (52 MB, rows of 5,120) 16.9 / 17.6.
#define FEW_ROWS_TWO_TILES 32
#define FEW_ROWS_TWO_TILES_BYTES (56l << 20)
#define FEW_ROWS_TWO_TILES_LONG_K 4096
#define FEW_ROWS_TWO_TILES_LONG_K_BYTES (32l << 20)
#define SWIGLU_TILES_BYTES (160l << 20)      // (see li_linear_swiglu)
extern "C" int li_few_rows_preferred(int M, long N, long K) {
    if (M <= FEW_ROWS_FUSED || (M <= 16 && N * K * 2 < FEW_ROWS_LARGE_BYTES)) return 1;
    if (M > FEW_ROWS_TWO_TILES || K % 8) return 0;
    const long bytes = N * K * 2;
    return bytes <= FEW_ROWS_TWO_TILES_BYTES && (K <= FEW_ROWS_TWO_TILES_LONG_K || bytes <= FEW_ROWS_TWO_TILES_LONG_K_BYTES);
}

static bool mid_rows_take(int M, int N, int K) {
    return !li_few_rows_preferred(M, N, K) && M <= 64;
}

static int linear_mid_rows(const bf16_t* x, const bf16_t* w, const float* bias, void* out, int M, int N,
                           int K, int out_dtype, int accumulate, void* work, long work_bytes,
                           hipStream_t stream) {
    if (!mid_rows_take(M, N, K) || K % 64 || (out_dtype != LI_F32 && out_dtype != LI_BF16)) return -1;
#define LI_MID(BN, NS, TO, dst, b, acc, split) launch_dma<64, BN, 64, NS, false, TO>(x, w, b, (TO*)(dst), M, N, K, acc, stream, split)
    if ((N + 255) / 256 >= 128)
        return out_dtype == LI_F32 ? LI_MID(256, 3, float, out, bias, accumulate, 1) : LI_MID(256, 3, bf16_t, out, bias, accumulate, 1);
    const int tiles = (N + 127) / 128;
    if (tiles >= 128)
        return out_dtype == LI_F32 ? LI_MID(128, 4, float, out, bias, accumulate, 1) : LI_MID(128, 4, bf16_t, out, bias, accumulate, 1);
    int nsplit = 256 / tiles;
    if (nsplit > 8) nsplit = 8;
    if (nsplit > K / 64 / 8) nsplit = K / 64 / 8;              // at least 8 steps a part
    const size_t mn = (size_t)M * N;
    if (nsplit < 2 || !work || (size_t)work_bytes < (size_t)nsplit * mn * sizeof(float)) return -1;
    const int rc = LI_MID(128, 4, float, work, nullptr, 0, nsplit);
    if (rc != LI_OK) return rc;
#undef LI_MID
    const unsigned blocks = (unsigned)((mn + 255) / 256);
    if (out_dtype == LI_F32) splitk_reduce_kernel<float><<<blocks, 256, 0, stream>>>((const float*)work, nsplit, mn, N, bias, (float*)out, accumulate);
    else splitk_reduce_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const float*)work, nsplit, mn, N, bias, (bf16_t*)out, accumulate);
    return li_launch_status();
}

extern "C" long li_linear_work_bytes(int M, int N, int K, int in_dtype);

// The packed q/k/v projection of 17 rows and more where it is cut along K (up to some hundred rows): the kernel that adds the parts up also adds
// the bias, rotates query and key heads (half-split pairs over the whole head, float32 tables
// [M, dh / 2]) and writes keys and values into their page slots, so that the rotation needs no
// kernel of its own.  Thread (row, head, pair): consecutive threads read consecutive sums.
__global__ __launch_bounds__(256) void splitk_reduce_rope_store_kernel(
    const float* __restrict__ part, int nsplit, size_t mn, int N, const float* __restrict__ bias, bf16_t* __restrict__ out,
    const float* __restrict__ cosv, const float* __restrict__ sinv, const int* __restrict__ slot_map,
    bf16_t* __restrict__ kc, bf16_t* __restrict__ vc, int nh, int nkv, int dh, int page_size, int num_pages, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int half = dh / 2, heads = nh + 2 * nkv;
    const int j = (int)(i % half), head = (int)((i / half) % heads), m = (int)(i / ((long)half * heads));
    const size_t i0 = (size_t)m * N + (size_t)head * dh + j, i1 = i0 + half;
    float a = part[i0], b = part[i1];
    for (int sp = 1; sp < nsplit; ++sp) { a += part[(size_t)sp * mn + i0]; b += part[(size_t)sp * mn + i1]; }
    if (bias) { a += bias[head * dh + j]; b += bias[head * dh + j + half]; }
    if (head < nh + nkv) {
        const float c = cosv[(size_t)m * half + j], sn = sinv[(size_t)m * half + j];
        const float ra = __builtin_fmaf(a, c, -__fmul_rn(b, sn)), rb = __builtin_fmaf(b, c, __fmul_rn(a, sn));
        a = ra; b = rb;
    }
    const uint16_t ba = float_to_bf16(a), bb = float_to_bf16(b);
    out[i0].bits = ba;
    out[i1].bits = bb;
    if (head >= nh) {
        const int slot = slot_map[m];
        if (slot < 0 || slot >= num_pages * page_size) return;               // never write outside the pool
        const bool is_k = head < nh + nkv;
        const int kvh = is_k ? head - nh : head - nh - nkv;
        const int page = slot / page_size, in_page = slot - page * page_size;
        bf16_t* dst = (is_k ? kc : vc) + (((size_t)page * nkv + kvh) * page_size + in_page) * dh;
        dst[j].bits = ba;
        dst[j + half].bits = bb;
    }
}

// Returns -1, having done nothing, where li_linear would not cut this product along K.
extern "C" int li_linear_rope_store_parts(const void* x, const void* w, const float* bias, void* out, int M, int K,
                                          const float* cos, const float* sin, const int* slot_map, void* kc, void* vc,
                                          int nh, int nkv, int dh, int page_size, int num_pages,
                                          void* work, long work_bytes, hipStream_t stream) {
    if (M <= 0 || K <= 0 || nh <= 0 || nkv <= 0 || dh <= 0 || dh % 2 || page_size <= 0 || num_pages <= 0 ||
        (long)(nh + 2 * nkv) * dh > 0x7fffffffL)
        return LI_ERR_SIZE;
    const int N = (nh + 2 * nkv) * dh;
    if (li_few_rows_preferred(M, N, K) || K % 64) return -1;
    const long need = li_linear_work_bytes(M, N, K, LI_BF16);            // (0 where li_linear would not cut this product)
    if (need <= 0 || !work || work_bytes < need) return -1;
    const size_t mn = (size_t)M * N;
    const int nsplit = (int)(need / (long)(mn * sizeof(float)));
    const int rc = M <= 64
        ? launch_dma<64, 128, 64, 4, false, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)work, M, N, K, 0, stream, nsplit)
        : launch_dma<128, 128, 64, 4, false, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)work, M, N, K, 0, stream, nsplit);
    if (rc != LI_OK) return rc;
    const long total = (long)M * (nh + 2 * nkv) * (dh / 2);
    splitk_reduce_rope_store_kernel<<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(
        (const float*)work, nsplit, mn, N, bias, (bf16_t*)out, cos, sin, slot_map, (bf16_t*)kc, (bf16_t*)vc,
        nh, nkv, dh, page_size, num_pages, total);
    return li_launch_status();
}

// Estimated time, in microseconds, of x w^T in tiles of bm x bn with K in steps of 64: rounds of tiles
// over the compute units x (steps x the longer of a step's MFMAs and a step's loads + a tile's start
// and end).  A compute unit multiplies at about 4 TFLOP/s under the chip's power limit, `speed` of
// that in this tiling (small tiles spend more of their time between steps; with four waves one
// above the other the LDS reads take nearly as long as the MFMAs), and takes in about 50 GB/s, rows
// of x that other units read too included: with few rows of x a tile waits for its part of w, and
// wide tiles read x less often.  A last round that does not fill the chip counts for less than a
// whole one: the units that run clock higher.  Fitted to measurements of all tilings at 128 to
// 8,192 rows of the 1.5B and 7B layer shapes: the tiling it takes is within 4 % of the best one
// there, but for the 7B's way back from the feed-forward at 4,096 rows and more (10 %).
static double tile_cost(int bm, int bn, double speed, int M, int N, int K) {
    const long tiles = (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const int cu = compute_units();
    const double filled = (double)tiles / cu, whole = (double)((tiles + cu - 1) / cu);
    const double rounds = filled + 0.4 * (whole - filled);
    const double mfma_us = (double)bm * bn * 64 * 2 / (4.0e6 * speed), load_us = (double)(bm + bn) * 128 / 50.0e3;
    return rounds * ((K / 64) * (mfma_us > load_us ? mfma_us : load_us) + 2.0);
}

// More than 64 rows but so few 128 x 128 tiles that half of the compute units would idle (a narrow
// matrix with a long K, like the feed-forward's way back at 128 to 512 rows): K is cut into parts
// here too.  Returns the number of parts, 1 for none.
static int split_parts_many_rows(int M, int N, int K) {
    if (M <= 64 || K % 64) return 1;
    const long tiles = (long)((M + 127) / 128) * ((N + 127) / 128);
    if (tiles >= 128) return 1;
    int nsplit = (int)(256 / tiles);
    if (nsplit > 8) nsplit = 8;
    if (nsplit > K / 64 / 8) nsplit = K / 64 / 8;              // at least 8 steps a part
    return nsplit < 2 ? 1 : nsplit;
}

// Bytes of workspace with which li_linear cuts this product along K (0: it would not).
extern "C" long li_linear_work_bytes(int M, int N, int K, int in_dtype) {
    if (in_dtype != LI_BF16 || N <= 0 || K <= 0 || K % 64 || li_few_rows_preferred(M, N, K)) return 0;
    int nsplit = 1;
    if (M <= 64) {
        const int tiles = (N + 127) / 128;
        if (tiles < 128) {
            nsplit = 256 / tiles;
            if (nsplit > 8) nsplit = 8;
            if (nsplit > K / 64 / 8) nsplit = K / 64 / 8;
        }
    } else {
        nsplit = split_parts_many_rows(M, N, K);
    }
    return nsplit < 2 ? 0 : (long)nsplit * M * N * (long)sizeof(float);
}

// out += x w^T + bias (float32 out: the residual sum) and xn = the RMS norm of the new out with weights
// gamma, where li_linear would cut K into parts anyway: the kernel that adds the parts up then has
// whole rows in its hands.  xn is bfloat16 (xn_dtype LI_BF16) or float32.  Returns -1, having done
// nothing, where the product is not cut (the caller then multiplies and norms in two calls).
extern "C" int li_linear_then_norm(const void* x, const void* w, const float* bias, float* out, int M, int N, int K,
                                   void* work, long work_bytes, const float* gamma, float eps, void* xn,
                                   int xn_dtype, hipStream_t stream) {
    if (N <= 0 || K <= 0 || (K % 64) || li_few_rows_preferred(M, N, K) || !gamma || !xn || eps < 0.f) return -1;
    if (N > REDUCE_NORM_NT * REDUCE_NORM_PER || (xn_dtype != LI_BF16 && xn_dtype != LI_F32)) return -1;
    const long need = li_linear_work_bytes(M, N, K, LI_BF16);
    if (need <= 0 || !work || work_bytes < need) return -1;
    const size_t mn = (size_t)M * N;
    const int nsplit = (int)(need / (long)(mn * sizeof(float)));
    if (nsplit > 8) return -1;                      // (the adding-up kernel takes up to 8 parts)
    const int rc = M <= 64
        ? launch_dma<64, 128, 64, 4, false, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)work, M, N, K, 0, stream, nsplit)
        : launch_dma<128, 128, 64, 4, false, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)work, M, N, K, 0, stream, nsplit);
    if (rc != LI_OK) return rc;
    if (xn_dtype == LI_BF16)
        splitk_reduce_norm_kernel<bf16_t, REDUCE_NORM_NT, REDUCE_NORM_PER><<<M, REDUCE_NORM_NT, 0, stream>>>(
            (const float*)work, nsplit, mn, N, bias, out, gamma, eps, (bf16_t*)xn);
    else
        splitk_reduce_norm_kernel<float, REDUCE_NORM_NT, REDUCE_NORM_PER><<<M, REDUCE_NORM_NT, 0, stream>>>(
            (const float*)work, nsplit, mn, N, bias, out, gamma, eps, (float*)xn);
    return li_launch_status();
}

// `work` (may be null): device memory of work_bytes for the partial sums of a product cut along K.
// Rows of the smallest tile that a product of more than 64 rows is cut into in this dtype: a
// product of a few rows more than a multiple of it pays for a whole tile more.  Whoever cuts work
// into steps (a scheduler) asks here instead of knowing the kernels' tilings.
extern "C" int li_linear_row_tile(int in_dtype) { return in_dtype == LI_F32 ? F32_BM : BF_BM; }

extern "C" int li_linear(const void* x, const void* w, const float* bias, void* out, int M, int N,
                         int K, int in_dtype, int out_dtype, int accumulate, void* work, long work_bytes,
                         hipStream_t stream) {
    if (M <= 0 || N <= 0 || K <= 0) return LI_ERR_SIZE;
    if (accumulate && out_dtype != LI_F32) return LI_ERR_DTYPE;
    if (in_dtype == LI_F32) {
        if (out_dtype != LI_F32) return LI_ERR_DTYPE;
        if (M <= F32_ROWS_MAX && K % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0)
            return launch_f32_rows((const float*)x, (const float*)w, bias, (float*)out, M, N, K, accumulate, stream);
        if (K % 4 == 0 && (((uintptr_t)x | (uintptr_t)w) & 15) == 0) {       // the matrix cores' float32 form
            dim3 tiles((N + F32M_BN - 1) / F32M_BN, (M + F32M_BM - 1) / F32M_BM);
            if (tiles.y > 65535) return LI_ERR_SIZE;
            gemm_f32_mfma_kernel<<<tiles, 256, 0, stream>>>((const float*)x, (const float*)w, bias, (float*)out, M, N, K, accumulate);
            return li_launch_status();
        }
        if (M >= 2 * F32B_BM && N >= F32B_BN) {              // enough of both for the large tile to fill the chip
            dim3 big((N + F32B_BN - 1) / F32B_BN, (M + F32B_BM - 1) / F32B_BM);
            if (big.y > 65535) return LI_ERR_SIZE;
            gemm_f32_big_kernel<<<big, 256, 0, stream>>>((const float*)x, (const float*)w, bias, (float*)out, M, N, K, accumulate);
            return li_launch_status();
        }
        dim3 grid((N + F32_BN - 1) / F32_BN, (M + F32_BM - 1) / F32_BM);
        if (grid.y > 65535) return LI_ERR_SIZE;
        gemm_f32_kernel<<<grid, 256, 0, stream>>>((const float*)x, (const float*)w, bias, (float*)out, M, N, K, accumulate);
    } else if (in_dtype == LI_BF16) {
        dim3 grid((N + BF_BN - 1) / BF_BN, (M + BF_BM - 1) / BF_BM);
        if (grid.y > 65535) return LI_ERR_SIZE;
        const bool aligned = (K % 8) == 0;
        if (aligned && M <= 64) {
            const int rc = linear_mid_rows((const bf16_t*)x, (const bf16_t*)w, bias, out, M, N, K, out_dtype,
                                           accumulate, work, work_bytes, stream);
            if (rc >= 0) return rc;
            return li_linear_skinny(x, w, bias, out, M, N, K, out_dtype, accumulate, 0, stream);
        }
        if (aligned && M > 64) {
#define LI_BIG(BM, BN, BK) (out_dtype == LI_F32 ? launch_big<BM, BN, BK, float>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)out, M, N, K, accumulate, stream) \
                                            : launch_big<BM, BN, BK, bf16_t>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)out, M, N, K, accumulate, stream))
            if (out_dtype != LI_F32 && out_dtype != LI_BF16) return LI_ERR_DTYPE;
#define LI_DMA(BM, BN, BK, NS) (out_dtype == LI_F32 ? launch_dma<BM, BN, BK, NS, false, float>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)out, M, N, K, accumulate, stream) \
                                               : launch_dma<BM, BN, BK, NS, false, bf16_t>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)out, M, N, K, accumulate, stream))
            if (K % 64 == 0) {
                const int nsplit = split_parts_many_rows(M, N, K);
                const size_t mn = (size_t)M * N;
                if (nsplit > 1 && work && (size_t)work_bytes >= (size_t)nsplit * mn * sizeof(float)) {
                    const int rc = launch_dma<128, 128, 64, 4, false, float>((const bf16_t*)x, (const bf16_t*)w, nullptr, (float*)work,
                                                                              M, N, K, 0, stream, nsplit);
                    if (rc != LI_OK) return rc;
                    const unsigned blocks = (unsigned)((mn + 255) / 256);
                    if (out_dtype == LI_F32) splitk_reduce_kernel<float><<<blocks, 256, 0, stream>>>((const float*)work, nsplit, mn, N, bias, (float*)out, accumulate);
                    else splitk_reduce_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const float*)work, nsplit, mn, N, bias, (bf16_t*)out, accumulate);
                    return li_launch_status();
                }
#define LI_DMA4(BM, BN, BK, NS) (out_dtype == LI_F32 ? launch_dma<BM, BN, BK, NS, false, float, 4>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)out, M, N, K, accumulate, stream) \
                                                : launch_dma<BM, BN, BK, NS, false, bf16_t, 4>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)out, M, N, K, accumulate, stream))
                // Seven tilings; the one with the least estimated time is taken (tile_cost).  The two with four
                // waves one above the other take any multiple of 32 columns: 224 or 288 columns cut 3,584 or
                // 4,608 into exactly as many tiles as 2,048 rows need to give every compute unit one.
                static const struct { int bm, bn; double speed; } shape[7] = {{256, 256, 1.0}, {256, 192, 0.95}, {256, 128, 1.0}, {192, 128, 0.95},
                                                                                {128, 128, 0.8}, {128, 224, 0.9}, {128, 288, 0.9}};
                int pick = 0;
                double best = 0.0;
                for (int i = 0; i < 7; ++i) {
                    const double c = tile_cost(shape[i].bm, shape[i].bn, shape[i].speed, M, N, K);
                    if (i == 0 || c < best) { best = c; pick = i; }
                }
                switch (pick) {
                case 0: return LI_DMA(256, 256, 64, 2);
                case 1: return LI_DMA(256, 192, 64, 2);
                case 2: return LI_DMA(256, 128, 64, 3);
                case 3: return LI_DMA(192, 128, 64, 3);
                case 4: return LI_DMA(128, 128, 64, 4);
                case 5: return LI_DMA4(128, 224, 64, 3);
                default: return LI_DMA4(128, 288, 64, 3);
                }
#undef LI_DMA4
            }
#undef LI_DMA
            return LI_BIG(128, 128, 64);             // K not a multiple of 64: loads staged in registers
#undef LI_BIG
        }
#define LI_GEMM(TO, AL) gemm_bf16_kernel<TO, AL><<<grid, 256, 0, stream>>>((const bf16_t*)x, (const bf16_t*)w, bias, (TO*)out, M, N, K, accumulate)
        if (out_dtype == LI_F32) { if (aligned) LI_GEMM(float, true); else LI_GEMM(float, false); }
        else if (out_dtype == LI_BF16) { if (aligned) LI_GEMM(bf16_t, true); else LI_GEMM(bf16_t, false); }
        else return LI_ERR_DTYPE;
#undef LI_GEMM
    } else return LI_ERR_DTYPE;
    return li_launch_status();
}

// The same in float32 for up to 64 rows (K a multiple of 4): the few-row product on the float32 matrix cores with
// the activation in its epilogue.
extern "C" int li_linear_swiglu_f32(const float* x, const float* w, float* out, int M, int I, int K, hipStream_t stream) {
    if (M <= 0 || M > F32_ROWS_MAX || I <= 0 || K <= 0 || K % 4 || I > 0x3fffffff) return LI_ERR_SIZE;
    if ((((uintptr_t)x | (uintptr_t)w) & 15) != 0) return LI_ERR_SIZE;
    return launch_f32_rows(x, w, nullptr, out, M, I, K, 0, stream, true);
}

// out[m, n] = up * gate / (1 + exp(-gate)) with [gate, up] = x w^T, w = [gate; up] of I rows each:
// the activation as the product's epilogue, so the 2 I columns never go to memory.  bfloat16;
// K a multiple of 8 for up to 64 rows, a multiple of 64 above.
// row_parts (may be null): x is the xg of li_linear_residual_norm and these are its sq_parts, nparts of
// them; every row's result is that of the RMS norm with eps (up to 16 rows).
extern "C" int li_linear_swiglu(const void* x, const void* w, void* out, int M, int I, int K,
                                const float* row_parts, int nparts, float eps, hipStream_t stream) {
    if (M <= 0 || I <= 0 || K <= 0 || I > 0x3fffffff) return LI_ERR_SIZE;
    const int N = 2 * I;
    if (row_parts && (M > 32 || (K % 8) || nparts <= 0 || nparts > SK_MAX_PARTS || eps < 0.f)) return LI_ERR_SIZE;
    // Up to 64 rows the product waits for w.  From 17 rows on (more than the few-row kernel's fused form takes),
    // and from 13 on where the matrix is large (li_few_rows_preferred: the 7B's at 16 rows 51.8 against 59.6 us),
    // it goes to tiles of 64 rows if the matrix has tiles enough to fill the chip: the width with the least
    // estimated time (a compute unit takes in only so much: more units, each with a narrower tile, stream
    // more, until the tiles no longer fit one round).
    // Below that the few-row kernel, but for a large matrix of rows that are not too long whose tiles fit ONE
    // round over the compute units: there the tiles' loads straight into LDS stream w at the rate of a kernel
    // that only reads (7B sizes, 272 MB: 48.8 us; the few-row kernel 49 to 54 us at 1 to 12 rows), and the
    // rows' factors of a fused RMS norm are applied in the tile kernel's epilogue.  Measured on one machine in
    // turn, whole decode steps: 7B sizes 3.34 -> 3.32 ms at 1 request, 3.72 -> 3.62 at 8, 4.06 -> 3.90 at 12;
    // 14B 6.5 -> 6.57 / 7.66 -> 7.45 / 8.49 -> 8.09; 32B (566 MB) 13.98 -> 13.05 at 1.  Not taken where it
    // loses: small matrices (3B's 90 MB, 1.5B's 55 MB: steps 4-5 % longer), rows of 8,192 (72B sizes 173
    // against 181 us; 28,672 x 8,192: 86 against 96), or no width whose tiles fit one round (73,728 x 4,096:
    // 109 against 130 us).
    const int cu = compute_units();
    const bool few = li_few_rows_preferred(M, N, K);
    // (since the few-row kernel's waves have their next chunk in flight while they multiply, it is the faster one
    // again where the rows are few: every one of its blocks reads all of x, the tiles read x once a tile.  7B sizes
    // at 1 / 8 / 12 / 16 rows: 46.4 / 47.6 / 49.5 / 52.0 us against the tiles' 49.0 / 48.6 / 49.5 / 50.2; 14B sizes
    // at 4 / 8: 48.8 / 50.9 against 50.4 / 50.1; 32B sizes at 1 / 4: 97.4 / 100.3 against 97.4 / 97.2: the tiles
    // from rows x matrix bytes of 2.2 GB on)
    const bool stream_tiles = (long)N * K * 2 >= SWIGLU_TILES_BYTES && K <= 6144 && (double)M * N * K * 2 > 2.2e9;
    if (M <= 64 && K % 64 == 0 && (!few || stream_tiles)) {
        const int widths[3] = {256, 192, 128};
        int pick = -1;
        double best = 0.0;
        for (int i = 0; i < 3; ++i) {
            const int tiles = (N + widths[i] - 1) / widths[i];
            if (tiles < 128) continue;                                   // too few tiles: the few-row kernel
            if (few && tiles > cu) continue;                             // (few rows: one round only, see above)
            const double c = tile_cost(64, widths[i], 1.0, M, N, K);
            if (pick < 0 || c < best) { best = c; pick = i; }
        }
#define LI_SW64(BN, NS) launch_dma<64, BN, 64, NS, true, bf16_t>((const bf16_t*)x, (const bf16_t*)w, nullptr, (bf16_t*)out, M, N, K, 0, stream, 1, row_parts, nparts, eps)
        if (pick == 0) return LI_SW64(256, 3);
        if (pick == 1) return LI_SW64(192, 4);
        if (pick == 2) return LI_SW64(128, 4);
#undef LI_SW64
    }
    if (row_parts) {
        SkinnyArgs a{(const bf16_t*)x, (const bf16_t*)w, nullptr, out, M, I, K, 0,
                     nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, nullptr, nullptr, nullptr, row_parts, nparts, eps};
        launch_skinny<true, bf16_t>(a, stream);
        return li_launch_status();
    }
    if (M <= 64) return li_linear_skinny(x, w, nullptr, out, M, I, K, LI_BF16, 0, 1, stream);
    if (K % 64) return LI_ERR_SIZE;
#define LI_DMA(BM, BN, BK, NS, WLM) launch_dma<BM, BN, BK, NS, true, bf16_t, WLM>((const bf16_t*)x, (const bf16_t*)w, nullptr, (bf16_t*)out, M, N, K, 0, stream)
    // (a tile's columns are gate and up columns in turn, 32 of each: its width is a multiple of 64)
    // (128 x 320: 160 gate columns in one wave, their ups in the wave beside it; for portions of a few hundred rows,
    // where no other width comes near whole rounds of the compute units: 512 rows against the 1.5B's 17,920
    // columns are 224 tiles of it, one round: 45.2 -> 38.7 us.  From four rows of tiles on: with two, 256 rows
    // against the 7B's 37,888 columns, it measured 107 us against the 101 us of 148 tiles of 256 x 256, which
    // read w once)
    static const struct { int bm, bn; double speed; } shape[6] = {{256, 256, 1.0}, {256, 128, 1.0}, {128, 256, 1.0}, {128, 128, 0.8}, {128, 192, 0.9},
                                                                  {128, 320, 0.9}};
    int pick = 0;
    double best = 0.0;
    for (int i = 0; i < 6; ++i) {
        if (i == 5 && M <= 3 * 128) continue;
        const double c = tile_cost(shape[i].bm, shape[i].bn, shape[i].speed, M, N, K);
        if (i == 0 || c < best) { best = c; pick = i; }
    }
    switch (pick) {
    case 0: return LI_DMA(256, 256, 64, 2, 2);
    case 1: return LI_DMA(256, 128, 64, 3, 2);
    case 2: return LI_DMA(128, 256, 64, 3, 2);
    case 3: return LI_DMA(128, 128, 64, 4, 2);
    case 4: return LI_DMA(128, 192, 64, 3, 4);
    default: return LI_DMA(128, 320, 64, 2, 2);
    }
#undef LI_DMA
}

// The packed q/k/v projection of up to 32 rows with the half-split rotary encoding of query and key
// heads and the write of keys and values into their page slots as its epilogue (see ROPE above).
// w [(nh + 2 nkv) dh, K] bfloat16, bias float32 or null, out [M, (nh + 2 nkv) dh] bfloat16 (rotated
// q, rotated k, v), cos/sin float32 [M, dh / 2], slot_map int32 [M], kc/vc the cache layer.
// row_parts, nparts, eps: as for li_linear_swiglu.
extern "C" int li_linear_rope_store(const void* x, const void* w, const float* bias, void* out, int M, int K,
                                    const float* cos, const float* sin, const int* slot_map, void* kc, void* vc,
                                    int nh, int nkv, int dh, int page_size, int num_pages,
                                    const float* row_parts, int nparts, float eps, hipStream_t stream) {
    if (M <= 0 || M > 32 || K <= 0 || K % 8 || nh <= 0 || nkv <= 0 || dh <= 0 || dh % 16 || page_size <= 0 ||
        num_pages <= 0 || (long)(nh + 2 * nkv) * dh > 0x7fffffffL)
        return LI_ERR_SIZE;
    const int N = (nh + 2 * nkv) * dh;
    SkinnyArgs a{(const bf16_t*)x, (const bf16_t*)w, bias, out, M, N, K, 0, cos, sin, slot_map,
                 (bf16_t*)kc, (bf16_t*)vc, nh, nkv, dh, page_size, num_pages,
                 nullptr, nullptr, nullptr, row_parts, row_parts ? nparts : 0, eps};
    if (row_parts && (nparts <= 0 || nparts > SK_MAX_PARTS || eps < 0.f)) return LI_ERR_SIZE;
    const int pairs = N / 2;
    a.cols = balanced_per_block(pairs, 8);
    const int per = a.cols ? a.cols : 8, blocks = (pairs + per - 1) / per;
    if (M <= 16) {
        if (per > 8) gemm_bf16_skinny_kernel<1, 2, 8, false, bf16_t, true><<<blocks, 8 * 64, 0, stream>>>(a);
        else gemm_bf16_skinny_kernel<1, 1, 8, false, bf16_t, true><<<blocks, 8 * 64, 0, stream>>>(a);
    } else {                                            // (two tiles of rows: four waves, as for the plain product)
        if (per > 8) gemm_bf16_skinny_kernel<2, 2, 4, false, bf16_t, true><<<blocks, 4 * 64, 0, stream>>>(a);
        else gemm_bf16_skinny_kernel<2, 1, 4, false, bf16_t, true><<<blocks, 4 * 64, 0, stream>>>(a);
    }
    return li_launch_status();
}
