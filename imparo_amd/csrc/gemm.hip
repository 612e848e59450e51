// Y[m, n] = X[m, k] . W[n, k]^T with float32 accumulation.
//
// float32: a register-tiled FMA kernel; every output element sums its products
// in the order k = 0, 1, 2, ... whatever the tile it falls in, so a row's
// result does not depend on how many other rows are in the batch.
// bfloat16: MFMA kernels, a 128x128 LDS-tiled one for many rows and a
// weight-streaming one with the K range split over the waves of a block for
// few rows (decode).
#include "common.h"

#include <algorithm>
#include "api.h"
#include "rows.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

union Frag8 {
    uint4 u;
    bf16x8 v;
};

#define EPI_NONE 0
#define EPI_SWIGLU 1   // weight rows interleaved gate, up, gate, up...: out[m, j] = silu(y[m, 2j]) * y[m, 2j+1]
#define EPI_ADD 2      // float32 out only: Y += y, what Y holds being read where the result is stored

__device__ __forceinline__ float silu_mul_f(float g, float u) { return g / (1.0f + expf(-g)) * u; }
// The same with the hardware's exp2 and reciprocal (an ulp each) for the bfloat16 kernels: the exact
// division and exponential cost some thirty instructions per output, ten microseconds per 256x256 tile
__device__ __forceinline__ float silu_mul_fast(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * g)) * u;
}

__device__ __forceinline__ uint4 zero_if(bool out, uint4 v) {
    return make_uint4(out ? 0u : v.x, out ? 0u : v.y, out ? 0u : v.z, out ? 0u : v.w);
}

// ------------------------------------------------------------------ float32
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename TOut>
__global__ __launch_bounds__(256) void k_gemm_f32(const float* __restrict__ X, const float* __restrict__ W,
                                                  const float* __restrict__ bias, TOut* __restrict__ Y,
                                                  int M, int N, int K, int epilogue) {
    __shared__ float As[F32_BK][F32_BM + 4];
    __shared__ float Bs[F32_BK][F32_BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int m0 = blockIdx.y * F32_BM, n0 = blockIdx.x * F32_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += F32_BK) {
        // 64 rows x 16 k per operand = 1024 values, 4 per thread
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = tid + j * 256;
            const int r = e / F32_BK, kk = e % F32_BK;
            const int k = k0 + kk;
            const int ma = m0 + r, nb = n0 + r;
            As[kk][r] = (ma < M && k < K) ? X[(size_t)ma * K + k] : 0.f;
            Bs[kk][r] = (nb < N && k < K) ? W[(size_t)nb * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < F32_BK; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        if (bias) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + tx * 4 + j;
                if (n < N) acc[i][j] += bias[n];
            }
        }
        if (epilogue == EPI_SWIGLU) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
                const int n = n0 + tx * 4 + j;
                if (n + 1 < N) store_f32<TOut>(Y, (size_t)m * (N / 2) + n / 2, silu_mul_f(acc[i][j], acc[i][j + 1]));
            }
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) store_f32<TOut>(Y, (size_t)m * N + n, acc[i][j]);
        }
    }
}

// The same sums for at most 16 rows (a decode step in the float32 engine): the tile above would
// leave three quarters of its rows empty and, with a weight of few rows, most CUs idle. A block
// takes 32 weight rows; thread (row, pair of weight rows) adds k = 0, 1, 2, ... exactly as the
// tile kernel does, so a token's sums are the same bits whichever kernel its batch met. The next
// chunk of K is asked for before the current one is multiplied.
#define F32R_BN 32
#define F32R_BK 64
template <typename TOut>
__global__ __launch_bounds__(256) void k_gemm_f32_rows(const float* __restrict__ X, const float* __restrict__ W,
                                                       const float* __restrict__ bias, TOut* __restrict__ Y,
                                                       int M, int N, int K, int epilogue) {
    __shared__ float Ws[F32R_BK][F32R_BN + 1];
    __shared__ float Xs[F32R_BK][16 + 1];
    const int tid = threadIdx.x;
    const int tx = tid % 16, ty = tid / 16;
    const int n0 = blockIdx.x * F32R_BN;
    float acc0 = 0.f, acc1 = 0.f;
    float wr[8], xr[4];
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {                    // 32 weight rows x 64 k, a row's 64 values side by side
            const int e = tid + j * 256;
            const int r = e / F32R_BK, k = k0 + e % F32R_BK;
            wr[j] = (n0 + r < N && k < K) ? W[(size_t)(n0 + r) * K + k] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {                    // 16 activation rows x 64 k
            const int e = tid + j * 256;
            const int r = e / F32R_BK, k = k0 + e % F32R_BK;
            xr[j] = (r < M && k < K) ? X[(size_t)r * K + k] : 0.f;
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += F32R_BK) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int e = tid + j * 256;
            Ws[e % F32R_BK][e / F32R_BK] = wr[j];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int e = tid + j * 256;
            Xs[e % F32R_BK][e / F32R_BK] = xr[j];
        }
        __syncthreads();
        fetch(k0 + F32R_BK);                             // (past the end: nothing is read, zeros)
#pragma unroll 16
        for (int kk = 0; kk < F32R_BK; ++kk) {
            const float a = Xs[kk][ty];
            acc0 = fmaf(a, Ws[kk][2 * tx], acc0);
            acc1 = fmaf(a, Ws[kk][2 * tx + 1], acc1);
        }
        __syncthreads();
    }
    const int m = ty, n = n0 + 2 * tx;
    if (m >= M) return;
    if (bias) {
        if (n < N) acc0 += bias[n];
        if (n + 1 < N) acc1 += bias[n + 1];
    }
    if (epilogue == EPI_SWIGLU) {
        if (n + 1 < N) store_f32<TOut>(Y, (size_t)m * (N / 2) + n / 2, silu_mul_f(acc0, acc1));
        return;
    }
    if (n < N) store_f32<TOut>(Y, (size_t)m * N + n, acc0);
    if (n + 1 < N) store_f32<TOut>(Y, (size_t)m * N + n + 1, acc1);
}

// ------------------------------------------------------------------ bfloat16, many rows
// 128x128 output tile per block of four waves (2x2, 64x64 each as 2x2 MFMA
// tiles of 32x32x16), K in steps of 64. Global loads run three K-steps ahead
// in registers, LDS is double-buffered, one barrier per K-step. Blocks are
// numbered so that those sharing rows of X and W sit on the same XCD (blocks
// go to the 8 XCDs round-robin, each XCD has its own L2).
#define BG_BM 128
#define BG_BN 128
#define BG_BK 64
#define BG_LD 72   // LDS row stride in elements: 144 bytes keeps 16-byte reads of 16 rows on distinct banks
#define BG_PF 3    // K-steps in flight
#define BG_GROUP_M 8
#define N_XCD 8

template <typename TOut>
__global__ __launch_bounds__(256, 2) void k_gemm_bf16_tile(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                           const float* __restrict__ bias, TOut* __restrict__ Y,
                                                           int M, int N, int K_all, int tiles_m, int tiles_n,
                                                           int epilogue, int k_per) {
    __shared__ __attribute__((aligned(16))) bf16_t As[2][BG_BM * BG_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[2][BG_BN * BG_LD];
    // slices of K (gridDim.y > 1): block (x, y) sums K range [y * k_per, (y+1) * k_per) into Y + y * M * N
    const int k_lo = blockIdx.y * k_per;
    const int K = min(K_all, k_lo + k_per) - k_lo;
    X += k_lo;
    W += k_lo;
    Y += (size_t)blockIdx.y * M * N;
    if (blockIdx.y > 0) bias = nullptr;
    // block id -> tile: consecutive logical ids on one XCD, grouped over 8 tile rows
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + N_XCD - 1) / N_XCD;
    const int logical = (blockIdx.x % N_XCD) * per_xcd + blockIdx.x / N_XCD;
    if (logical >= total) return;
    const int per_group = BG_GROUP_M * tiles_n;
    const int first_m = (logical / per_group) * BG_GROUP_M;
    const int gsize = min(tiles_m - first_m, BG_GROUP_M);
    const int tile_m = first_m + (logical % per_group) % gsize;
    const int tile_n = (logical % per_group) / gsize;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = tile_m * BG_BM, n0 = tile_n * BG_BN;

    // this thread's four 16-byte pieces of each operand tile: rows tid/8 + 32 j, columns (tid%8)*8
    const int kc8 = (tid & 7) * 8;
    const bf16_t* pa[4];
    const bf16_t* pb[4];
    int lds_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = (tid >> 3) + 32 * j;
        pa[j] = X + (size_t)min(m0 + row, M - 1) * K_all;
        pb[j] = W + (size_t)min(n0 + row, N - 1) * K_all;
        lds_off[j] = row * BG_LD + kc8;
    }
    const int nk = (K + BG_BK - 1) / BG_BK;
    // three register sets, one per K-step in flight (named apart so that they stay in registers)
    uint4 a0[4], b0[4], a1[4], b1[4], a2[4], b2[4];

    // No load sits under a branch (the compiler would wait for every load in flight at the
    // next use of any): addresses are clamped into the row, a step past the end reads the
    // last one again, and what a cut step reads at or beyond K is zeroed on its way to LDS.
    auto fetch = [&](int kt, uint4 (&a)[4], uint4 (&b)[4]) {
        const int k = min(min(kt, nk - 1) * BG_BK + kc8, K - 8);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            a[j] = *reinterpret_cast<const uint4*>(pa[j] + k);
            b[j] = *reinterpret_cast<const uint4*>(pb[j] + k);
        }
    };
    auto stash = [&](int kt, int buf, uint4 (&a)[4], uint4 (&b)[4]) {
        if ((kt + 1) * BG_BK > K) {                               // only a cut step, or one past the end
            const bool out = kt * BG_BK + kc8 >= K;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                a[j] = zero_if(out, a[j]);
                b[j] = zero_if(out, b[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint4*>(&As[buf][lds_off[j]]) = a[j];
            *reinterpret_cast<uint4*>(&Bs[buf][lds_off[j]]) = b[j];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
    const int a_base = (wm * 64 + frag_row) * BG_LD + frag_k;
    const int b_base = (wn * 64 + frag_row) * BG_LD + frag_k;
    // The operand fragments of K-sub-step ks+1 are read from LDS while the products of sub-step ks
    // run: without that every sub-step waits a full LDS latency before its first product.
    auto read_frags = [&](int buf, int ks, Frag8 (&fa)[2], Frag8 (&fb)[2]) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
            fa[ii].u = *reinterpret_cast<const uint4*>(&As[buf][a_base + ii * 32 * BG_LD + ks * 16]);
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
            fb[jj].u = *reinterpret_cast<const uint4*>(&Bs[buf][b_base + jj * 32 * BG_LD + ks * 16]);
    };
    auto multiply = [&](const Frag8 (&fa)[2], const Frag8 (&fb)[2]) {
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
                acc[ii][jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ii].v, fb[jj].v, acc[ii][jj], 0, 0, 0);
    };
    auto compute = [&](int buf) {
        Frag8 fa0[2], fb0[2], fa1[2], fb1[2];
        read_frags(buf, 0, fa0, fb0);
        read_frags(buf, 1, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(fa0, fb0);
        read_frags(buf, 2, fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(fa1, fb1);
        read_frags(buf, 3, fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(fa1, fb1);
    };
    // K-step i: the next step's tile goes from its registers to LDS, those registers
    // take the load of step i+1+BG_PF, then step i is multiplied out of LDS
    auto step = [&](int i, uint4 (&na)[4], uint4 (&nb)[4]) {
        const int buf = i & 1;
        stash(i + 1, buf ^ 1, na, nb);
        fetch(i + 1 + BG_PF, na, nb);
        compute(buf);
        __syncthreads();
    };

    fetch(0, a0, b0);
    fetch(1, a1, b1);
    fetch(2, a2, b2);
    stash(0, 0, a0, b0);
    fetch(3, a0, b0);
    __syncthreads();
    int kt = 0;
    for (; kt + BG_PF <= nk; kt += BG_PF) {        // whole rounds of the three sets, free of branches
        step(kt, a1, b1);
        step(kt + 1, a2, b2);
        step(kt + 2, a0, b0);
    }
    if (kt < nk) {
        step(kt, a1, b1);
        if (kt + 1 < nk) step(kt + 1, a2, b2);
    }
    // D layout of the 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
            const float bn = (bias && n < N) ? bias[n] : 0.f;
            if (epilogue == EPI_SWIGLU) {
                // gate and up of one output sit in neighbouring lanes (n even, n odd)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float mine = acc[i][j][r] + bn;
                    const float other = __shfl_xor(mine, 1, WAVE);
                    const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                    if (!(lane & 1) && n + 1 < N && m < M)
                        store_f32<TOut>(Y, (size_t)m * (N / 2) + n / 2, silu_mul_fast(mine, other));
                }
                continue;
            }
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (m < M) store_f32<TOut>(Y, (size_t)m * N + n, acc[i][j][r] + bn);
            }
        }
}

// ------------------------------------------------------------------ bfloat16, many rows, large tiles
// The throughput of these tile kernels follows the number of products per fragment read from
// LDS: the 128x128 kernel's waves (2x2 MFMA tiles each) read one 1 KB fragment per product and
// reach 660-700 TFLOP/s, a 256x128 tile with the same ratio reaches the same, and this kernel's
// 256x256 tile (a WM x WN grid of waves, each TM x TN MFMA tiles of 32x32; with 4x2 tiles a wave
// reads three fragments per four products) reaches 830-900. Counters say the matrix pipes are
// busy a third of the time and LDS a quarter: what is exposed is the wait for fragments, with
// two waves per SIMD to hide it. One block per CU (its LDS holds two K-steps of both operands),
// global loads two K-steps ahead in registers. (Four waves of 128x128 each halve the reads per
// product again, but only fit the register file when the operands bypass it: the kernel after
// this one, which takes K in multiples of 128; this one takes the rest.)
template <typename TOut, int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM * WN * 64) void k_gemm_bf16_big(const bf16_t* __restrict__ X,
                                                                const bf16_t* __restrict__ W,
                                                                const float* __restrict__ bias,
                                                                TOut* __restrict__ Y, int M, int N, int K,
                                                                int tiles_m, int tiles_n, int epilogue) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, NT = WM * WN * 64;
    constexpr int PA = BM * 8 / NT, PB = BN * 8 / NT;      // 16-byte pieces of a K-step per thread
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile rows must divide over the threads");
    extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
    bf16_t* As = lds;                                      // [2][BM * BG_LD]
    bf16_t* Bs = lds + 2 * BM * BG_LD;                     // [2][BN * BG_LD]
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + N_XCD - 1) / N_XCD;
    const int logical = (blockIdx.x % N_XCD) * per_xcd + blockIdx.x / N_XCD;
    if (logical >= total) return;
    const int per_group = BG_GROUP_M * tiles_n;
    const int first_m = (logical / per_group) * BG_GROUP_M;
    const int gsize = min(tiles_m - first_m, BG_GROUP_M);
    const int tile_m = first_m + (logical % per_group) % gsize;
    const int tile_n = (logical % per_group) / gsize;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kc8 = (tid & 7) * 8;
    const bf16_t* pa[PA];
    const bf16_t* pb[PB];
    int la[PA], lb[PB];
#pragma unroll
    for (int j = 0; j < PA; ++j) {
        const int row = (tid >> 3) + (NT / 8) * j;
        pa[j] = X + (size_t)min(m0 + row, M - 1) * K;
        la[j] = row * BG_LD + kc8;
    }
#pragma unroll
    for (int j = 0; j < PB; ++j) {
        const int row = (tid >> 3) + (NT / 8) * j;
        pb[j] = W + (size_t)min(n0 + row, N - 1) * K;
        lb[j] = row * BG_LD + kc8;
    }
    const int nk = (K + BG_BK - 1) / BG_BK;
    uint4 a0[PA], b0[PB], a1[PA], b1[PB];
    // as in the 128x128 kernel: no load under a branch, addresses clamped, cut steps zeroed on the way to LDS
    auto fetch = [&](int kt, uint4 (&a)[PA], uint4 (&b)[PB]) {
        const int k = min(min(kt, nk - 1) * BG_BK + kc8, K - 8);
#pragma unroll
        for (int j = 0; j < PA; ++j) a[j] = *reinterpret_cast<const uint4*>(pa[j] + k);
#pragma unroll
        for (int j = 0; j < PB; ++j) b[j] = *reinterpret_cast<const uint4*>(pb[j] + k);
    };
    auto stash = [&](int kt, int buf, uint4 (&a)[PA], uint4 (&b)[PB]) {
        if ((kt + 1) * BG_BK > K) {
            const bool out = kt * BG_BK + kc8 >= K;
#pragma unroll
            for (int j = 0; j < PA; ++j) a[j] = zero_if(out, a[j]);
#pragma unroll
            for (int j = 0; j < PB; ++j) b[j] = zero_if(out, b[j]);
        }
#pragma unroll
        for (int j = 0; j < PA; ++j) *reinterpret_cast<uint4*>(&As[buf * BM * BG_LD + la[j]]) = a[j];
#pragma unroll
        for (int j = 0; j < PB; ++j) *reinterpret_cast<uint4*>(&Bs[buf * BN * BG_LD + lb[j]]) = b[j];
    };
    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
    const int a_base = (wm * TM * 32 + frag_row) * BG_LD + frag_k;
    const int b_base = (wn * TN * 32 + frag_row) * BG_LD + frag_k;
    // (reading the fragments of sub-step ks+1 by hand before the products of ks, as the 128x128
    // kernel does, costs registers this tile does not have: it spills and runs slower)
    auto compute = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BG_BK / 16; ++ks) {
            Frag8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                fa[i].u = *reinterpret_cast<const uint4*>(&As[buf * BM * BG_LD + a_base + i * 32 * BG_LD + ks * 16]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                fb[j].u = *reinterpret_cast<const uint4*>(&Bs[buf * BN * BG_LD + b_base + j * 32 * BG_LD + ks * 16]);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i].v, fb[j].v, acc[i][j], 0, 0, 0);
        }
    };
    auto step = [&](int i, uint4 (&na)[PA], uint4 (&nb)[PB]) {
        const int buf = i & 1;
        stash(i + 1, buf ^ 1, na, nb);
        fetch(i + 3, na, nb);
        compute(buf);
        __syncthreads();
    };
    fetch(0, a0, b0);
    fetch(1, a1, b1);
    stash(0, 0, a0, b0);
    fetch(2, a0, b0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt += 2) {           // rounds of the two sets, free of branches: with an odd
        step(kt, a1, b1);                          // number of K-steps the last round multiplies a step of zeros
        step(kt + 1, a0, b0);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 32 + (lane & 31);
            const float bn = (bias && n < N) ? bias[n] : 0.f;
            if (epilogue == EPI_SWIGLU) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float mine = acc[i][j][r] + bn;
                    const float other = __shfl_xor(mine, 1, WAVE);
                    const int m = m0 + (wm * TM + i) * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                    if (!(lane & 1) && n + 1 < N && m < M)
                        store_f32<TOut>(Y, (size_t)m * (N / 2) + n / 2, silu_mul_fast(mine, other));
                }
                continue;
            }
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + (wm * TM + i) * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (m < M) store_f32<TOut>(Y, (size_t)m * N + n, acc[i][j][r] + bn);
            }
        }
}

template <typename TOut, int WM, int WN, int TM, int TN>
static int launch_big(const bf16_t* x, const bf16_t* w, const float* bias, TOut* y, int m, int n, int k, int epilogue,
                      hipStream_t s) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr size_t lds_bytes = (size_t)2 * (BM + BN) * BG_LD * sizeof(bf16_t);
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void*)k_gemm_bf16_big<TOut, WM, WN, TM, TN>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
            return IMPARO_LAUNCH_FAILED;
        configured = true;
    }
    const int tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    const long long total = (long long)tiles_m * tiles_n;
    const unsigned blocks = (unsigned)(((total + N_XCD - 1) / N_XCD) * N_XCD);
    k_gemm_bf16_big<TOut, WM, WN, TM, TN><<<blocks, WM * WN * 64, lds_bytes, s>>>(x, w, bias, y, m, n, k, tiles_m,
                                                                                 tiles_n, epilogue);
    return launch_status();
}

// ------------------------------------------------------------------ bfloat16, many rows, loads straight into LDS
// A tile of 256 or 128 activation rows by 256, 192 or 128 weight rows on eight waves, two per
// SIMD, so that one's products run while the other waits or writes its results (12% faster than
// four waves of 128x128 on the gate/up product at 2,048 rows, 5 to 15% on the narrower tiles).
// A wave has 128 (or 64) rows by 64 or 32 of it, 4x2 or 4x1 MFMA tiles of 32x32 (2x2, 2x1 with
// 128 activation rows); the 192 wide tile's waves 64 rows by 96 (2x3). The operands never pass through registers
// on their way in: global_load_lds writes 16 bytes per
// lane straight into LDS, a wave's 64 lanes to 1 KB in a row. LDS rows are the 128 bytes of
// a K-step without padding, so the eight 16-byte pieces of row r are stored in the order
// piece ^ swz(r), swz(r) = (r & 7) ^ ((r >> 3) & 1): the loading lane picks its global piece
// accordingly, and the 16 rows that a quarter of a wave reads for one fragment fall on
// distinct banks. Two stages of 64 KB are two separate arrays: the compiler can then tell
// that reads of one stage need not wait for loads in flight to the other. A wave keeps the
// fragments of the next K-sub-step in flight while it multiplies (two register sets), and the
// barrier of a K-step sits before the last sub-step's products, so the matrix pipe has
// work queued while the waves meet. Needs K a multiple of 128 (two K-steps).
#define DM_BK 64

// What the output holds where four results of a row will go (the epilogue that adds; float32 out only)
template <typename T> __device__ __forceinline__ float4 held_vector(const T*) { return make_float4(0.f, 0.f, 0.f, 0.f); }
template <> __device__ __forceinline__ float4 held_vector<float>(const float* dst) {
    return *reinterpret_cast<const float4*>(dst);
}
template <typename T> __device__ __forceinline__ float held_f32(const T*, int) { return 0.f; }
template <> __device__ __forceinline__ float held_f32<float>(const float* dst, int c) { return dst[c]; }

// Two (`pair`) or four outputs of one row in one store; the address is aligned to the store
template <typename T> __device__ __forceinline__ void store_vector(T* dst, const float (&o)[4], bool pair);
template <> __device__ __forceinline__ void store_vector<float>(float* dst, const float (&o)[4], bool pair) {
    if (pair)
        *reinterpret_cast<float2*>(dst) = make_float2(o[0], o[1]);
    else
        *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
}
template <> __device__ __forceinline__ void store_vector<bf16_t>(bf16_t* dst, const float (&o)[4], bool pair) {
    const unsigned lo = f32x2_to_bf16x2(o[0], o[1]);
    if (pair)
        *reinterpret_cast<unsigned*>(dst) = lo;
    else
        *reinterpret_cast<uint2*>(dst) = make_uint2(lo, f32x2_to_bf16x2(o[2], o[3]));
}

__device__ __forceinline__ void load_to_lds(const bf16_t* src, bf16_t* dst_wave_uniform) {
    __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                     (void __attribute__((address_space(3)))*)dst_wave_uniform, 16, 0, 0);
}

// The same load written out, for the kernel that keeps the loads of several K-steps in flight. The compiler
// answers a fragment read from LDS that follows any load into LDS it knows of with a wait for every load
// (it counts such a load as one that may come back out of order), which empties the pipeline; a load it
// does not know of it does not wait for, and the kernel waits itself, by count. `lds_byte` is the same
// for the whole wave.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_to_lds_uncounted(const bf16_t* src, unsigned lds_byte) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(src), "s"(lds_byte)
                 : "memory", "m0");
}
#pragma clang diagnostic pop

// TMI, TN: MFMA tiles of 32x32 down a wave's part of the activation rows and across its part of
// the weight rows; NWM, NWN: waves down and across (eight in all). The launcher's plan chooses
// the tile so that the blocks come out in whole rounds of the CUs.
template <typename TOut, int TMI, int TN, int NWN, int NWM = 2, int STAGES = 2>
__global__ __launch_bounds__(64 * NWM * NWN) void k_gemm_bf16_dma(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                             const float* __restrict__ bias, TOut* __restrict__ Y,
                                                             int M, int N, int K_all, int k_per, int tiles_m,
                                                             int tiles_n, int epilogue) {
    constexpr int NW = NWM * NWN;                      // waves of the block
    constexpr int WN = 32 * TN;                        // weight rows of one wave's part
    constexpr int BN = NWN * WN;                       // of the block's tile
    constexpr int WM = 32 * TMI;                       // activation rows of one wave's part
    constexpr int BM = NWM * WM;                       // of the block's tile
    constexpr int LX = BM / (8 * NW), LW = BN / (8 * NW);   // load instructions per wave and K-step
    static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "the waves share the tile's rows evenly");
    __shared__ __attribute__((aligned(1024))) bf16_t stage0[(BM + BN) * DM_BK];   // X rows, then W rows
    __shared__ __attribute__((aligned(1024))) bf16_t stage1[(BM + BN) * DM_BK];
    // four stages (a block alone on its CU): the loads of three K-steps in flight while one is multiplied
    static_assert(STAGES == 2 || STAGES == 4, "two stages or four");
    __shared__ __attribute__((aligned(1024))) bf16_t stage2[STAGES == 4 ? (BM + BN) * DM_BK : 8];
    __shared__ __attribute__((aligned(1024))) bf16_t stage3[STAGES == 4 ? (BM + BN) * DM_BK : 8];
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + N_XCD - 1) / N_XCD;
    const int logical = (blockIdx.x % N_XCD) * per_xcd + blockIdx.x / N_XCD;
    if (logical >= total) return;
    const int per_group = BG_GROUP_M * tiles_n;
    const int first_m = (logical / per_group) * BG_GROUP_M;
    const int gsize = min(tiles_m - first_m, BG_GROUP_M);
    const int tile_m = first_m + (logical % per_group) % gsize;
    const int tile_n = (logical % per_group) / gsize;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    // slices of K (gridDim.y > 1): block (x, y) sums K range [y * k_per, (y+1) * k_per) into Y + y * M * N
    const int k_lo = blockIdx.y * k_per;
    const int K = min(K_all, k_lo + k_per) - k_lo;
    X += k_lo;
    W += k_lo;
    Y += (size_t)blockIdx.y * M * N;
    if (blockIdx.y > 0) bias = nullptr;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / NWN, wn = wave % NWN;
    // loading: instruction j of a wave fills rows j*8*NW + wave*8 .. +7; lane -> row lane/8, slot lane%8
    const int load_row = wave * 8 + (lane >> 3);
    const int load_piece = (lane & 7) ^ (lane >> 3) ^ (wave & 1);          // lane%8 ^ swz(row)
    unsigned off_x[LX], off_w[LW];
#pragma unroll
    for (int j = 0; j < LX; ++j)
        off_x[j] = (unsigned)min(m0 + j * 8 * NW + load_row, M - 1) * (unsigned)K_all + load_piece * 8;
#pragma unroll
    for (int j = 0; j < LW; ++j)
        off_w[j] = (unsigned)min(n0 + j * 8 * NW + load_row, N - 1) * (unsigned)K_all + load_piece * 8;
    auto load_step = [&](bf16_t* stage, int kt) __attribute__((always_inline)) {
        const bf16_t* xk = X + (size_t)kt * DM_BK;
        const bf16_t* wk = W + (size_t)kt * DM_BK;
        if (STAGES == 4) {
            const unsigned to = __builtin_amdgcn_readfirstlane(
                (unsigned)(size_t)(__attribute__((address_space(3))) bf16_t*)stage + wave * 8 * DM_BK * 2);
#pragma unroll
            for (int j = 0; j < LX; ++j) load_to_lds_uncounted(xk + off_x[j], to + j * 8 * NW * DM_BK * 2);
#pragma unroll
            for (int j = 0; j < LW; ++j) load_to_lds_uncounted(wk + off_w[j], to + (BM + j * 8 * NW) * DM_BK * 2);
            return;
        }
#pragma unroll
        for (int j = 0; j < LX; ++j) load_to_lds(xk + off_x[j], stage + (j * 8 * NW + wave * 8) * DM_BK);
#pragma unroll
        for (int j = 0; j < LW; ++j) load_to_lds(wk + off_w[j], stage + (BM + j * 8 * NW + wave * 8) * DM_BK);
    };
    // fragments: lane holds row lane%32, K-half lane/32 of a 32x16 piece; sub-step ks is pieces 2ks, 2ks+1
    const int frag_row = lane & 31;
    const int swz = (frag_row & 7) ^ ((frag_row >> 3) & 1);
    const int a_base = (wm * WM + frag_row) * DM_BK + (((lane >> 5) ^ swz) << 3);
    const int b_base = (BM + wn * WN + frag_row) * DM_BK + (((lane >> 5) ^ swz) << 3);
    f32x16 acc[TMI][TN];
#pragma unroll
    for (int i = 0; i < TMI; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    auto read = [&](const bf16_t* stage, int ks, Frag8 (&fa)[TMI], Frag8 (&fb)[TN]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TMI; ++i)
            fa[i].u = *reinterpret_cast<const uint4*>(&stage[(a_base ^ (ks << 4)) + i * 32 * DM_BK]);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            fb[j].u = *reinterpret_cast<const uint4*>(&stage[(b_base ^ (ks << 4)) + j * 32 * DM_BK]);
    };
    auto multiply = [&](const Frag8 (&fa)[TMI], const Frag8 (&fb)[TN]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < TMI; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i].v, fb[j].v, acc[i][j], 0, 0, 0);
    };
    const int nk = K / DM_BK;
    Frag8 fa0[TMI], fb0[TN], fa1[TMI], fb1[TN];
    // K-step kt from `cur`: on entry set 0 holds its first sub-step and the loads of step kt+1
    // into `next` are in flight (and with four stages those of kt+2 and kt+3); on exit set 0 holds
    // the first sub-step of kt+1 and the loads of kt+STAGES into `cur` are in flight
    auto k_step = [&](bf16_t* cur, bf16_t* next, int kt) __attribute__((always_inline)) {
        // (the scheduling barriers keep each sub-step's reads and products where they are written:
        // left alone, the compiler sinks the loads of the next step to just before the wait for them)
        read(cur, 1, fa1, fb1);
        multiply(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        read(cur, 2, fa0, fb0);
        multiply(fa1, fb1);
        __builtin_amdgcn_sched_barrier(0);
        read(cur, 3, fa1, fb1);
        multiply(fa0, fb0);
        __builtin_amdgcn_sched_barrier(0);
        // this wave's part of `next` has landed and `cur` is read; after the barrier, so for every wave
        if (STAGES == 4) {             // the loads of the two steps after `next` stay in flight: a bare barrier
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(2 * (LX + LW)) : "memory");
            __builtin_amdgcn_s_barrier();
        } else {
            __syncthreads();
        }
        read(next, 0, fa0, fb0);
        load_step(cur, min(kt + STAGES, nk - 1));   // past the end: the last step again, into a stage nobody reads any more
        multiply(fa1, fb1);
#pragma unroll
        for (int q = 0; q < TMI * TN; ++q) {        // one product, (one fragment read,) one load or two
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (q < TMI + TN) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (q < LX + LW - TMI * TN)
                __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
            else if (q < LX + LW)
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    if (STAGES == 4) {
        load_step(stage0, 0);
        load_step(stage1, 1);
        load_step(stage2, 2);
        load_step(stage3, 3);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(3 * (LX + LW)) : "memory");
        __builtin_amdgcn_s_barrier();
        read(stage0, 0, fa0, fb0);
        for (int kt = 0; kt < nk; kt += 4) {           // K-steps in fours: one loop, one way round it
            k_step(stage0, stage1, kt);
            k_step(stage1, stage2, kt + 1);
            k_step(stage2, stage3, kt + 2);
            k_step(stage3, stage0, kt + 3);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the loads past the end: nothing may land in what the tile leaves through
    } else {
        load_step(stage0, 0);
        __syncthreads();
        load_step(stage1, 1);
        read(stage0, 0, fa0, fb0);
        for (int kt = 0; kt < nk; kt += 2) {           // an even number of K-steps: one loop, one way round it
            k_step(stage0, stage1, kt);
            k_step(stage1, stage0, kt + 1);
        }
    }
    // The tile leaves through LDS, a wave's 32 rows x 128 columns at a time (one row of its MFMA
    // tiles): the wave writes the accumulators as the matrix pipe left them, reads whole rows
    // back, four columns per lane, and stores 16 (or 8, or 4) bytes per lane, half a wave to a row.
    // That keeps the 256 accumulators out of the vector registers (where the compiler would
    // otherwise gather them all at once, spilling what the K loop needs) and gives row-long
    // stores. A staged row is 136 floats: the two rows a store instruction touches, 4 apart,
    // fall on disjoint banks. Each wave has a region of its own, so no barrier between passes.
    __syncthreads();                                   // every wave is done with the operands in LDS
    constexpr int EP_LD = (NWN == 2 && NWM == 2 && TN > 1) ? 136 : WN + 8;
    constexpr int LPR = ((NWN == 2 && NWM == 2 && TN > 1) || 64 % (WN / 4)) ? 32 : WN / 4;   // lanes to a staged row
    static_assert((4 * EP_LD) % 64 == 32 && NW / 2 * 32 * EP_LD * 4 <= (BM + BN) * DM_BK * 2, "staging layout");
    float* staged = reinterpret_cast<float*>(wave >= NW / 2 ? stage1 : stage0) + (wave % (NW / 2)) * (32 * EP_LD);
    const int out_col = (lane % LPR) * 4;              // of the wave's columns: lanes past them (narrow tiles) sit out
    const bool lane_on = out_col < WN;
    const int n = n0 + wn * WN + out_col;
    float bn[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias && lane_on) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (n + c < N) bn[c] = bias[n + c];
    }
    const bool swiglu = epilogue == EPI_SWIGLU;
    const bool adds = epilogue == EPI_ADD;             // (float32 out; the launcher sees to it)
    const int out_n = swiglu ? N / 2 : N;              // columns of Y
    const int per_lane = swiglu ? 2 : 4;               // outputs a lane holds of a row
    // whole vectors: every row of this tile inside, the lane's columns inside, rows of Y aligned
    const bool vectors = m0 + BM <= M && n0 + BN <= N && out_n % per_lane == 0 &&
                         ((uintptr_t)Y % (per_lane * sizeof(TOut))) == 0;
    constexpr int ITS = 32 * LPR / 64;                 // rows of a pass that a lane stores
    constexpr bool CAN_ADD = std::is_same<TOut, float>::value;
#pragma unroll
    for (int i = 0; i < TMI; ++i) {
        // what the output holds (the epilogue that adds): a pass's rows asked for together, before the
        // accumulators go through LDS, so that the trips to memory overlap each other and the staging
        float4 held[CAN_ADD ? ITS : 1];
        if (CAN_ADD && adds && vectors && lane_on) {
#pragma unroll
            for (int it = 0; it < ITS; ++it) {
                const int m = m0 + wm * WM + i * 32 + it * (64 / LPR) + lane / LPR;
                held[CAN_ADD ? it : 0] = held_vector<TOut>(Y + (size_t)m * out_n + n);
            }
        }
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                staged[((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) * EP_LD + j * 32 + (lane & 31)] = acc[i][j][r];
#pragma unroll
        for (int it = 0; it < ITS; ++it) {
            if (!lane_on) continue;
            const int row = it * (64 / LPR) + lane / LPR;
            const float4 v = *reinterpret_cast<const float4*>(&staged[row * EP_LD + out_col]);
            const int m = m0 + wm * WM + i * 32 + row;
            float o[4] = {v.x + bn[0], v.y + bn[1], v.z + bn[2], v.w + bn[3]};
            if (swiglu) {
                o[0] = silu_mul_fast(o[0], o[1]);
                o[1] = silu_mul_fast(o[2], o[3]);
            }
            TOut* dst = Y + (size_t)m * out_n + (swiglu ? n / 2 : n);
            if (vectors) {
                if (CAN_ADD && adds) {
                    const float4 h = held[CAN_ADD ? it : 0];
                    o[0] = h.x + o[0], o[1] = h.y + o[1], o[2] = h.z + o[2], o[3] = h.w + o[3];
                }
                store_vector<TOut>(dst, o, swiglu);
            } else if (m < M) {
                if (swiglu) {
                    if (n + 1 < N) store_f32<TOut>(dst, 0, o[0]);
                    if (n + 3 < N) store_f32<TOut>(dst, 1, o[1]);
                } else {
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        if (n + c < N) store_f32<TOut>(dst, c, adds ? held_f32<TOut>(dst, c) + o[c] : o[c]);
                }
            }
        }
    }
}

static bool dma_tile_takes(int m, int n, int k) {
    // the operands' offsets are kept in 32 bits
    return k % (2 * DM_BK) == 0 && (long long)m * k < (1LL << 31) && (long long)n * k < (1LL << 31);
}

// Which tile (bm = 256 or 128 activation rows, tn = 4, 3, 2, 1 for 256, 192, 128, 64 weight rows; 192 with
// bm 256 only, 64 with bm 128 only), on how many stages, and how many slices of K suit a product of many rows; tn = 0:
// none (a K the kernel does not take). A model of the time, fitted to this machine over 128 to 8,192
// rows and seven weight shapes, every tile and 1 to 8 slices measured (what it picks is within 1 % of
// the fastest on average and within 7 % on every shape whose consumer can add slices):
//   - a K-step of 64 takes a block alone on its CU the first figure below with few CUs busy and the
//     second with all 256 (clocks, L2), in between in proportion:
//         128x128 0.46 .. 0.78 us    128x256 0.70 .. 1.08    256x128 0.66 .. 1.08
//         256x192 0.89 .. 1.30       256x256 1.03 .. 1.58
//   - a tile of 128 rows by 64 weight rows on four waves and four stages takes 0.35 .. 0.50 us a step: with at
//     most 128 rows (one tile down the rows) it makes twice the blocks of the 128x128 tile out of a weight
//     that is streamed once, and a block's share of the weights is what bounds such a product (measured at
//     96 and 128 rows: 21 us against 27 on gate/up, 8 to 13 against 11 to 18 on the sliced products);
//   - two blocks fit a CU where their stages take 80 KB or less each (the 128x128 tile on two
//     stages); a step of both then takes 1.09 us, and with two on some CUs only, in between;
//   - the 128x128 tile can instead keep four stages (one block a CU, three steps' loads in flight):
//     0.33 .. 0.53 us a step, which pays where the tiles are one round of the CUs or less;
//   - with one or two tiles down the rows (a decode batch of 65 to 256 rows) every block meets its
//     weights first, and cold: a step then takes 0.55 us at least on two stages and 0.36 on four;
//   - a block's beginning and end take 4.3 us + 0.116 us per MFMA of a SIMD in a K-step
//     (bm * bn / 1024 of them);
//   - blocks run in rounds of what fits the chip at once; the operands have to come from memory
//     once (5.5 TB/s) and the results have to go there (7.6 TB/s); a slice beyond the first costs
//     its consumer one more pass over rows x width of float32 (5 TB/s).
// `fixed_slices` > 0: the caller has decided (1: its consumer cannot add slices).
struct DmaPlan {
    int bm, tn, slices, stages;
};
static DmaPlan dma_plan(int m, int n, int k, int fixed_slices) {
    DmaPlan best{0, 0, fixed_slices > 0 ? fixed_slices : 1, 2};
    if (m <= 64 || !dma_tile_takes(m, n, k)) return best;
    double best_cost = 0.0;
    for (int slices : {1, 2, 3, 4, 6, 8}) {                 // (3 and 6: a K of 27 or 9 times 256 has no other cut)
        if (fixed_slices > 0 && slices != fixed_slices) continue;
        if (k % (128 * slices) != 0 || (slices > 1 && k / slices < 512)) continue;
        for (int bm = 256; bm >= 128; bm /= 2) {
            const int tiles_m = (m + bm - 1) / bm;
            for (int tn = 4; tn >= 1; --tn) {
                if (tn == 3 && bm != 256) continue;
                if (tn == 1 && bm != 128) continue;
                const int bn = 64 * tn;
                for (int stages = 2; stages <= 4; stages += 2) {
                    // four stages: the 128x128 tile and the 128x64 one (which runs on four only), K-steps in fours
                    if (stages == 4 && (bm != 128 || tn > 2 || (k / slices) % (4 * DM_BK) != 0)) continue;
                    if (stages == 2 && tn == 1) continue;
                    const long long blocks = (long long)tiles_m * ((n + bn - 1) / bn) * slices;
                    const int at_once = 256 * ((bm + bn) * DM_BK * 2 * stages <= 80 * 1024 ? 2 : 1);
                    const long long rounds = (blocks + at_once - 1) / at_once;
                    const long long per_round = (blocks + rounds - 1) / rounds;
                    const double cus = (double)std::min<long long>(256, per_round);
                    double few, all;
                    if (bm == 128 && tn == 1) few = 0.35, all = 0.50;
                    else if (bm == 128 && tn == 2) few = stages == 4 ? 0.33 : 0.46, all = stages == 4 ? 0.53 : 0.78;
                    else if (bm == 128) few = 0.70, all = 1.08;
                    else if (tn == 2) few = 0.66, all = 1.08;
                    else if (tn == 3) few = 0.89, all = 1.30;
                    else few = 1.03, all = 1.58;
                    double step = per_round > 256 ? all + (1.09 - all) * (per_round - 256) / 256.0    // some CUs, or all, with two
                                                  : few + (all - few) * cus / 256.0;
                    if (tiles_m <= 2) step = std::max(step, stages == 4 ? 0.36 : 0.55);
                    // one tile down the rows: a block streams its weight rows alone, 128 bytes of each a
                    // step, and one CU draws about 28 GB/s of cold weights (0.60 us a step measured on the
                    // 128x128 tile at 128 rows, where the figures above would have it at 0.43)
                    if (tiles_m == 1) step = std::max(step, bn * 128.0 / 28e3);
                    const double ends = 4.3 + 0.116 * (bm * bn / 1024.0);
                    const double from_memory = ((double)m + n) * k * 2.0 / 5.5e6;
                    const double cost = std::max(rounds * (k / slices / DM_BK * step + ends), from_memory + ends) +
                                        (double)slices * m * n * 4.0 / 7.6e6 + (slices - 1) * ((double)m * n * 4.0 / 5e6);
                    if (best.tn == 0 || cost < best_cost) {
                        best = DmaPlan{bm, tn, slices, stages};
                        best_cost = cost;
                    }
                }
            }
        }
    }
    return best;
}

// `slices` must leave every slice a multiple of 128 of K (dma_tile_takes(m, n, k / slices) and k % slices == 0).
// bm: 256 or 128 activation rows to a tile; tn: 4, 3 (bm 256 only), 2 or 1 (bm 128 only) for 256, 192, 128 or 64 weight rows.
template <typename TOut>
static int launch_dma(const bf16_t* x, const bf16_t* w, const float* bias, TOut* y, int m, int n, int k, int epilogue,
                      int bm, int tn, int slices, hipStream_t s, int stages = 2) {
    const int tiles_m = (m + bm - 1) / bm, tiles_n = (n + 64 * tn - 1) / (64 * tn);
    const long long total = (long long)tiles_m * tiles_n;
    const dim3 grid((unsigned)(((total + N_XCD - 1) / N_XCD) * N_XCD), (unsigned)slices);
#define DMA_GO(TMI, TN, NWN)                                                                                         \
    k_gemm_bf16_dma<TOut, TMI, TN, NWN><<<grid, 128 * NWN, 0, s>>>(x, w, bias, y, m, n, k, k / slices, tiles_m,     \
                                                                   tiles_n, epilogue)
    if (bm == 128 && tn == 1 && stages == 4)   // 64 wide: four waves of 64 rows by 32
        k_gemm_bf16_dma<TOut, 2, 1, 2, 2, 4><<<grid, 256, 0, s>>>(x, w, bias, y, m, n, k, k / slices, tiles_m, tiles_n, epilogue);
    else if (bm == 128 && tn == 1)
        k_gemm_bf16_dma<TOut, 2, 1, 2, 2, 2><<<grid, 256, 0, s>>>(x, w, bias, y, m, n, k, k / slices, tiles_m, tiles_n, epilogue);
    else if (bm == 128 && tn == 4)
        DMA_GO(2, 2, 4);
    else if (bm == 128 && stages == 4)
        k_gemm_bf16_dma<TOut, 2, 1, 4, 2, 4><<<grid, 512, 0, s>>>(x, w, bias, y, m, n, k, k / slices, tiles_m, tiles_n, epilogue);
    else if (bm == 128)
        DMA_GO(2, 1, 4);
    else if (tn == 4)     // 256 wide: eight waves
        DMA_GO(4, 2, 4);
    else if (tn == 3)     // 192 wide: eight waves of 64 rows by 96
        k_gemm_bf16_dma<TOut, 2, 3, 2, 4><<<grid, 512, 0, s>>>(x, w, bias, y, m, n, k, k / slices, tiles_m, tiles_n, epilogue);
    else                  // 128 wide: eight waves
        DMA_GO(4, 1, 4);
#undef DMA_GO
    return launch_status();
}

// ------------------------------------------------------------------ bfloat16, few rows
// One block per 16 weight rows. Its NW waves split K in chunks of 128: wave w
// takes chunks w, w + NW, ... so the block reads each weight row as one
// contiguous stream. The 16 weight rows are the MFMA's M side, up to 16*MT
// activation rows its N side. A decode step is a chain of such products, each
// a few megabytes: what counts is how few memory round trips one of them
// takes, so a wave has the loads of its next chunk in flight while it
// multiplies the current one, and NW is chosen so that a wave has few chunks.
// Partial sums meet in LDS and are added in wave order, so the result is the
// same from run to run.
template <int MT>
struct SkinnyFrags {
    Frag8 w[4];
    Frag8 x[MT][4];
};

// With slices (gridDim.y > 1) block (x, y) sums only K range [y * k_per, (y+1) * k_per) and
// writes it to Y + y * M * N: the consumer adds the slices in order.
template <typename TOut, int MT, int NW>
__global__ __launch_bounds__(NW * 64) void k_gemm_bf16_skinny(const bf16_t* __restrict__ X,
                                                              const bf16_t* __restrict__ W,
                                                              const float* __restrict__ bias,
                                                              TOut* __restrict__ Y, int M, int N, int K_all,
                                                              int k_per, int epilogue) {
    __shared__ float red[NW][MT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 16;
    const int k_lo = blockIdx.y * k_per;
    const int K = min(K_all, k_lo + k_per) - k_lo;       // this block's part of K, re-based to 0
    X += k_lo;
    W += k_lo;
    Y += (size_t)blockIdx.y * M * N;
    if (blockIdx.y > 0) bias = nullptr;                  // the bias belongs to one slice only
    const int r16 = lane & 15, g = lane >> 4;
    const bf16_t* wrow = W + (size_t)min(n0 + r16, N - 1) * K_all + g * 8;
    const bf16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xrow[mt] = X + (size_t)min(mt * 16 + r16, M - 1) * K_all + g * 8;
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load = [&](int k0, SkinnyFrags<MT>& f) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int k = k0 + s * 32;
            const bool in = k + g * 8 < K;
            f.w[s].u = in ? *reinterpret_cast<const uint4*>(wrow + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                f.x[mt][s].u = in ? *reinterpret_cast<const uint4*>(xrow[mt] + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto multiply = [&](const SkinnyFrags<MT>& f) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int s = 0; s < 4; ++s)
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.w[s].v, f.x[mt][s].v, acc[mt], 0, 0, 0);
    };

    SkinnyFrags<MT> cur, nxt;
    int k0 = wave * 128;
    if (k0 < K) load(k0, cur);
    while (k0 < K) {
        const int k1 = k0 + NW * 128;
        if (k1 < K) load(k1, nxt);
        multiply(cur);
        cur = nxt;
        k0 = k1;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[wave][mt][lane][i] = acc[mt][i];
    __syncthreads();
    if (wave != 0) return;
    // D layout of the 16x16 tile: lane holds column lane%16 (an activation row),
    // rows 4*(lane/16) + i (weight rows)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[i] = red[0][mt][lane][i];
#pragma unroll
            for (int w = 1; w < NW; ++w) v[i] += red[w][mt][lane][i];
            const int n = n0 + g * 4 + i;
            if (bias && n < N) v[i] += bias[n];
        }
        if (m >= M) continue;
        if (epilogue == EPI_SWIGLU) {
#pragma unroll
            for (int i = 0; i < 4; i += 2) {
                const int n = n0 + g * 4 + i;
                if (n + 1 < N) store_f32<TOut>(Y, (size_t)m * (N / 2) + n / 2, silu_mul_fast(v[i], v[i + 1]));
            }
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + g * 4 + i;
            if (n < N) store_f32<TOut>(Y, (size_t)m * N + n, v[i]);
        }
    }
}

template <typename TOut, int MT>
static void launch_skinny(const bf16_t* x, const bf16_t* w, const float* bias, TOut* y, int m, int n, int k,
                          int epilogue, int slices, hipStream_t s) {
    const int k_per = ((k + slices - 1) / slices + 127) / 128 * 128;
    dim3 grid((unsigned)((n + 15) / 16), (unsigned)((k + k_per - 1) / k_per));
    // few chunks of 128 per wave: 4 waves up to 512 of K per block, 8 up to 2048, 16 beyond
    if (k_per <= 512)
        k_gemm_bf16_skinny<TOut, MT, 4><<<grid, 4 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue);
    else if (k_per <= 2048)
        k_gemm_bf16_skinny<TOut, MT, 8><<<grid, 8 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue);
    else if constexpr (MT <= 2)
        k_gemm_bf16_skinny<TOut, MT, 16><<<grid, 16 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue);
    else   // 64 activation rows keep too many fragments in registers for 1024 threads
        k_gemm_bf16_skinny<TOut, MT, 8><<<grid, 8 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue);
}

// ------------------------------------------------------------------ conv input projection + gated conv, single tokens
// For a decode step's rows (one token each, at most 16): the projection to [B | C | x] and the
// gated short convolution that consumes it in one launch. A block takes 8 channels: its first
// MFMA tile holds the B rows of those channels (tile rows 0..7) and their x rows (8..15), its
// second the C rows (0..7, and again in 8..15: the same cache lines, nothing more to fetch).
// K is split over the waves as in the kernel above and the partial sums meet in LDS in wave
// order; then 32 lanes of wave 0 each own one token and four channels: u = B * x, the taps
// oldest first exactly as the conv kernels sum them, the C gate, and the shift of the state
// (a lane owns its channels' history, so nothing races). With HIST > 0 the history, the taps
// and the biases are asked for before the walk along K, so they are there when it ends.
// With ssq_in, X is the residual stream times a norm's weight, not yet scaled: the partial sums of
// squares of its rows [n_parts, 16] give each row's scale, which multiplies B, C and x at the end (rows.h).
template <typename TOut, int NW, int HIST>
__global__ __launch_bounds__(NW * 64) void k_in_proj_conv_decode(
    const bf16_t* __restrict__ X, const float* __restrict__ ssq_in, int n_parts, float eps,
    const bf16_t* __restrict__ W, const float* __restrict__ in_bias,
    const float* __restrict__ conv_w, const float* __restrict__ conv_b, float* __restrict__ state,
    const int32_t* __restrict__ slot, TOut* __restrict__ out, int M, int E, int K, int taps) {
    __shared__ float red[NW][2][64][4];
    __shared__ float norm_part[NW * 4 * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int c0 = blockIdx.x * 8;
    const bf16_t* wrow0 = W + (size_t)(r16 < 8 ? c0 + r16 : 2 * E + c0 + (r16 - 8)) * K + g * 8;
    const bf16_t* wrow1 = W + (size_t)(E + c0 + (r16 & 7)) * K + g * 8;
    const bf16_t* xrow = X + (size_t)min(r16, M - 1) * K + g * 8;
    const int history = HIST > 0 ? HIST : taps - 1;
    // the lanes that finish the block: token r16, channels cb .. cb+3
    const bool finisher = wave == 0 && g < 2 && r16 < M;
    const int cb = c0 + 4 * (g & 1);
    float* st = state + (size_t)(finisher ? slot[r16] : 0) * history * E;
    constexpr int HN = HIST > 0 ? HIST : 1;
    float hist[HN][4], tap[HN + 1][4], bias_b[4], bias_c[4], bias_x[4], bias_conv[4];
    if (HIST > 0 && finisher) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int k = 0; k < HIST; ++k) hist[k][i] = st[(size_t)k * E + cb + i];
#pragma unroll
            for (int k = 0; k <= HIST; ++k) tap[k][i] = conv_w[(size_t)(cb + i) * (HIST + 1) + k];
            bias_b[i] = in_bias ? in_bias[cb + i] : 0.f;
            bias_c[i] = in_bias ? in_bias[E + cb + i] : 0.f;
            bias_x[i] = in_bias ? in_bias[2 * E + cb + i] : 0.f;
            bias_conv[i] = conv_b ? conv_b[cb + i] : 0.f;
        }
    }
    struct Frags {
        Frag8 w0[4], w1[4], x[4];
    };
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    auto load = [&](int k0, Frags& f) {
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) {
            const int k = k0 + s2 * 32;
            const bool in = k + g * 8 < K;
            f.w0[s2].u = in ? *reinterpret_cast<const uint4*>(wrow0 + k) : make_uint4(0, 0, 0, 0);
            f.w1[s2].u = in ? *reinterpret_cast<const uint4*>(wrow1 + k) : make_uint4(0, 0, 0, 0);
            f.x[s2].u = in ? *reinterpret_cast<const uint4*>(xrow + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto multiply = [&](const Frags& f) {
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2) {
            acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.w0[s2].v, f.x[s2].v, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.w1[s2].v, f.x[s2].v, acc1, 0, 0, 0);
        }
    };
    Frags cur, nxt;
    int k0 = wave * 128;
    if (k0 < K) load(k0, cur);
    // the row's scale multiplies the sums at the end: its sums of squares are asked for now
    RowsSsq early;
    if (ssq_in) rows_ssq_ask(early, ssq_in, n_parts, 0);
    while (k0 < K) {
        const int k1 = k0 + NW * 128;
        if (k1 < K) load(k1, nxt);
        multiply(cur);
        cur = nxt;
        k0 = k1;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        red[wave][0][lane][i] = acc0[i];
        red[wave][1][lane][i] = acc1[i];
    }
    if (ssq_in) norm_part[(threadIdx.x >> 4) * 16 + (threadIdx.x & 15)] = rows_ssq_sum(early, ssq_in, n_parts);
    __syncthreads();
    if (!finisher) return;
    const float scale = ssq_in ? rows_scale(norm_part, r16, K, eps) : 1.f;
    // D layout: lane holds column lane%16 (a token), tile rows 4*(lane/16) + i: B and C of channel
    // cb + i sit in this lane's entries, x of the same channel 8 tile rows further: lane + 32
    float b[4], c[4], x[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        b[i] = red[0][0][lane][i];
        x[i] = red[0][0][lane + 32][i];
        c[i] = red[0][1][lane][i];
#pragma unroll
        for (int w = 1; w < NW; ++w) {
            b[i] += red[w][0][lane][i];
            x[i] += red[w][0][lane + 32][i];
            c[i] += red[w][1][lane][i];
        }
        if (ssq_in) {
            b[i] = __fmul_rn(b[i], scale);
            x[i] = __fmul_rn(x[i], scale);
            c[i] = __fmul_rn(c[i], scale);
        }
    }
    float y[4];
    if (HIST > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float u = (b[i] + bias_b[i]) * (x[i] + bias_x[i]);
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < HIST; ++k) {
                a = fmaf(tap[k][i], hist[k][i], a);
                st[(size_t)k * E + cb + i] = k + 1 < HIST ? hist[k + 1][i] : u;
            }
            a = fmaf(tap[HIST][i], u, a);
            a += bias_conv[i];
            y[i] = (c[i] + bias_c[i]) * a;
        }
    } else {
        for (int i = 0; i < 4; ++i) {
            const int ch = cb + i;
            const float bv = b[i] + (in_bias ? in_bias[ch] : 0.f);
            const float cv = c[i] + (in_bias ? in_bias[E + ch] : 0.f);
            const float xv = x[i] + (in_bias ? in_bias[2 * E + ch] : 0.f);
            const float u = bv * xv;
            float a = 0.f;
            float prev = st[ch];                                  // oldest
            for (int k = 0; k < history; ++k) {
                a = fmaf(conv_w[(size_t)ch * taps + k], prev, a);
                const float next = (k + 1 < history) ? st[(size_t)(k + 1) * E + ch] : u;
                st[(size_t)k * E + ch] = next;
                prev = next;
            }
            a = fmaf(conv_w[(size_t)ch * taps + history], u, a);
            a += conv_b ? conv_b[ch] : 0.f;
            y[i] = cv * a;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) store_f32<TOut>(out, (size_t)r16 * E + cb + i, y[i]);
}

template <typename TOut, int NW>
static void launch_in_proj_conv(const bf16_t* x, const float* ssq_in, int n_parts, float eps, const bf16_t* w,
                                const float* in_bias, const float* conv_w, const float* conv_b, float* state,
                                const int32_t* slot, TOut* out, int m, int e, int k, int taps, hipStream_t s) {
    const unsigned blocks = (unsigned)(e / 8);
#define CONV_GO(HIST)                                                                                              \
    k_in_proj_conv_decode<TOut, NW, HIST><<<blocks, NW * 64, 0, s>>>(x, ssq_in, n_parts, eps, w, in_bias, conv_w, conv_b, \
                                                                   state, slot, out, m, e, k, taps)
    switch (taps - 1) {
        case 1: CONV_GO(1); break;
        case 2: CONV_GO(2); break;
        case 3: CONV_GO(3); break;
        default: CONV_GO(0);
    }
#undef CONV_GO
}

// x [m, k] bfloat16 (m <= 16 single tokens), w [3 e, k] bfloat16, conv_w [e, taps], state
// [n_slots, taps-1, e], slot [m] (distinct): out [m, e] = the gated conv's output, state shifted.
// ssq_in [n_parts, 16] (or null) and eps: x is the residual stream times a norm's weight, each row
// still to be scaled by rsqrt(sum of its partial sums of squares / k + eps), which the launch does.
extern "C" int imparo_in_proj_conv_decode_normed(const void* x, const float* ssq_in, int n_parts, float eps,
                                                 const void* w, const float* in_bias, const float* conv_w,
                                                 const float* conv_b, float* state, const int32_t* slot, void* out,
                                                 int out_dtype, int m, int e, int k, int taps, int n_slots,
                                                 imparo_stream stream) {
    if (!x || !w || !conv_w || !state || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (ssq_in && (n_parts <= 0 || !(eps > 0.f))) return IMPARO_BAD_ARGUMENT;
    if (m < 0 || m > 16 || e <= 0 || e % 8 != 0 || k <= 0 || k % 8 != 0 || taps < 2 || taps > 64 || n_slots <= 0)
        return IMPARO_BAD_ARGUMENT;
    if (((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return IMPARO_BAD_ARGUMENT;
    if (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    if (m == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    // waves over K as the K-split kernel has them: chunks of 128, few per wave
#define CONV_CALL(TOut, NW)                                                                                          \
    launch_in_proj_conv<TOut, NW>(xb, ssq_in, n_parts, eps, wb, in_bias, conv_w, conv_b, state, slot, (TOut*)out, m, e, \
                                  k, taps, s)
    if (out_dtype == IMPARO_F32) {
        if (k <= 512) CONV_CALL(float, 4);
        else CONV_CALL(float, 8);
    } else {
        if (k <= 512) CONV_CALL(bf16_t, 4);
        else CONV_CALL(bf16_t, 8);
    }
#undef CONV_CALL
    return launch_status();
}

extern "C" int imparo_in_proj_conv_decode(const void* x, const void* w, const float* in_bias, const float* conv_w,
                                          const float* conv_b, float* state, const int32_t* slot, void* out,
                                          int out_dtype, int m, int e, int k, int taps, int n_slots,
                                          imparo_stream stream) {
    return imparo_in_proj_conv_decode_normed(x, nullptr, 0, 0.f, w, in_bias, conv_w, conv_b, state, slot, out, out_dtype,
                                             m, e, k, taps, n_slots, stream);
}


// Which kernel takes a product of up to 64 rows: 0 for the K-split kernel, else the waves per
// block of the shared-activation kernel. Measured with cold weights (they never stay in cache
// between decode steps): from about 12k weight rows on the shared-activation kernel wins at
// any number of rows; below that it wins when every wave would fetch its own copy of more
// than 16 activation rows, or when K is long.
static int stream_waves(int m, int n, int k) {
    if (n >= 12288) return 4;
    if (m > 16 || k >= 4096) return 2;
    return 0;
}

// A slice's length is rounded up to the kernel's step along K; with a ragged K that can leave the
// last slices empty. The consumer adds every slice it was promised: fewer slices then, all of
// them non-empty.
static int whole_slices(int slices, int k, int step) {
    while (slices > 1) {
        const int k_per = ((k + slices - 1) / slices + step - 1) / step * step;
        if ((k + k_per - 1) / k_per == slices) break;
        slices /= 2;
    }
    return slices;
}

// Into how many slices of K a product may be cut when its consumer adds the slices. A weight
// with few rows gives too few blocks to keep the memory system busy otherwise (one CU draws
// about 50 GB/s at best, so it takes all of them): the measured optimum, with cold weights,
// is about 256 blocks, with at least 512 of K per slice and at most 8 slices.
extern "C" int imparo_gemm_slices(int m, int n, int k, int dtype) {
    if (dtype != IMPARO_BF16) return 1;
    if (m > 64) {
        const DmaPlan plan = dma_plan(m, n, k, 0);
        if (plan.tn) return plan.slices;
        // many rows: with about one tile of 128x128 per CU or fewer, a block has a CU to itself and
        // nothing hides its waits; slices of K (at least 1024 each, at most 4) multiply the blocks
        const long long tiles = (long long)((m + BG_BM - 1) / BG_BM) * ((n + BG_BN - 1) / BG_BN);
        int slices = 1;
        while (slices < 4 && tiles * slices * 2 <= 512 && k / (slices * 2) >= 1024) slices *= 2;
        return whole_slices(slices, k, BG_BK);
    }
    const int nw = stream_waves(m, n, k);
    const int rows_per_block = nw ? nw * 16 : 16;
    const int blocks = (n + rows_per_block - 1) / rows_per_block;
    int slices = 1;
    while (slices < 8 && blocks * slices * 2 <= 256 && k / (slices * 2) >= 512) slices *= 2;
    return whole_slices(slices, k, 128);
}

// Whether imparo_gemm takes the epilogue that adds the product to what Y holds (float32 out, K in one
// piece) for this shape: where the tile kernel with loads straight into LDS runs it.
extern "C" int imparo_gemm_adds(int m, int n, int k, int dtype) {
    return dtype == IMPARO_BF16 && m > 64 && dma_plan(m, n, k, 1).tn != 0;
}


// ------------------------------------------------------------------ bfloat16, some rows (17..64)
// A block of ST_WAVES waves takes 16 weight rows per wave and up to 16*MT
// activation rows, and walks its part of K in chunks of 128. The activation
// chunk is staged in LDS once per block and shared by the waves (with more
// than 16 rows every wave fetching its own activations costs several times the
// weight traffic); weights go from memory straight into the MFMA operand
// registers. Loads run three chunks ahead of the products: four register sets
// in rotation, the activation part of a set goes to LDS one step before its
// chunk is multiplied. With slices (gridDim.y > 1) block (x, y) sums K range
// [y * k_per, (y+1) * k_per) into Y + y * M * N and the consumer adds the slices.
#define ST_BK 128
#define ST_LD (ST_BK + 8)   // LDS row stride in elements: 272 bytes, 16 rows of 16-byte reads on distinct banks

template <int XP>
struct StreamSet {
    Frag8 w[4];       // this wave's weight rows, chunk columns s*32 + g*8
    uint4 x[XP];      // this thread's pieces of the activation chunk
};

// With ssq_in (at most 16 rows, K in one piece) the activations are the residual stream times a norm's
// weight, and each row's result is multiplied at the end by the row's scale rsqrt(sum of squares / K +
// eps) (rows.h): the partial sums are asked for at the start and needed only then.
template <typename TOut, int MT, int ST_WAVES>
__global__ __launch_bounds__(ST_WAVES * 64) void k_gemm_bf16_stream(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, const float* __restrict__ bias,
    TOut* __restrict__ Y, int M, int N, int K_all, int k_per, int epilogue, const float* __restrict__ ssq_in,
    int n_parts, float eps) {
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16 * ST_LD];
    __shared__ float norm_part[ST_WAVES * 4 * 16];
    RowsSsq early;
    if (ssq_in) rows_ssq_ask(early, ssq_in, n_parts, 0);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (ST_WAVES * 16) + wave * 16;
    const int k_lo = blockIdx.y * k_per;
    const int K = min(K_all, k_lo + k_per) - k_lo;       // this block's part of K, re-based to 0
    X += k_lo;
    W += k_lo;
    Y += (size_t)blockIdx.y * M * N;
    if (blockIdx.y > 0) bias = nullptr;                  // the bias belongs to one slice only
    const bf16_t* wrow = W + (size_t)min(n0 + r16, N - 1) * K_all;

    // the activation chunk: MT*16 rows x 16 pieces of 16 bytes, XP pieces per thread
    constexpr int PIECES = MT * 16 * (ST_BK / 8);
    constexpr int XP = (PIECES + ST_WAVES * 64 - 1) / (ST_WAVES * 64);
    const bf16_t* xsrc[XP];
    int xdst[XP], xkc[XP];
#pragma unroll
    for (int j = 0; j < XP; ++j) {
        const int p = min(tid + j * ST_WAVES * 64, PIECES - 1);
        const int row = p / (ST_BK / 8);
        xkc[j] = (p % (ST_BK / 8)) * 8;
        xsrc[j] = X + (size_t)min(row, M - 1) * K_all;
        xdst[j] = row * ST_LD + xkc[j];
    }
    const int nk = (K + ST_BK - 1) / ST_BK;
    // The walk along K is free of branches: a load under a branch, or a step under one, makes
    // the compiler wait for every load in flight at the next use of any. So every load is
    // issued unconditionally from an address clamped into the row, what a chunk reads at or
    // beyond K is zeroed before use, and the number of steps is rounded up to the four
    // register sets (a chunk past the end reads the last one again and counts as zeros).
    // Blocks start their walk at different chunks and wrap around: rows are a power of two
    // apart in memory, so blocks in step would ask the same few cache channels for the same
    // activation chunk at the same time.
    const int rot = (blockIdx.x + blockIdx.y) % nk;
    auto chunk_of = [&](int kt) {                        // kt >= nk: past the end
        const int c = kt + rot;
        return kt >= nk ? kt : (c >= nk ? c - nk : c);
    };
    auto fetch = [&](int kt, StreamSet<XP>& f) {
        const int k0 = min(chunk_of(kt), nk - 1) * ST_BK;
#pragma unroll
        for (int s2 = 0; s2 < 4; ++s2)
            f.w[s2].u = *reinterpret_cast<const uint4*>(wrow + min(k0 + s2 * 32 + g * 8, K - 8));
#pragma unroll
        for (int j = 0; j < XP; ++j) f.x[j] = *reinterpret_cast<const uint4*>(xsrc[j] + min(k0 + xkc[j], K - 8));
    };
    // (What an activation chunk holds at or beyond K is real data read again from inside the row; only
    // the weights there are zeroed, in `compute`: one select per weight value instead of one more per
    // activation value, which with 64 rows were a third of the kernel's vector instructions.)
    auto stash = [&](int buf, const StreamSet<XP>& f) {
#pragma unroll
        for (int j = 0; j < XP; ++j)     // threads beyond the last piece repeat it: same value, same place
            *reinterpret_cast<uint4*>(&xs[buf][xdst[j]]) = f.x[j];
    };
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    // The activation fragments of K-sub-step s2+1 are read from LDS while the products of
    // sub-step s2 run: a block may be alone on its CU, with nothing else to hide the LDS latency.
    auto read_x = [&](int buf, int s2, Frag8 (&xf)[MT]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            xf[mt].u = *reinterpret_cast<const uint4*>(&xs[buf][(mt * 16 + r16) * ST_LD + s2 * 32 + g * 8]);
    };
    auto multiply = [&](const Frag8& wf, const Frag8 (&xf)[MT]) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, xf[mt].v, acc[mt], 0, 0, 0);
    };
    auto compute = [&](int kt, int buf, const StreamSet<XP>& f) {
        const int k0 = chunk_of(kt) * ST_BK + g * 8;
        Frag8 xa[MT], xb[MT], wf;
        read_x(buf, 0, xa);
        read_x(buf, 1, xb);
        __builtin_amdgcn_sched_barrier(0);
        wf.u = zero_if(k0 >= K, f.w[0].u);
        multiply(wf, xa);
        read_x(buf, 2, xa);
        __builtin_amdgcn_sched_barrier(0);
        wf.u = zero_if(k0 + 32 >= K, f.w[1].u);
        multiply(wf, xb);
        read_x(buf, 3, xb);
        __builtin_amdgcn_sched_barrier(0);
        wf.u = zero_if(k0 + 64 >= K, f.w[2].u);
        multiply(wf, xa);
        __builtin_amdgcn_sched_barrier(0);
        wf.u = zero_if(k0 + 96 >= K, f.w[3].u);
        multiply(wf, xb);
    };
    // chunk i: the next chunk's activations go from their registers to LDS, the set that
    // chunk i-1 used takes the loads of chunk i+3, then chunk i is multiplied
    auto step = [&](int i, const StreamSet<XP>& cur, const StreamSet<XP>& next, StreamSet<XP>& refill) {
        const int buf = i & 1;
        stash(buf ^ 1, next);
        fetch(i + 3, refill);
        compute(i, buf, cur);
        __syncthreads();
    };
    StreamSet<XP> s0, s1, s2, s3;
    fetch(0, s0);
    fetch(1, s1);
    fetch(2, s2);
    stash(0, s0);
    __syncthreads();
    for (int kt = 0; kt < nk; kt += 4) {
        step(kt, s0, s1, s3);
        step(kt + 1, s1, s2, s0);
        step(kt + 2, s2, s3, s1);
        step(kt + 3, s3, s0, s2);
    }
    float row_scale = 1.f;
    if (ssq_in) {        // (rows beyond 16 have no sums: the host sends such products elsewhere)
        norm_part[(tid >> 4) * 16 + (tid & 15)] = rows_ssq_sum(early, ssq_in, n_parts);
        __syncthreads();
        row_scale = rows_scale(norm_part, min(r16, M - 1), K_all, eps);
    }
    // D layout of the 16x16 tile: lane holds column lane%16 (an activation row), rows 4*(lane/16)+i (weight rows)
    const int nq = n0 + g * 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r16;
        if (m >= M) continue;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            v[i] = (ssq_in ? __fmul_rn(acc[mt][i], row_scale) : acc[mt][i]) + ((bias && nq + i < N) ? bias[nq + i] : 0.f);
        if (epilogue == EPI_SWIGLU) {
#pragma unroll
            for (int i = 0; i < 4; i += 2)
                if (nq + i + 1 < N) store_f32<TOut>(Y, (size_t)m * (N / 2) + (nq + i) / 2, silu_mul_fast(v[i], v[i + 1]));
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (nq + i < N) store_f32<TOut>(Y, (size_t)m * N + nq + i, v[i]);
    }
}

template <typename TOut, int MT>
static void launch_stream(const bf16_t* x, const bf16_t* w, const float* bias, TOut* y, int m, int n, int k,
                          int epilogue, int nw, int slices, hipStream_t s, const float* ssq_in = nullptr,
                          int n_parts = 0, float eps = 0.f) {
    const int k_per = ((k + slices - 1) / slices + ST_BK - 1) / ST_BK * ST_BK;
    dim3 grid((unsigned)((n + nw * 16 - 1) / (nw * 16)), (unsigned)((k + k_per - 1) / k_per));
    if (nw == 8)
        k_gemm_bf16_stream<TOut, MT, 8><<<grid, 8 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue, ssq_in, n_parts, eps);
    else if (nw == 4)
        k_gemm_bf16_stream<TOut, MT, 4><<<grid, 4 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue, ssq_in, n_parts, eps);
    else
        k_gemm_bf16_stream<TOut, MT, 2><<<grid, 2 * 64, 0, s>>>(x, w, bias, y, m, n, k, k_per, epilogue, ssq_in, n_parts, eps);
}

// For the products of a step of at most 16 rows (decode_rows.hip): a weight of many rows is streamed
// faster by this kernel, whose waves share the activations, than by one block per 16 weight rows.
bool imparo_stream_rows_pays(int m, int n, int k) { return m <= 16 && stream_waves(m, n, k) == 4; }

int imparo_stream_rows(const bf16_t* x, const bf16_t* w, const float* bias, void* y, int out_dtype, int m, int n, int k,
                       int epilogue, const float* ssq_in, int n_parts, float eps, hipStream_t s) {
    const int nw = stream_waves(m, n, k);
    if (!nw || m > 16) return IMPARO_BAD_ARGUMENT;
    if (out_dtype == IMPARO_F32)
        launch_stream<float, 1>(x, w, bias, (float*)y, m, n, k, epilogue, nw, 1, s, ssq_in, n_parts, eps);
    else
        launch_stream<bf16_t, 1>(x, w, bias, (bf16_t*)y, m, n, k, epilogue, nw, 1, s, ssq_in, n_parts, eps);
    return launch_status();
}

// With a K that the kernel with loads straight into LDS does not take: the 256x256 tile with register
// staging (one block per CU) pays once its tiles keep most of the chip's 256 CUs busy: measured, from
// about 160 tiles on (192 tiles: +15% over 128x128; 96 tiles: -30%).
static bool big_tile_pays(int m, int n, int k) {
    (void)k;
    return (long long)((m + 255) / 256) * ((n + 255) / 256) >= 160;
}

template <typename TOut>
static int launch_bf16(const bf16_t* x, const bf16_t* w, const float* bias, TOut* y, int m, int n, int k, int epilogue,
                       int force, int slices, hipStream_t s) {
    // `force` (for measurements): 1 = K-split kernel, 2/4/8 = shared activations with that many waves
    // 452: the 128 by 128 tile on four stages, at any number of rows
    if (force == 452 && k % slices == 0 && (k / slices) % (4 * DM_BK) == 0 && dma_tile_takes(m, n, k))
        return launch_dma<TOut>(x, w, bias, y, m, n, k, epilogue, 128, 2, slices, s, 4);
    int nw = stream_waves(m, n, k);
    if (force == 1) nw = 0;
    if (force == 2 || force == 4 || force == 8) nw = force;
    if (m <= 64 && nw) {
        if (m <= 16)
            launch_stream<TOut, 1>(x, w, bias, y, m, n, k, epilogue, nw, slices, s);
        else if (m <= 32)
            launch_stream<TOut, 2>(x, w, bias, y, m, n, k, epilogue, nw, slices, s);
        else
            launch_stream<TOut, 4>(x, w, bias, y, m, n, k, epilogue, nw, slices, s);
        return launch_status();
    }
    if (m <= 64) {
        if (m <= 16)
            launch_skinny<TOut, 1>(x, w, bias, y, m, n, k, epilogue, slices, s);
        else if (m <= 32)
            launch_skinny<TOut, 2>(x, w, bias, y, m, n, k, epilogue, slices, s);
        else
            launch_skinny<TOut, 4>(x, w, bias, y, m, n, k, epilogue, slices, s);
    } else {
        // by shape: the tile kernel with loads straight into LDS where it takes the K, as its plan says;
        // `force` (for measurements) 256: the 256x256 tile with register staging
        if (force == 0) {
            const DmaPlan plan = dma_plan(m, n, k, slices);
            if (plan.tn)
                return launch_dma<TOut>(x, w, bias, y, m, n, k, epilogue, plan.bm, plan.tn, slices, s, plan.stages);
        }
        if (slices == 1 && (force == 256 || (force == 0 && big_tile_pays(m, n, k))))
            return launch_big<TOut, 2, 4, 4, 2>(x, w, bias, y, m, n, k, epilogue, s);
        // 258: the tile that loads straight into LDS, 256 wide; 262, 263: 128 and 192 wide
        if ((force == 258 || force == 262 || force == 263) && k % slices == 0 && dma_tile_takes(m, n, k / slices) &&
            dma_tile_takes(m, n, k))
            return launch_dma<TOut>(x, w, bias, y, m, n, k, epilogue, 256, force == 258 ? 4 : force - 260, slices, s);
        // 358, 352: 128 activation rows to a tile, 256 and 128 wide
        if ((force == 358 || force == 352) && k % slices == 0 && dma_tile_takes(m, n, k / slices) && dma_tile_takes(m, n, k))
            return launch_dma<TOut>(x, w, bias, y, m, n, k, epilogue, 128, force == 358 ? 4 : 2, slices, s);
        // 351, 451: 128 activation rows by 64 weight rows, on two stages and on four
        if ((force == 351 || force == 451) && k % slices == 0 && dma_tile_takes(m, n, k / slices) && dma_tile_takes(m, n, k) &&
            (force == 351 || (k / slices) % (4 * DM_BK) == 0))
            return launch_dma<TOut>(x, w, bias, y, m, n, k, epilogue, 128, 1, slices, s, force == 451 ? 4 : 2);
        const int tiles_m = (m + BG_BM - 1) / BG_BM, tiles_n = (n + BG_BN - 1) / BG_BN;
        const long long total = (long long)tiles_m * tiles_n;
        if (total > 0x7fffff00LL) return IMPARO_BAD_ARGUMENT;
        const unsigned blocks = (unsigned)(((total + N_XCD - 1) / N_XCD) * N_XCD);
        const int k_per = ((k + slices - 1) / slices + BG_BK - 1) / BG_BK * BG_BK;
        dim3 grid(blocks, (unsigned)((k + k_per - 1) / k_per));
        k_gemm_bf16_tile<TOut><<<grid, 256, 0, s>>>(x, w, bias, y, m, n, k, tiles_m, tiles_n, epilogue, k_per);
    }
    return launch_status();
}


// `variant` 0 lets the library choose the kernel. The others are for measurements and tests only, so
// that each kernel can be met at any shape: 1 the K-split kernel, 2, 4 or 8 the shared-activation
// kernel with that many waves, 256 the 256x256 tile with register staging, 258 / 263 / 262 the tile
// with loads straight into LDS at 256 rows by 256 / 192 / 128, 358 / 352 the same at 128 rows by
// 256 / 128, 452 the 128 by 128 tile on four stages, 351 / 451 the 128 by 64 tile on two / four stages;
// with a variant, any number of K slices is taken.
static int gemm_variant(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                        int m, int n, int k, int epilogue, int slices, int variant, imparo_stream stream) {
    if (!x || !w || !y || m < 0 || n <= 0 || k <= 0) return IMPARO_BAD_ARGUMENT;
    if (slices < 1) return IMPARO_BAD_ARGUMENT;
    // slices: only what imparo_gemm_slices allows, float32 out, no epilogue that is not linear
    const int slices_ok = imparo_gemm_slices(m, n, k, dtype);
    if (slices > 1 && ((slices != slices_ok && variant == 0) || out_dtype != IMPARO_F32 || epilogue != EPI_NONE))
        return IMPARO_BAD_ARGUMENT;
    if (epilogue != EPI_NONE && epilogue != EPI_SWIGLU && epilogue != EPI_ADD) return IMPARO_BAD_ARGUMENT;
    if (epilogue == EPI_SWIGLU && (n % 2 != 0)) return IMPARO_BAD_ARGUMENT;
    // adding into Y: the tile kernel that loads straight into LDS only, chosen by the library, K in one piece
    if (epilogue == EPI_ADD && (variant != 0 || slices != 1 || out_dtype != IMPARO_F32 || !imparo_gemm_adds(m, n, k, dtype)))
        return IMPARO_BAD_ARGUMENT;
    if (m == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32) {
        if (m <= 16 && out_dtype == IMPARO_F32) {
            k_gemm_f32_rows<float><<<(n + F32R_BN - 1) / F32R_BN, 256, 0, s>>>((const float*)x, (const float*)w, bias,
                                                                             (float*)y, m, n, k, epilogue);
            return launch_status();
        }
        if (m <= 16 && out_dtype == IMPARO_BF16) {
            k_gemm_f32_rows<bf16_t><<<(n + F32R_BN - 1) / F32R_BN, 256, 0, s>>>((const float*)x, (const float*)w, bias,
                                                                              (bf16_t*)y, m, n, k, epilogue);
            return launch_status();
        }
        dim3 grid((n + F32_BN - 1) / F32_BN, (m + F32_BM - 1) / F32_BM);
        if (grid.y > 65535) return IMPARO_BAD_ARGUMENT;
        if (out_dtype == IMPARO_F32)
            k_gemm_f32<float><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, bias, (float*)y, m, n, k, epilogue);
        else if (out_dtype == IMPARO_BF16)
            k_gemm_f32<bf16_t><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, bias, (bf16_t*)y, m, n, k, epilogue);
        else
            return IMPARO_BAD_ARGUMENT;
        return launch_status();
    }
    if (dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    // 16-byte loads along K: rows must start 16-byte aligned
    if (k % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return IMPARO_BAD_ARGUMENT;
    if (out_dtype == IMPARO_F32)
        return launch_bf16<float>((const bf16_t*)x, (const bf16_t*)w, bias, (float*)y, m, n, k, epilogue,
                                  variant, slices, s);
    if (out_dtype == IMPARO_BF16)
        return launch_bf16<bf16_t>((const bf16_t*)x, (const bf16_t*)w, bias, (bf16_t*)y, m, n, k, epilogue,
                                   variant, slices, s);
    return IMPARO_BAD_ARGUMENT;
}

extern "C" int imparo_gemm(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                           int m, int n, int k, int epilogue, int slices, imparo_stream stream) {
    return gemm_variant(x, w, bias, y, dtype, out_dtype, m, n, k, epilogue, slices, 0, stream);
}

extern "C" int imparo_gemm_variant(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                                   int m, int n, int k, int epilogue, int slices, int variant, imparo_stream stream) {
    return gemm_variant(x, w, bias, y, dtype, out_dtype, m, n, k, epilogue, slices, variant, stream);
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_gemm() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_gemm_f32_rows<float>)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
