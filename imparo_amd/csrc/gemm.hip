// Y[m, n] = X[m, k] . W[n, k]^T with float32 accumulation.
//
// float32: a register-tiled FMA kernel; every output element sums its products
// in the order k = 0, 1, 2, ... whatever the tile it falls in, so a row's
// result does not depend on how many other rows are in the batch.
// bfloat16: MFMA kernels, a 128x128 LDS-tiled one for many rows and a
// weight-streaming one with the K range split over the waves of a block for
// few rows (decode).
#include "common.h"
#include "api.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

union Frag8 {
    uint4 u;
    bf16x8 v;
};

// ------------------------------------------------------------------ float32
#define F32_BM 64
#define F32_BN 64
#define F32_BK 16

template <typename TOut>
__global__ __launch_bounds__(256) void k_gemm_f32(const float* __restrict__ X, const float* __restrict__ W,
                                                  TOut* __restrict__ Y, int M, int N, int K) {
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
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) store_f32<TOut>(Y, (size_t)m * N + n, acc[i][j]);
        }
    }
}

// ------------------------------------------------------------------ bfloat16, many rows
#define BG_BM 128
#define BG_BN 128
#define BG_BK 32
#define BG_LD 40   // LDS row stride in elements: 80 bytes keeps 16-byte reads of 16 rows on distinct banks

template <typename TOut>
__global__ __launch_bounds__(256) void k_gemm_bf16_tile(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                        TOut* __restrict__ Y, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) bf16_t As[2][BG_BM * BG_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[2][BG_BN * BG_LD];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BG_BM, n0 = blockIdx.x * BG_BN;

    // this thread's two 16-byte pieces of each operand tile
    const bf16_t* pa[2];
    const bf16_t* pb[2];
    int lds_off[2], kc8[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int c = tid + j * 256;
        const int row = c >> 2;
        kc8[j] = (c & 3) * 8;
        pa[j] = X + (size_t)min(m0 + row, M - 1) * K + kc8[j];
        pb[j] = W + (size_t)min(n0 + row, N - 1) * K + kc8[j];
        lds_off[j] = row * BG_LD + kc8[j];
    }
    const int nk = (K + BG_BK - 1) / BG_BK;
    uint4 ra[2], rb[2];
    const uint4 zero = make_uint4(0, 0, 0, 0);

    auto fetch = [&](int kt) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const bool in = kt * BG_BK + kc8[j] < K;
            ra[j] = in ? *reinterpret_cast<const uint4*>(pa[j] + (size_t)kt * BG_BK) : zero;
            rb[j] = in ? *reinterpret_cast<const uint4*>(pb[j] + (size_t)kt * BG_BK) : zero;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            *reinterpret_cast<uint4*>(&As[buf][lds_off[j]]) = ra[j];
            *reinterpret_cast<uint4*>(&Bs[buf][lds_off[j]]) = rb[j];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    fetch(0);
    stash(0);
    __syncthreads();
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) fetch(kt + 1);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            Frag8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i)
                a[i].u = *reinterpret_cast<const uint4*>(&As[buf][(wm * 64 + i * 32 + frag_row) * BG_LD + ks * 16 + frag_k]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                b[j].u = *reinterpret_cast<const uint4*>(&Bs[buf][(wn * 64 + j * 32 + frag_row) * BG_LD + ks * 16 + frag_k]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i].v, b[j].v, acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) stash(buf ^ 1);
        __syncthreads();
    }
    // D layout of the 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int n = n0 + wn * 64 + j * 32 + (lane & 31);
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (m < M) store_f32<TOut>(Y, (size_t)m * N + n, acc[i][j][r]);
            }
        }
}

// ------------------------------------------------------------------ bfloat16, few rows
// One block per 16 weight rows. Its waves split K in chunks of 128: wave w
// takes chunks w, w + n_waves, ... so the block reads each weight row as one
// contiguous stream. The 16 weight rows are the MFMA's M side, up to 16*MT
// activation rows its N side. Partial sums meet in LDS and are added in wave
// order, so the result is the same from run to run.
#define SK_WAVES 4
template <typename TOut, int MT>
__global__ __launch_bounds__(SK_WAVES * 64) void k_gemm_bf16_skinny(const bf16_t* __restrict__ X,
                                                                    const bf16_t* __restrict__ W,
                                                                    TOut* __restrict__ Y, int M, int N, int K) {
    __shared__ float red[SK_WAVES][MT][64][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 16;
    const int r16 = lane & 15, g = lane >> 4;
    const bf16_t* wrow = W + (size_t)min(n0 + r16, N - 1) * K + g * 8;
    const bf16_t* xrow[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) xrow[mt] = X + (size_t)min(mt * 16 + r16, M - 1) * K + g * 8;
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    const uint4 zero = make_uint4(0, 0, 0, 0);

    for (int k0 = wave * 128; k0 < K; k0 += SK_WAVES * 128) {
        Frag8 wf[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int k = k0 + s * 32;
            wf[s].u = (k + g * 8 < K) ? *reinterpret_cast<const uint4*>(wrow + k) : zero;
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int k = k0 + s * 32;
                Frag8 xf;
                xf.u = (k + g * 8 < K) ? *reinterpret_cast<const uint4*>(xrow[mt] + k) : zero;
                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s].v, xf.v, acc[mt], 0, 0, 0);
            }
        }
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
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = red[0][mt][lane][i];
#pragma unroll
            for (int w = 1; w < SK_WAVES; ++w) v += red[w][mt][lane][i];
            const int n = n0 + g * 4 + i;
            if (m < M && n < N) store_f32<TOut>(Y, (size_t)m * N + n, v);
        }
    }
}

template <typename TOut>
static int launch_bf16(const bf16_t* x, const bf16_t* w, TOut* y, int m, int n, int k, hipStream_t s) {
    if (m <= 64) {
        const unsigned blocks = (unsigned)((n + 15) / 16);
        if (m <= 16)
            k_gemm_bf16_skinny<TOut, 1><<<blocks, SK_WAVES * 64, 0, s>>>(x, w, y, m, n, k);
        else if (m <= 32)
            k_gemm_bf16_skinny<TOut, 2><<<blocks, SK_WAVES * 64, 0, s>>>(x, w, y, m, n, k);
        else
            k_gemm_bf16_skinny<TOut, 4><<<blocks, SK_WAVES * 64, 0, s>>>(x, w, y, m, n, k);
    } else {
        dim3 grid((n + BG_BN - 1) / BG_BN, (m + BG_BM - 1) / BG_BM);
        if (grid.y > 65535) return IMPARO_BAD_ARGUMENT;
        k_gemm_bf16_tile<TOut><<<grid, 256, 0, s>>>(x, w, y, m, n, k);
    }
    return launch_status();
}

extern "C" int imparo_gemm(const void* x, const void* w, void* y, int dtype, int out_dtype,
                           int m, int n, int k, imparo_stream stream) {
    if (!x || !w || !y || m < 0 || n <= 0 || k <= 0) return IMPARO_BAD_ARGUMENT;
    if (m == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32) {
        dim3 grid((n + F32_BN - 1) / F32_BN, (m + F32_BM - 1) / F32_BM);
        if (grid.y > 65535) return IMPARO_BAD_ARGUMENT;
        if (out_dtype == IMPARO_F32)
            k_gemm_f32<float><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, (float*)y, m, n, k);
        else if (out_dtype == IMPARO_BF16)
            k_gemm_f32<bf16_t><<<grid, 256, 0, s>>>((const float*)x, (const float*)w, (bf16_t*)y, m, n, k);
        else
            return IMPARO_BAD_ARGUMENT;
        return launch_status();
    }
    if (dtype != IMPARO_BF16) return IMPARO_BAD_ARGUMENT;
    // 16-byte loads along K: rows must start 16-byte aligned
    if (k % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15)) return IMPARO_BAD_ARGUMENT;
    if (out_dtype == IMPARO_F32) return launch_bf16<float>((const bf16_t*)x, (const bf16_t*)w, (float*)y, m, n, k, s);
    if (out_dtype == IMPARO_BF16) return launch_bf16<bf16_t>((const bf16_t*)x, (const bf16_t*)w, (bf16_t*)y, m, n, k, s);
    return IMPARO_BAD_ARGUMENT;
}
