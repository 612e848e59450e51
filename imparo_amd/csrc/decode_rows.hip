// Products for a step of at most 16 tokens (a decode step's rows), bfloat16 weights, with the work
// that surrounds a product on the residual stream folded into it, so that a layer of such a step is a
// chain of four to six launches instead of six to eight:
//
//   * the result may be added to the residual stream in place, and the block leaves the sum of
//     squares of its columns of the new rows: x += y, ssq[block][row] -- no add, and what the next
//     norm needs is there. Told the weight of the norm that reads the stream next, it also leaves
//     the new rows times that weight in bfloat16. A block adds the whole of K (no slices of K over
//     blocks): nothing meets across blocks, so there are no counters and no fences;
//   * the activations may be such rows (the stream times a norm's weight, not yet scaled) with the
//     partial sums of squares beside them: the block multiplies each row's result by the row's scale
//     rsqrt(sum / K + eps) at the end, in float32 -- no norm launch.
//
// The reference fuses the same neighbours: add + norm as one op, the gate/up pair with its
// activation (/root/reference/crates/imparo-backend/src/lib.rs:2603-2609, 1835-1869).
//
// A block takes RB weight rows (8 or 16: with 8 the matrix core's other eight rows repeat them,
// which costs nothing where memory is the bound, and a weight of 2,048 rows still makes 256
// blocks). Its NW waves split K in chunks of 128; a wave asks for all the weights of a round of
// CH chunks before it touches the activations. The block copies its activations into LDS once and
// its waves read them there (a block of 8 weight rows would otherwise ask the caches for twice as
// many activation bytes as weight bytes). Partial sums meet in LDS and are added in wave order.
#include "common.h"

#include <algorithm>
#include "api.h"
#include "rows.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

union RowFrag {
    uint4 u;
    bf16x8 v;
};

#define ROWS_STORE 0
#define ROWS_SWIGLU 1
#define ROWS_RESID 2

__device__ __forceinline__ float rows_silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * g)) * u;
}

// XLDS: the activations go through LDS (they fit there); else every wave loads its chunks from memory.
template <typename TOut, int RB, int NW, int CH, int EPI, bool XLDS>
__global__ __launch_bounds__(NW * 64) void k_rows_gemm(
    const bf16_t* __restrict__ X, const float* __restrict__ ssq_in, int n_parts, float eps,
    const bf16_t* __restrict__ W, const float* __restrict__ bias, TOut* __restrict__ Y, float* __restrict__ x_io,
    float* __restrict__ ssq_out, bf16_t* __restrict__ weighted_out, const float* __restrict__ weighted_by, int M, int N,
    int K) {
    __shared__ float red[NW][64][4];
    __shared__ float part[NW * 4 * 16];
    extern __shared__ __attribute__((aligned(16))) bf16_t staged[];     // XLDS: [M][K + 8]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * RB;
    const bf16_t* wrow = W + (size_t)min(n0 + (r16 & (RB - 1)), N - 1) * K;
    const int token = min(r16, M - 1);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const int n_chunks = (K + 127) / 128;
    // what the finishing lanes add to is asked for first: it has arrived long before the walk is over
    float x_old[4] = {0.f, 0.f, 0.f, 0.f}, by[4] = {0.f, 0.f, 0.f, 0.f};
    if (EPI == ROWS_RESID && wave == 0 && g * 4 < RB && r16 < M) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = min(n0 + g * 4 + i, N - 1);
            x_old[i] = x_io[(size_t)r16 * N + n];
            if (weighted_by) by[i] = weighted_by[n];
        }
    }
    RowFrag wf[CH][4];
    // This wave's turns are wave, wave + NW, ...: CH of them a round; turn c takes chunk c of K, 128 wide.
    // (Every block walks K in the same order, so a column's sum does not depend on which block has it.)
    auto load_weights = [&](int first) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int k0 = (first + j * NW) * 128;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int k = k0 + s * 32 + g * 8;
                // (lanes of weight rows beyond RB ask for nothing: their rows of the tile are nobody's)
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (r16 < RB) v = *reinterpret_cast<const uint4*>(wrow + min(k, K - 8));
                wf[j][s].u = make_uint4(k < K ? v.x : 0u, k < K ? v.y : 0u, k < K ? v.z : 0u, k < K ? v.w : 0u);
            }
        }
    };
    load_weights(wave);
    RowsSsq early;
    if (ssq_in) rows_ssq_ask(early, ssq_in, n_parts, 0);      // asked for now, needed when the walk is over
    if (XLDS) {
        // 16-byte pieces, each block starting its copy somewhere else (blocks in step would ask the
        // same few cache channels for the same piece at the same time)
        const int per_row = K / 8, pieces = M * per_row;
        const int start = (int)((blockIdx.x * 1031u) % (unsigned)pieces);
        for (int p0 = 0; p0 < pieces; p0 += NW * 64 * 4) {
            uint4 v[4];
            int at[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int q = p0 + (int)threadIdx.x + j * NW * 64;
                int p = min(q, pieces - 1) + start;
                p = p >= pieces ? p - pieces : p;
                const int row = p / per_row, col = (p - row * per_row) * 8;
                at[j] = q < pieces ? row * (K + 8) + col : -1;
                v[j] = *reinterpret_cast<const uint4*>(X + (size_t)row * K + col);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (at[j] >= 0) *reinterpret_cast<uint4*>(&staged[at[j]]) = v[j];
        }
        __syncthreads();
    }
    for (int first = wave; first < n_chunks; first += NW * CH) {
        if (first != wave) load_weights(first);
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const int k0 = (first + j * NW) * 128;
            RowFrag xa[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                // what lies at or beyond K meets zero weights: any finite activation will do there
                const int k = min(k0 + s * 32 + g * 8, K - 8);
                if (XLDS) {
                    xa[s].u = make_uint4(0u, 0u, 0u, 0u);       // (likewise the lanes of tokens beyond M)
                    if (r16 < M) xa[s].u = *reinterpret_cast<const uint4*>(&staged[(size_t)token * (K + 8) + k]);
                } else {
                    xa[s].u = *reinterpret_cast<const uint4*>(X + (size_t)token * K + k);
                }
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[j][s].v, xa[s].v, acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][lane][i] = acc[i];
    if (ssq_in) part[(threadIdx.x >> 4) * 16 + (threadIdx.x & 15)] = rows_ssq_sum(early, ssq_in, n_parts);
    __syncthreads();
    if (wave != 0 || g * 4 >= RB) return;
    // D layout of the 16x16 tile: lane holds column lane % 16 (a token), rows 4 * (lane / 16) + i (weight rows)
    const float scale = ssq_in ? rows_scale(part, token, K, eps) : 1.f;
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[i] = red[0][lane][i];
#pragma unroll
        for (int w = 1; w < NW; ++w) v[i] += red[w][lane][i];
        // each step rounded on its own (no fused multiply-add), so that every epilogue gives the same bits
        v[i] = __fmul_rn(v[i], scale);
        const int n = n0 + g * 4 + i;
        if (bias && n < N) v[i] = __fadd_rn(v[i], bias[n]);
    }
    const bool live = r16 < M;
    if (EPI == ROWS_SWIGLU) {
        if (!live) return;
#pragma unroll
        for (int i = 0; i < 4; i += 2) {
            const int n = n0 + g * 4 + i;
            if (n + 1 < N) store_f32<TOut>(Y, (size_t)r16 * (N / 2) + n / 2, rows_silu_mul(v[i], v[i + 1]));
        }
        return;
    }
    if (EPI == ROWS_STORE) {
        if (!live) return;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + g * 4 + i;
            if (n < N) store_f32<TOut>(Y, (size_t)r16 * N + n, v[i]);
        }
        return;
    }
    // ROWS_RESID: the stream takes the result; the block leaves the sum of squares of its columns
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int n = n0 + g * 4 + i;
        if (live && n < N) {
            const float xn = __fadd_rn(x_old[i], v[i]);
            x_io[(size_t)r16 * N + n] = xn;
            sq = fmaf(xn, xn, sq);
            if (weighted_out) weighted_out[(size_t)r16 * N + n] = f32_to_bf16(xn * by[i]);
        }
    }
    // the lanes of one token sit 16 apart: 2 of them for 8 weight rows, 4 for 16 (all of them are here)
    sq += __shfl_xor(sq, 16, WAVE);
    if (RB == 16) sq += __shfl_xor(sq, 32, WAVE);
    if (g == 0) ssq_out[(size_t)blockIdx.x * ROWS_PARTS + r16] = sq;
}

// How the waves of a block share K: few chunks of 128 a wave, all of a round's weights asked for at once.
struct RowsShape {
    int nw, ch;
};
static RowsShape rows_shape(int k) {
    const int chunks = (k + 127) / 128;
    if (chunks <= 4) return {4, 1};
    if (chunks <= 8) return {8, 1};
    if (chunks <= 16) return {8, 2};
    if (chunks <= 32) return {8, 4};
    return {16, 4};
}

#define ROWS_XLDS_BYTES (136 * 1024)      // LDS a block may spend on a copy of its activations (a CU has 160 KB, and
                                          // the sums that meet at the end take up to 20 KB of it)

template <typename TOut, int RB, int EPI>
static void rows_launch(const bf16_t* X, const float* ssq_in, int n_parts, float eps, const bf16_t* W, const float* bias,
                        TOut* Y, float* x_io, float* ssq_out, bf16_t* weighted_out, const float* weighted_by, int M,
                        int N, int K, hipStream_t s) {
    const unsigned blocks = (unsigned)((N + RB - 1) / RB);
    const size_t x_bytes = (size_t)M * (K + 8) * sizeof(bf16_t);
    const bool xlds = x_bytes <= ROWS_XLDS_BYTES;
    const size_t lds = xlds ? x_bytes : 0;
    const RowsShape sh = rows_shape(K);
#define ROWS_GO2(NW, CH, XL)                                                                                         \
    do {                                                                                                             \
        auto kern = k_rows_gemm<TOut, RB, NW, CH, EPI, XL>;                                                          \
        if (lds > 64 * 1024 &&                                                                                       \
            hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) \
            return;   /* the error stays for launch_status() */                                                      \
        kern<<<blocks, NW * 64, lds, s>>>(X, ssq_in, n_parts, eps, W, bias, Y, x_io, ssq_out, weighted_out,          \
                                          weighted_by, M, N, K);                                                     \
    } while (0)
#define ROWS_GO(NW, CH)                                                                                              \
    do {                                                                                                             \
        if (xlds) ROWS_GO2(NW, CH, true);                                                                            \
        else ROWS_GO2(NW, CH, false);                                                                                \
    } while (0)
    if (sh.nw == 4) ROWS_GO(4, 1);
    else if (sh.nw == 8 && sh.ch == 1) ROWS_GO(8, 1);
    else if (sh.nw == 8 && sh.ch == 2) ROWS_GO(8, 2);
    else if (sh.nw == 8) ROWS_GO(8, 4);
    else ROWS_GO(16, 4);
#undef ROWS_GO
#undef ROWS_GO2
}

// blocks of a ROWS_RESID product with `n` weight rows: the partial sums of squares it leaves
extern "C" int imparo_rows_parts(int n) { return (n + 7) / 8; }

extern "C" int imparo_rows_gemm(const void* x, const float* ssq_in, int n_parts, float eps, const void* w,
                                const float* bias, void* y, int out_dtype, float* x_io, float* ssq_out,
                                void* weighted_out, const float* weighted_by, int m, int n, int k, int epilogue,
                                imparo_stream stream) {
    if (!x || !w || m < 0 || m > ROWS_MAX || n <= 0 || k <= 0 || k % 8 != 0) return IMPARO_BAD_ARGUMENT;
    if (ssq_in && (n_parts <= 0 || !(eps > 0.f))) return IMPARO_BAD_ARGUMENT;
    if (((uintptr_t)w & 15) || ((uintptr_t)x & 15)) return IMPARO_BAD_ARGUMENT;
    if (epilogue == ROWS_RESID) {
        if (!x_io || !ssq_out || ((weighted_out == nullptr) != (weighted_by == nullptr))) return IMPARO_BAD_ARGUMENT;
    } else if (epilogue == ROWS_STORE || epilogue == ROWS_SWIGLU) {
        if (!y || (out_dtype != IMPARO_F32 && out_dtype != IMPARO_BF16)) return IMPARO_BAD_ARGUMENT;
        if (epilogue == ROWS_SWIGLU && n % 2 != 0) return IMPARO_BAD_ARGUMENT;
    } else {
        return IMPARO_BAD_ARGUMENT;
    }
    if (m == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const bf16_t* xb = (const bf16_t*)x;
    const bf16_t* wb = (const bf16_t*)w;
    bf16_t* wo = (bf16_t*)weighted_out;
    // a weight of many rows: the kernel that shares the activations between a block's waves (gemm.hip)
    // streams such a weight faster
    if (epilogue != ROWS_RESID && imparo_stream_rows_pays(m, n, k))
        return imparo_stream_rows(xb, wb, bias, y, out_dtype, m, n, k, epilogue, ssq_in, n_parts, eps, s);
    if (epilogue == ROWS_RESID)
        rows_launch<float, 8, ROWS_RESID>(xb, ssq_in, n_parts, eps, wb, bias, nullptr, x_io, ssq_out, wo, weighted_by, m,
                                          n, k, s);
    else if (epilogue == ROWS_SWIGLU && out_dtype == IMPARO_BF16)
        rows_launch<bf16_t, 16, ROWS_SWIGLU>(xb, ssq_in, n_parts, eps, wb, bias, (bf16_t*)y, nullptr, nullptr, nullptr,
                                             nullptr, m, n, k, s);
    else if (epilogue == ROWS_SWIGLU)
        rows_launch<float, 16, ROWS_SWIGLU>(xb, ssq_in, n_parts, eps, wb, bias, (float*)y, nullptr, nullptr, nullptr,
                                            nullptr, m, n, k, s);
    else if (out_dtype == IMPARO_BF16)
        rows_launch<bf16_t, 16, ROWS_STORE>(xb, ssq_in, n_parts, eps, wb, bias, (bf16_t*)y, nullptr, nullptr, nullptr,
                                            nullptr, m, n, k, s);
    else
        rows_launch<float, 16, ROWS_STORE>(xb, ssq_in, n_parts, eps, wb, bias, (float*)y, nullptr, nullptr, nullptr,
                                           nullptr, m, n, k, s);
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_decode_rows() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_rows_gemm<float, 8, 4, 1, ROWS_RESID, true>)) ==
                   hipSuccess
               ? IMPARO_OK
               : IMPARO_LAUNCH_FAILED;
}
