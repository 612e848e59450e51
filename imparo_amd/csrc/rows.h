// Shared by the kernels for steps of at most 16 tokens in which a norm of the residual stream is
// folded into the products around it: the product that adds its result to the stream leaves the
// partial sums of squares of the new rows and the rows times the next norm's weight in bfloat16;
// the product behind that norm runs on those rows and multiplies each row's result at the end by
// scale[t] = rsqrt(sum_p ssq[p][t] / width + eps). The scale is one number a row, so the walk along
// K does not wait for the sums, and there is no launch for the norm.
#pragma once
#include "common.h"

#define ROWS_MAX 16          // tokens of a step these kernels take
#define ROWS_PARTS 16        // floats per partial sum of squares: one per token
#define ROWS_ASK 8           // partial sums a thread has in flight at once

struct RowsSsq {
    float v[ROWS_ASK];
};

// Thread i gathers the partials p = first + i / 16, + threads / 16, ... of token i % 16.
__device__ __forceinline__ void rows_ssq_ask(RowsSsq& r, const float* __restrict__ ssq, int n_parts, int first) {
    const int t = threadIdx.x & 15, group = threadIdx.x >> 4, groups = blockDim.x >> 4;
#pragma unroll
    for (int j = 0; j < ROWS_ASK; ++j) {
        const int p = first + group + j * groups;
        const float v = ssq[(size_t)min(p, n_parts - 1) * ROWS_PARTS + t];
        r.v[j] = p < n_parts ? v : 0.f;
    }
}

// This thread's share of its token's sum, in the order of the partials: `early` holds the first
// round, asked for before the walk along K; further rounds are fetched here.
__device__ __forceinline__ float rows_ssq_sum(const RowsSsq& early, const float* __restrict__ ssq, int n_parts) {
    const int groups = blockDim.x >> 4;
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < ROWS_ASK; ++j) s += early.v[j];
    for (int first = ROWS_ASK * groups; first < n_parts; first += ROWS_ASK * groups) {
        RowsSsq r;
        rows_ssq_ask(r, ssq, n_parts, first);
#pragma unroll
        for (int j = 0; j < ROWS_ASK; ++j) s += r.v[j];
    }
    return s;
}

// After every thread has put its share at part[thread / 16][thread % 16] and the block has met:
// the groups' shares are added in group order.
__device__ __forceinline__ float rows_scale(const float* part, int token, int width, float eps) {
    const int groups = blockDim.x >> 4;
    float total = 0.f;
    for (int gi = 0; gi < groups; ++gi) total += part[gi * 16 + token];
    return 1.0f / sqrtf(total / (float)width + eps);
}

// (gemm.hip) The kernel whose waves share the activations through LDS, for at most 16 rows, with the
// rows' scales from their sums of squares applied at the end (ssq_in null: none): whether it is the
// faster one for a shape, and the launch. epilogue 0 or 1 (SwiGLU); out_dtype as in the C API.
bool imparo_stream_rows_pays(int m, int n, int k);
int imparo_stream_rows(const bf16_t* x, const bf16_t* w, const float* bias, void* y, int out_dtype, int m, int n, int k,
                       int epilogue, const float* ssq_in, int n_parts, float eps, hipStream_t s);
