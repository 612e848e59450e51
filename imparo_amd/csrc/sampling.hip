// Picking the next token from float32 logits: argmax (smallest index at the
// maximum, NaN never wins) and temperature sampling by inverse CDF.
#include "common.h"
#include "api.h"
#include <limits.h>

struct Best {
    float v;
    int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

__device__ __forceinline__ Best block_best(Best b, Best* scratch) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Best o;
        o.v = __shfl_xor(b.v, off, WAVE);
        o.i = __shfl_xor(b.i, off, WAVE);
        b = better(b, o);
    }
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
    __syncthreads();
    if (lane == 0) scratch[wave] = b;
    __syncthreads();
    Best r = scratch[0];
    for (int w = 1; w < n_waves; ++w) r = better(r, scratch[w]);
    return r;
}

__device__ __forceinline__ Best row_best(const float* __restrict__ row, int vocab, Best* scratch) {
    Best b;
    b.v = -INFINITY;
    b.i = INT_MAX;
    if ((vocab & 3) == 0 && (((uintptr_t)row) & 15) == 0) {
        // four values a load, four loads in flight; a thread meets its indices in ascending
        // order, so "greater than" alone keeps the smallest index at the maximum
        // (sixteen loads in flight: a row of 65,536 on 1,024 threads is one trip to memory, not four;
        // no load sits under a branch: past the end the row's last piece is read again and not counted)
        const float4* row4 = reinterpret_cast<const float4*>(row);
        const int n4 = vocab >> 2;
        constexpr int DEEP = 16;
        for (int first = threadIdx.x; first < n4; first += DEEP * (int)blockDim.x) {
            float4 v[DEEP];
#pragma unroll
            for (int k = 0; k < DEEP; ++k) v[k] = row4[min(first + k * (int)blockDim.x, n4 - 1)];
#pragma unroll
            for (int k = 0; k < DEEP; ++k) {
                const int i = first + k * (int)blockDim.x;
                const float vs[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (i < n4 && (vs[j] > b.v || (vs[j] == b.v && 4 * i + j < b.i))) {
                        b.v = vs[j];
                        b.i = 4 * i + j;
                    }
            }
        }
    } else {
        for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
            const float v = row[i];
            if (v > b.v || (v == b.v && i < b.i)) {
                b.v = v;
                b.i = i;
            }
        }
    }
    b = block_best(b, scratch);
    if (b.i == INT_MAX) b.i = 0;   // every value was NaN
    return b;
}

__global__ void k_argmax_rows(const float* __restrict__ logits, int32_t* __restrict__ out, int vocab) {
    __shared__ Best scratch[16];
    const Best b = row_best(logits + (size_t)blockIdx.x * vocab, vocab, scratch);
    if (threadIdx.x == 0) out[blockIdx.x] = b.i;
}

extern "C" int imparo_argmax_rows(const float* logits, int32_t* out, int n_rows, int vocab, imparo_stream stream) {
    if (!logits || !out || n_rows < 0 || vocab <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    const int threads = vocab >= 16384 ? 1024 : 256;
    k_argmax_rows<<<n_rows, threads, 0, (hipStream_t)stream>>>(logits, out, vocab);
    return launch_status();
}

// Each thread owns one contiguous piece of the row. Piece sums are scanned in
// thread order, the piece holding u * total is walked element by element: the
// pick is the first index whose running sum exceeds the target.
__global__ void k_sample_rows(const float* __restrict__ logits, const float* __restrict__ temperature,
                              const float* __restrict__ uniform, int32_t* __restrict__ out, int vocab) {
    __shared__ Best scratch[16];
    __shared__ float sums[1024];
    __shared__ int owner;
    __shared__ float owner_prefix;
    const float* row = logits + (size_t)blockIdx.x * vocab;
    const Best top = row_best(row, vocab, scratch);
    const float temp = temperature[blockIdx.x];
    if (!(temp > 0.f)) {
        if (threadIdx.x == 0) out[blockIdx.x] = top.i;
        return;
    }
    const float inv_t = 1.0f / temp;
    const int piece = (vocab + blockDim.x - 1) / blockDim.x;
    const int begin = min(vocab, (int)threadIdx.x * piece);
    const int end = min(vocab, begin + piece);
    float local = 0.f;
    for (int i = begin; i < end; ++i) {
        const float e = expf((row[i] - top.v) * inv_t);
        if (e == e) local += e;   // a NaN logit has probability zero
    }
    sums[threadIdx.x] = local;
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.f;
        for (int t = 0; t < (int)blockDim.x; ++t) total += sums[t];
        const float target = uniform[blockIdx.x] * total;
        float prefix = 0.f;
        int pick = -1, last = 0;
        float last_prefix = 0.f;
        for (int t = 0; t < (int)blockDim.x; ++t) {
            if (sums[t] > 0.f) {
                last = t;
                last_prefix = prefix;
                if (prefix + sums[t] > target) {
                    pick = t;
                    break;
                }
            }
            prefix += sums[t];
        }
        if (pick < 0) {   // rounding pushed the target past the total
            pick = last;
            prefix = last_prefix;
        }
        owner = pick;
        owner_prefix = prefix;
        // stash the target where the owner finds it
        sums[0] = target;
    }
    __syncthreads();
    if ((int)threadIdx.x != owner) return;
    const float target = sums[0];
    float cum = owner_prefix;
    int pick = -1, last = top.i;
    for (int i = begin; i < end; ++i) {
        const float e = expf((row[i] - top.v) * inv_t);
        if (!(e > 0.f)) continue;
        last = i;
        cum += e;
        if (cum > target) {
            pick = i;
            break;
        }
    }
    out[blockIdx.x] = pick >= 0 ? pick : last;
}

extern "C" int imparo_sample_rows(const float* logits, const float* temperature, const float* uniform, int32_t* out,
                                  int n_rows, int vocab, imparo_stream stream) {
    if (!logits || !temperature || !uniform || !out || n_rows < 0 || vocab <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    const int threads = vocab >= 16384 ? 1024 : 256;
    k_sample_rows<<<n_rows, threads, 0, (hipStream_t)stream>>>(logits, temperature, uniform, out, vocab);
    return launch_status();
}

// The hash of the sources this library was built from (given by the build), so that a
// library older than its sources is noticed when it is loaded.
#ifndef IMPARO_SOURCE_HASH
#define IMPARO_SOURCE_HASH "unknown"
#endif
extern "C" const char* imparo_hip_source_hash() { return IMPARO_SOURCE_HASH; }

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_sampling() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_argmax_rows)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
