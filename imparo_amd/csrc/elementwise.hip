// Row-wise and element-wise kernels: embedding gather, RMS norm (with the
// residual add fused in), SiLU gating, bias, fill, and the gated short
// convolution with its per-request state.
#include "common.h"
#include "api.h"

// ---------------------------------------------------------------- embedding
template <typename T>
__global__ void k_embed_gather(const T* __restrict__ table, const int32_t* __restrict__ ids,
                               float* __restrict__ x, int width) {
    const int t = blockIdx.x;
    const size_t src = (size_t)ids[t] * width;
    const size_t dst = (size_t)t * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) x[dst + i] = load_f32<T>(table, src + i);
}

extern "C" int imparo_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x,
                                   int n_tokens, int width, int vocab, imparo_stream stream) {
    if (!table || !ids || !x || n_tokens < 0 || width <= 0 || vocab <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const int threads = width >= 1024 ? 256 : 64;
    if (table_dtype == IMPARO_F32)
        k_embed_gather<float><<<n_tokens, threads, 0, s>>>((const float*)table, ids, x, width);
    else if (table_dtype == IMPARO_BF16)
        k_embed_gather<bf16_t><<<n_tokens, threads, 0, s>>>((const bf16_t*)table, ids, x, width);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// Token ids that are still on the device (sampled by the step before, not yet read back):
// ids[dst[i]] = src[src_index[i]], clamped into the vocabulary.
__global__ void k_place_tokens(int32_t* __restrict__ ids, const int32_t* __restrict__ dst,
                               const int32_t* __restrict__ src, const int32_t* __restrict__ src_index, int n,
                               int vocab) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) ids[dst[i]] = min(max(src[src_index[i]], 0), vocab - 1);
}

extern "C" int imparo_place_tokens(int32_t* ids, const int32_t* dst, const int32_t* src, const int32_t* src_index,
                                   int n, int vocab, imparo_stream stream) {
    if (!ids || !dst || !src || !src_index || n < 0 || vocab <= 0) return IMPARO_BAD_ARGUMENT;
    if (n == 0) return IMPARO_OK;
    k_place_tokens<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(ids, dst, src, src_index, n, vocab);
    return launch_status();
}

// ---------------------------------------------------------------- RMS norm
// One block per output row. Sum of squares in float32, reduced in an order
// fixed by the block size. Two passes over the row; the second re-reads what
// the first left in registers when the row fits (width <= 8 * blockDim).
template <typename TOut, int PER_THREAD>
__global__ void k_rms_norm(float* __restrict__ x, const float* __restrict__ delta, int n_delta, size_t delta_stride,
                           const int32_t* __restrict__ rows, const float* __restrict__ weight,
                           TOut* __restrict__ out, int width, float eps, int write_back) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[i_out] : i_out) * width;
    const size_t dst = (size_t)i_out * width;
    float v[PER_THREAD];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        float a = 0.f;
        if (i < width) {
            a = x[src + i];
            float d = 0.f;                   // the slices make up the delta first, then the delta joins x
            for (int s = 0; s < n_delta; ++s) d += delta[s * delta_stride + src + i];
            a += d;
            if (write_back) x[src + i] = a;
        }
        v[j] = a;
        ss += a * a;
    }
    // rows wider than PER_THREAD * blockDim: the tail is not kept in registers
    for (int i = threadIdx.x + PER_THREAD * blockDim.x; i < width; i += blockDim.x) {
        float a = x[src + i], d = 0.f;
        for (int s = 0; s < n_delta; ++s) d += delta[s * delta_stride + src + i];
        a += d;
        if (write_back) x[src + i] = a;
        ss += a * a;
    }
    const float total = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(total / (float)width + eps);
#pragma unroll
    for (int j = 0; j < PER_THREAD; ++j) {
        const int i = threadIdx.x + j * blockDim.x;
        if (i < width) store_f32<TOut>(out, dst + i, v[j] * scale * weight[i]);
    }
    for (int i = threadIdx.x + PER_THREAD * blockDim.x; i < width; i += blockDim.x) {
        float a = x[src + i];
        if (!write_back) {
            float d = 0.f;
            for (int s = 0; s < n_delta; ++s) d += delta[s * delta_stride + src + i];
            a += d;
        }
        store_f32<TOut>(out, dst + i, a * scale * weight[i]);
    }
}

// The same for rows whose width is a multiple of 4 and at most 4 * blockDim:
// one float4 per thread. Every load of the row is issued before anything
// waits, the slices of the delta four at a time from clamped addresses: what a
// decode step hands this kernel was written a moment ago by another kernel and
// is in no near cache, so a load that waits for the one before costs a trip to
// memory each.
template <typename TOut>
__global__ void k_rms_norm_v4(float* __restrict__ x, const float* __restrict__ delta, int n_delta, size_t delta_stride,
                              const int32_t* __restrict__ rows, const float* __restrict__ weight,
                              TOut* __restrict__ out, int width, float eps, int write_back) {
    __shared__ float scratch[16];
    const int i_out = blockIdx.x;
    const size_t src = (size_t)(rows ? rows[i_out] : i_out) * width;
    const size_t dst = (size_t)i_out * width;
    const bool in = (int)threadIdx.x * 4 < width;
    const int i = min((int)threadIdx.x * 4, width - 4);      // threads past the row repeat its end and store nothing
    float4 a = *reinterpret_cast<const float4*>(x + src + i);
    const float4 w = *reinterpret_cast<const float4*>(weight + i);
    float4 d = make_float4(0.f, 0.f, 0.f, 0.f);   // the slices make up the delta first, then the delta joins x
    for (int s0 = 0; s0 < n_delta; s0 += 4) {
        float4 p[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            p[j] = *reinterpret_cast<const float4*>(delta + (size_t)min(s0 + j, n_delta - 1) * delta_stride + src + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool on = s0 + j < n_delta;
            d.x += on ? p[j].x : 0.f;
            d.y += on ? p[j].y : 0.f;
            d.z += on ? p[j].z : 0.f;
            d.w += on ? p[j].w : 0.f;
        }
    }
    a.x += d.x;
    a.y += d.y;
    a.z += d.z;
    a.w += d.w;
    if (write_back && in) *reinterpret_cast<float4*>(x + src + i) = a;
    // the same order of squares as the scalar kernel would not matter: each kernel is
    // used for a given width whatever the batch, so a row always sums the same way
    const float ss = in ? a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w : 0.f;
    const float total = block_sum(ss, scratch);
    const float scale = 1.0f / sqrtf(total / (float)width + eps);
    if (in) {
        store_f32<TOut>(out, dst + i, a.x * scale * w.x);
        store_f32<TOut>(out, dst + i + 1, a.y * scale * w.y);
        store_f32<TOut>(out, dst + i + 2, a.z * scale * w.z);
        store_f32<TOut>(out, dst + i + 3, a.w * scale * w.w);
    }
}

extern "C" int imparo_rms_norm(float* x, const float* delta, int n_delta, int n_x_rows, const int32_t* rows,
                               const float* weight, void* out, int out_dtype, int n_rows, int width, float eps,
                               int write_back, imparo_stream stream) {
    if (!x || !weight || !out || n_rows < 0 || width <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_delta < 0 || n_delta > 64 || (n_delta > 0 && !delta) || n_x_rows < 0) return IMPARO_BAD_ARGUMENT;
    if (!delta) n_delta = 0;
    const size_t delta_stride = (size_t)n_x_rows * width;
    if (write_back && rows) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = !(((uintptr_t)x | (uintptr_t)delta | (uintptr_t)weight) & 15);
    if (width % 4 == 0 && width >= 512 && width <= 4096 && aligned) {
        const int threads = ((width / 4) + 63) / 64 * 64;
        if (out_dtype == IMPARO_F32)
            k_rms_norm_v4<float><<<n_rows, threads, 0, s>>>(x, delta, n_delta, delta_stride, rows, weight, (float*)out, width, eps,
                                                            write_back);
        else if (out_dtype == IMPARO_BF16)
            k_rms_norm_v4<bf16_t><<<n_rows, threads, 0, s>>>(x, delta, n_delta, delta_stride, rows, weight, (bf16_t*)out, width,
                                                             eps, write_back);
        else
            return IMPARO_BAD_ARGUMENT;
        return launch_status();
    }
    const int threads = width <= 256 ? 64 : 256;
    if (out_dtype == IMPARO_F32)
        k_rms_norm<float, 8><<<n_rows, threads, 0, s>>>(x, delta, n_delta, delta_stride, rows, weight, (float*)out, width, eps,
                                                        write_back);
    else if (out_dtype == IMPARO_BF16)
        k_rms_norm<bf16_t, 8><<<n_rows, threads, 0, s>>>(x, delta, n_delta, delta_stride, rows, weight, (bf16_t*)out, width, eps,
                                                         write_back);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// ---------------------------------------------------------------- fill
__global__ void k_fill_f32(float* __restrict__ p, float value, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

extern "C" int imparo_fill_f32(float* p, float value, int64_t n, imparo_stream stream) {
    if (!p || n < 0) return IMPARO_BAD_ARGUMENT;
    if (n == 0) return IMPARO_OK;
    k_fill_f32<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(p, value, n);
    return launch_status();
}

// Every fixed-state site's row of one slot in one launch: site i's row is per_slot[i] floats at
// base[i] + slot * per_slot[i] and is filled with value[i]. grid (sites, blocks along the row).
__global__ void k_fill_sites(const uint64_t* __restrict__ base, const int64_t* __restrict__ per_slot,
                             const float* __restrict__ value, int slot) {
    const int site = blockIdx.x;
    const int64_t n = per_slot[site];
    float* p = reinterpret_cast<float*>(base[site]) + (int64_t)slot * n;
    const float v = value[site];
    for (int64_t i = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.y * blockDim.x)
        p[i] = v;
}

extern "C" int imparo_fill_sites(const uint64_t* base, const int64_t* per_slot, const float* value, int n_sites,
                                 int slot, imparo_stream stream) {
    if (n_sites < 0 || slot < 0 || (n_sites > 0 && (!base || !per_slot || !value))) return IMPARO_BAD_ARGUMENT;
    if (n_sites == 0) return IMPARO_OK;
    if (n_sites > 65535) return IMPARO_BAD_ARGUMENT;
    k_fill_sites<<<dim3((unsigned)n_sites, 16), 256, 0, (hipStream_t)stream>>>(base, per_slot, value, slot);
    return launch_status();
}

// ---------------------------------------------------------------- short conv
// One thread per (token, channel). seq index e = (t - seg_start) + k runs over
// state (e < taps-1) then this segment's B*x values; tap 0 multiplies the
// oldest value. The state is only read here; the state kernel runs after.
template <typename TOut>
__global__ void k_short_conv(const float* __restrict__ bcx, const float* __restrict__ weight,
                             const float* __restrict__ bias, const float* __restrict__ state,
                             const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ seg_start,
                             const int32_t* __restrict__ slot, TOut* __restrict__ out,
                             int n_tokens, int width, int taps) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    const int t = blockIdx.y;
    if (ch >= width) return;
    const int r = row_of_token[t];
    const int local = t - seg_start[r];
    const int history = taps - 1;
    const float* st = state + (size_t)slot[r] * history * width;
    float acc = 0.f;
    for (int k = 0; k < taps; ++k) {
        const int e = local + k;            // index into state ++ values
        float v;
        if (e < history) {
            v = st[(size_t)e * width + ch];
        } else {
            const size_t row = (size_t)(t - (history - k)) * 3 * width;
            v = bcx[row + ch] * bcx[row + 2 * width + ch];
        }
        acc = fmaf(weight[(size_t)ch * taps + k], v, acc);
    }
    if (bias) acc += bias[ch];
    const float c = bcx[(size_t)t * 3 * width + width + ch];
    store_f32<TOut>(out, (size_t)t * width + ch, c * acc);
}

__device__ __forceinline__ void store_four(float* dst, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store_four(bf16_t* dst, float a, float b, float c, float d) {
    *reinterpret_cast<uint2*>(dst) = make_uint2(f32x2_to_bf16x2(a, b), f32x2_to_bf16x2(c, d));
}

// The same, four channels to a thread with 16-byte loads (width a multiple of 4, rows 16-byte
// aligned): a prompt's portion is bound by how many bytes a memory instruction moves. Each
// channel's taps are summed exactly as above.
template <typename TOut>
__global__ void k_short_conv_v4(const float* __restrict__ bcx, const float* __restrict__ weight,
                                const float* __restrict__ bias, const float* __restrict__ state,
                                const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ seg_start,
                                const int32_t* __restrict__ slot, TOut* __restrict__ out,
                                int n_tokens, int width, int taps) {
    const int ch = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const int t = blockIdx.y;
    if (ch >= width) return;
    const int r = row_of_token[t];
    const int local = t - seg_start[r];
    const int history = taps - 1;
    const float* st = state + (size_t)slot[r] * history * width;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < taps; ++k) {
        const int e = local + k;            // index into state ++ values
        float4 v;
        if (e < history) {
            v = *reinterpret_cast<const float4*>(st + (size_t)e * width + ch);
        } else {
            const size_t row = (size_t)(t - (history - k)) * 3 * width;
            const float4 b = *reinterpret_cast<const float4*>(bcx + row + ch);
            const float4 x = *reinterpret_cast<const float4*>(bcx + row + 2 * width + ch);
            v = make_float4(b.x * x.x, b.y * x.y, b.z * x.z, b.w * x.w);
        }
        acc[0] = fmaf(weight[(size_t)ch * taps + k], v.x, acc[0]);
        acc[1] = fmaf(weight[(size_t)(ch + 1) * taps + k], v.y, acc[1]);
        acc[2] = fmaf(weight[(size_t)(ch + 2) * taps + k], v.z, acc[2]);
        acc[3] = fmaf(weight[(size_t)(ch + 3) * taps + k], v.w, acc[3]);
    }
    if (bias) {
        const float4 bv = *reinterpret_cast<const float4*>(bias + ch);
        acc[0] += bv.x;
        acc[1] += bv.y;
        acc[2] += bv.z;
        acc[3] += bv.w;
    }
    const float4 c = *reinterpret_cast<const float4*>(bcx + (size_t)t * 3 * width + width + ch);
    store_four(out + (size_t)t * width + ch, c.x * acc[0], c.y * acc[1], c.z * acc[2], c.w * acc[3]);
}

// For prompt portions and a short history (HIST = taps - 1 <= 3): four channels and TT
// consecutive tokens to a thread. The thread reads B*x of its tokens and of the HIST tokens
// before them once (the plain kernel reads each value taps times), every load issued before
// the first use and none under a branch; only a token among the first HIST of its segment
// takes its oldest values from the request's state instead. Each channel's taps are summed
// exactly as above.
template <typename TOut, int HIST, int TT>
__global__ void k_short_conv_tile(const float* __restrict__ bcx, const float* __restrict__ weight,
                                  const float* __restrict__ bias, const float* __restrict__ state,
                                  const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ seg_start,
                                  const int32_t* __restrict__ slot, TOut* __restrict__ out, int n_tokens, int width) {
    const int ch = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    const int t0 = blockIdx.y * TT;
    if (ch >= width) return;
    typedef float f4 __attribute__((ext_vector_type(4)));
    f4 u[TT + HIST], c[TT];
#pragma unroll
    for (int j = 0; j < TT + HIST; ++j) {
        const int tj = min(max(t0 - HIST + j, 0), n_tokens - 1);
        const float* row = bcx + (size_t)tj * 3 * width + ch;
        u[j] = *reinterpret_cast<const f4*>(row) * *reinterpret_cast<const f4*>(row + 2 * width);
    }
#pragma unroll
    for (int i = 0; i < TT; ++i)
        c[i] = *reinterpret_cast<const f4*>(bcx + (size_t)min(t0 + i, n_tokens - 1) * 3 * width + width + ch);
    float w[4][HIST + 1];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int k = 0; k <= HIST; ++k) w[q][k] = weight[(size_t)(ch + q) * (HIST + 1) + k];
    f4 bv = {0.f, 0.f, 0.f, 0.f};
    if (bias) bv = *reinterpret_cast<const f4*>(bias + ch);
#pragma unroll
    for (int i = 0; i < TT; ++i) {
        const int t = t0 + i;
        if (t >= n_tokens) break;
        const int r = row_of_token[t];
        const int local = t - seg_start[r];
        f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k <= HIST; ++k) {
            f4 v = u[i + k];                                   // token t - (HIST - k)
            if (local + k < HIST)                               // before the segment's first token: the state
                v = *reinterpret_cast<const f4*>(state + ((size_t)slot[r] * HIST + local + k) * width + ch);
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[q] = fmaf(w[q][k], v[q], acc[q]);
        }
        acc += bv;
        const f4 y = c[i] * acc;
        store_four(out + (size_t)t * width + ch, y.x, y.y, y.z, y.w);
    }
}

template <typename TOut, int HIST>
static void launch_conv_tile(const float* bcx, const float* weight, const float* bias, const float* state,
                             const int32_t* row_of_token, const int32_t* seg_start, const int32_t* slot, TOut* out,
                             int n_tokens, int width, hipStream_t s) {
    constexpr int TT = 4;
    const int threads = width >= 1024 ? 256 : 64;
    dim3 grid((width / 4 + threads - 1) / threads, (n_tokens + TT - 1) / TT);
    k_short_conv_tile<TOut, HIST, TT><<<grid, threads, 0, s>>>(bcx, weight, bias, state, row_of_token, seg_start, slot,
                                                               out, n_tokens, width);
}

extern "C" int imparo_short_conv(const float* bcx, const float* weight, const float* bias, const float* state,
                                 const int32_t* row_of_token, const int32_t* seg_start, const int32_t* slot,
                                 void* out, int out_dtype, int n_tokens, int width, int taps, int n_slots,
                                 int n_rows, imparo_stream stream) {
    if (!bcx || !weight || !state || !row_of_token || !seg_start || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || width <= 0 || taps < 2 || taps > 64 || n_slots <= 0 || n_rows < 0) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    if (n_tokens > 65535) return IMPARO_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    if (width % 4 == 0 && n_tokens >= 32 && ((uintptr_t)bcx % 16) == 0 && ((uintptr_t)state % 16) == 0 &&
        ((uintptr_t)out % 16) == 0 && (!bias || ((uintptr_t)bias % 16) == 0) &&
        (out_dtype == IMPARO_F32 || out_dtype == IMPARO_BF16)) {
        if (taps <= 4 && (n_tokens + 3) / 4 <= 65535) {
#define CONV_TILE(T)                                                                                                 \
    switch (taps - 1) {                                                                                              \
        case 1: launch_conv_tile<T, 1>(bcx, weight, bias, state, row_of_token, seg_start, slot, (T*)out, n_tokens, width, s); break; \
        case 2: launch_conv_tile<T, 2>(bcx, weight, bias, state, row_of_token, seg_start, slot, (T*)out, n_tokens, width, s); break; \
        default: launch_conv_tile<T, 3>(bcx, weight, bias, state, row_of_token, seg_start, slot, (T*)out, n_tokens, width, s);      \
    }
            if (out_dtype == IMPARO_F32) {
                CONV_TILE(float)
            } else {
                CONV_TILE(bf16_t)
            }
#undef CONV_TILE
            return launch_status();
        }
        const int threads4 = width >= 1024 ? 256 : 64;
        dim3 grid4((width / 4 + threads4 - 1) / threads4, n_tokens);
        if (out_dtype == IMPARO_F32)
            k_short_conv_v4<float><<<grid4, threads4, 0, s>>>(bcx, weight, bias, state, row_of_token, seg_start, slot,
                                                              (float*)out, n_tokens, width, taps);
        else
            k_short_conv_v4<bf16_t><<<grid4, threads4, 0, s>>>(bcx, weight, bias, state, row_of_token, seg_start,
                                                               slot, (bf16_t*)out, n_tokens, width, taps);
        return launch_status();
    }
    const int threads = width >= 256 ? 256 : 64;
    dim3 grid((width + threads - 1) / threads, n_tokens);
    if (out_dtype == IMPARO_F32)
        k_short_conv<float><<<grid, threads, 0, s>>>(bcx, weight, bias, state, row_of_token, seg_start, slot,
                                                      (float*)out, n_tokens, width, taps);
    else if (out_dtype == IMPARO_BF16)
        k_short_conv<bf16_t><<<grid, threads, 0, s>>>(bcx, weight, bias, state, row_of_token, seg_start, slot,
                                                       (bf16_t*)out, n_tokens, width, taps);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// Single-token rows: one thread per (row, channel) reads the history, writes
// the output and the shifted history. It owns its channel, so nothing races.
// HIST > 0: the history length is known at compile time and everything the
// thread needs is loaded before the first value is used (one trip to memory
// instead of one per tap; what a decode step hands this kernel is in no near
// cache). HIST == 0: any length, tap by tap.
template <typename TOut, int HIST>
__global__ void k_short_conv_decode(const float* __restrict__ bcx, const float* __restrict__ weight,
                                    const float* __restrict__ bias, float* __restrict__ state,
                                    const int32_t* __restrict__ slot, TOut* __restrict__ out, int width, int taps) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = blockIdx.y;
    if (ch >= width) return;
    const int history = HIST > 0 ? HIST : taps - 1;
    float* st = state + (size_t)slot[r] * history * width;
    const size_t row = (size_t)r * 3 * width;
    const float b_in = bcx[row + ch], c_in = bcx[row + width + ch], x_in = bcx[row + 2 * width + ch];
    const float bias_v = bias ? bias[ch] : 0.f;
    // the taps are summed oldest first, exactly as the general kernel sums them
    float acc = 0.f;
    if (HIST > 0) {
        float h[HIST > 0 ? HIST : 1], w[(HIST > 0 ? HIST : 1) + 1];
#pragma unroll
        for (int k = 0; k < HIST; ++k) h[k] = st[(size_t)k * width + ch];
#pragma unroll
        for (int k = 0; k <= HIST; ++k) w[k] = weight[(size_t)ch * (HIST + 1) + k];
        const float u = b_in * x_in;
#pragma unroll
        for (int k = 0; k < HIST; ++k) {
            acc = fmaf(w[k], h[k], acc);
            st[(size_t)k * width + ch] = k + 1 < HIST ? h[k + 1] : u;
        }
        acc = fmaf(w[HIST], u, acc);
    } else {
        const float u = b_in * x_in;
        float prev = st[ch];                                  // oldest
        for (int k = 0; k < history; ++k) {
            acc = fmaf(weight[(size_t)ch * taps + k], prev, acc);
            const float next = (k + 1 < history) ? st[(size_t)(k + 1) * width + ch] : u;
            st[(size_t)k * width + ch] = next;
            prev = next;
        }
        acc = fmaf(weight[(size_t)ch * taps + history], u, acc);
    }
    acc += bias_v;
    store_f32<TOut>(out, (size_t)r * width + ch, c_in * acc);
}

template <typename TOut>
static void launch_conv_decode(dim3 grid, int threads, hipStream_t s, const float* bcx, const float* weight,
                               const float* bias, float* state, const int32_t* slot, TOut* out, int width, int taps) {
    switch (taps - 1) {
        case 1: k_short_conv_decode<TOut, 1><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 2: k_short_conv_decode<TOut, 2><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 3: k_short_conv_decode<TOut, 3><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 4: k_short_conv_decode<TOut, 4><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 5: k_short_conv_decode<TOut, 5><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 6: k_short_conv_decode<TOut, 6><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        case 7: k_short_conv_decode<TOut, 7><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps); break;
        default: k_short_conv_decode<TOut, 0><<<grid, threads, 0, s>>>(bcx, weight, bias, state, slot, out, width, taps);
    }
}

extern "C" int imparo_short_conv_decode(const float* bcx, const float* weight, const float* bias, float* state,
                                        const int32_t* slot, void* out, int out_dtype, int n_rows, int width,
                                        int taps, int n_slots, imparo_stream stream) {
    if (!bcx || !weight || !state || !slot || !out) return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || width <= 0 || taps < 2 || taps > 64 || n_slots <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    if (n_rows > 65535) return IMPARO_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    const int threads = width >= 256 ? 256 : 64;
    dim3 grid((width + threads - 1) / threads, n_rows);
    if (out_dtype == IMPARO_F32)
        launch_conv_decode<float>(grid, threads, s, bcx, weight, bias, state, slot, (float*)out, width, taps);
    else if (out_dtype == IMPARO_BF16)
        launch_conv_decode<bf16_t>(grid, threads, s, bcx, weight, bias, state, slot, (bf16_t*)out, width, taps);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// One thread per (request, channel) owns that channel's whole shift, so the
// update is race-free in place: it reads every value it needs before it
// writes. Works for segments shorter than the history.
#define IMPARO_MAX_TAPS 64
__global__ void k_short_conv_state(const float* __restrict__ bcx, float* __restrict__ state,
                                   const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                   const int32_t* __restrict__ slot, int width, int taps) {
    const int ch = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = blockIdx.y;
    if (ch >= width) return;
    const int history = taps - 1;
    const int n = seg_len[r];
    const int t0 = seg_start[r];
    float* st = state + (size_t)slot[r] * history * width;
    float next[IMPARO_MAX_TAPS - 1];
    for (int s = 0; s < history; ++s) {
        const int e = n + s;                // index into state ++ values
        if (e < history) {
            next[s] = st[(size_t)e * width + ch];
        } else {
            const size_t row = (size_t)(t0 + e - history) * 3 * width;
            next[s] = bcx[row + ch] * bcx[row + 2 * width + ch];
        }
    }
    for (int s = 0; s < history; ++s) st[(size_t)s * width + ch] = next[s];
}

extern "C" int imparo_short_conv_state(const float* bcx, float* state, const int32_t* seg_start,
                                       const int32_t* seg_len, const int32_t* slot, int n_rows, int n_tokens,
                                       int width, int taps, int n_slots, imparo_stream stream) {
    if (!bcx || !state || !seg_start || !seg_len || !slot) return IMPARO_BAD_ARGUMENT;
    if (n_rows < 0 || width <= 0 || taps < 2 || taps > IMPARO_MAX_TAPS || n_slots <= 0) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    if (n_rows > 65535) return IMPARO_BAD_ARGUMENT;
    const int threads = width >= 256 ? 256 : 64;
    dim3 grid((width + threads - 1) / threads, n_rows);
    k_short_conv_state<<<grid, threads, 0, (hipStream_t)stream>>>(bcx, state, seg_start, seg_len, slot, width, taps);
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_elementwise() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_fill_f32)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
