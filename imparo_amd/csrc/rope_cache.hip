// Per-head RMS norm + NeoX rotation of q and k, and the write of k and v into
// the paged cache, in one launch over every (token, head) of the fused qkv row.
#include "common.h"
#include "api.h"

#define ROPE_MAX_HEAD_DIM 512
#define ROPE_WAVES 4

// The arithmetic both kernels below share, written with explicit fused operations so that
// the two compile to the same roundings: which of them a token meets depends on how many
// tokens came with it, and its results must not.
__device__ __forceinline__ void rotation_of(int pos, float inv_freq, float& sn, float& cs) {
    const float theta = (float)((double)pos * (double)inv_freq);
    sincosf(theta, &sn, &cs);
}
__device__ __forceinline__ float head_norm_scale(float sum_squares, int head_dim, float eps) {
    return 1.0f / sqrtf(sum_squares / (float)head_dim + eps);
}
// lane-owned pair i of a row staged in LDS: elements (i, i + n_freq), or with `interleaved`
// (2i, 2i + 1); reads both, then writes both
__device__ __forceinline__ void rotate_pair(float* row, int i, int n_freq, int interleaved, float sn, float cs) {
    const int a = interleaved ? 2 * i : i, b = interleaved ? 2 * i + 1 : i + n_freq;
    const float x0 = row[a], x1 = row[b];
    row[a] = fmaf(x0, cs, -(x1 * sn));
    row[b] = fmaf(x0, sn, x1 * cs);
}

// One wave per (token, unit), unit in [0, heads + 2*kv_heads): q heads, then k
// heads, then v heads. The row is staged in LDS as float32; the sum of squares
// is a wave reduction; angles are pos * inv_freq[i] with the product taken in
// float64 and rounded to float32, sin/cos in float32.
template <typename T>
__global__ void k_qk_norm_rope_store(const float* __restrict__ qkv, const float* __restrict__ q_weight,
                                     const float* __restrict__ k_weight, float eps,
                                     const float* __restrict__ inv_freq, int n_freq, int interleaved,
                                     const int32_t* __restrict__ positions, const int32_t* __restrict__ row_of_token,
                                     const int32_t* __restrict__ block_table, int table_stride, int page_size,
                                     T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     int write_kv, int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                                     int v_transposed) {
    __shared__ float rows[ROPE_WAVES][ROPE_MAX_HEAD_DIM];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int units = heads + 2 * kv_heads;
    const long long id = (long long)blockIdx.x * ROPE_WAVES + wave;
    if (id >= (long long)n_tokens * units) return;
    const int t = (int)(id / units);
    const int u = (int)(id - (long long)t * units);
    const float* src = qkv + (size_t)t * units * head_dim + (size_t)u * head_dim;
    float* row = rows[wave];
    const bool is_q = u < heads;
    const bool is_v = u >= heads + kv_heads;
    const float* weight = is_q ? q_weight : k_weight;

    // Everything the wave needs is asked for before the first value is used: what a decode
    // step hands this kernel is in no near cache, and each load that waits for the one
    // before costs a trip to memory.
    constexpr int PER_LANE = ROPE_MAX_HEAD_DIM / WAVE;
    const int pos = positions[t];
    int page = -1;
    if (!is_q && write_kv) page = block_table[(size_t)row_of_token[t] * table_stride + pos / page_size];
    float a[PER_LANE], w[PER_LANE], freq[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int i = lane + j * WAVE;
        a[j] = i < head_dim ? src[i] : 0.f;
        w[j] = (i < head_dim && weight && !is_v) ? weight[i] : 1.f;
        freq[j] = (i < n_freq && !is_v) ? inv_freq[i] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) ss = fmaf(a[j], a[j], ss);     // in the order i = lane, lane + 64, ...
    if (!is_v) {
        float scale = 1.f;
        if (weight) {
            ss = wave_sum(ss);
            scale = head_norm_scale(ss, head_dim, eps);
        }
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int i = lane + j * WAVE;
            if (i < head_dim) row[i] = weight ? a[j] * scale * w[j] : a[j];
        }
        wave_lds_sync();   // a pair's second element may have been written by another lane
        if (n_freq > 0) {
            // each lane owns pair (i, i + n_freq): reads both, then writes both
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j) {
                const int i = lane + j * WAVE;
                if (i < n_freq) {
                    float sn, cs;
                    rotation_of(pos, freq[j], sn, cs);
                    rotate_pair(row, i, n_freq, interleaved, sn, cs);
                }
            }
        }
    } else {
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int i = lane + j * WAVE;
            if (i < head_dim) row[i] = a[j];
        }
    }
    wave_lds_sync();

    if (is_q) {
        T* dst = q_out + ((size_t)t * heads + u) * head_dim;
        for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, i, row[i]);
        return;
    }
    if (!write_kv) return;
    const int kvh = is_v ? u - heads - kv_heads : u - heads;
    if (page < 0 || page >= n_pages) return;   // never write outside the pool
    if (is_v && v_transposed) {
        // [page, kv head, dim, slot]: the keys of one dimension lie side by side
        T* dst = v_cache + ((size_t)page * kv_heads + kvh) * page_size * head_dim + (pos % page_size);
        for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, (size_t)i * page_size, row[i]);
        return;
    }
    T* cache = is_v ? v_cache : k_cache;
    T* dst = cache + (((size_t)page * kv_heads + kvh) * page_size + (pos % page_size)) * head_dim;
    for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, i, row[i]);
}

// The same for many tokens (a prompt's portion): one block per token. The rotation's sines and
// cosines depend on the position only, so the block works them out once (they are most of the
// arithmetic) and its four waves share them over all heads; a wave takes UB units in a row and
// has all their loads in flight together. NPL is the elements of a unit's row per lane.
template <typename T, int NPL, int UB>
__global__ __launch_bounds__(ROPE_WAVES * WAVE) void k_qk_norm_rope_store_token(
    const float* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ inv_freq, int n_freq, int interleaved, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ block_table, int table_stride,
    int page_size, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int write_kv,
    int n_tokens, int heads, int kv_heads, int head_dim, int n_pages, int v_transposed) {
    __shared__ float sn_tab[ROPE_MAX_HEAD_DIM / 2], cs_tab[ROPE_MAX_HEAD_DIM / 2];
    __shared__ float rows[ROPE_WAVES][NPL * WAVE];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int units = heads + 2 * kv_heads;
    const int t = blockIdx.x;
    const int pos = positions[t];
    int page = -1;
    if (write_kv) page = block_table[(size_t)row_of_token[t] * table_stride + pos / page_size];
    for (int i = threadIdx.x; i < n_freq; i += ROPE_WAVES * WAVE) rotation_of(pos, inv_freq[i], sn_tab[i], cs_tab[i]);
    float wq[NPL], wk[NPL];
#pragma unroll
    for (int j = 0; j < NPL; ++j) {
        const int i = lane + j * WAVE;
        wq[j] = (q_weight && i < head_dim) ? q_weight[i] : 1.f;
        wk[j] = (k_weight && i < head_dim) ? k_weight[i] : 1.f;
    }
    __syncthreads();
    const float* src = qkv + (size_t)t * units * head_dim;
    float* row = rows[wave];
    for (int u0 = wave * UB; u0 < units; u0 += ROPE_WAVES * UB) {
        float a[UB][NPL];
#pragma unroll
        for (int b = 0; b < UB; ++b)
#pragma unroll
            for (int j = 0; j < NPL; ++j) {
                const int i = lane + j * WAVE;
                a[b][j] = i < head_dim ? src[(size_t)min(u0 + b, units - 1) * head_dim + i] : 0.f;
            }
#pragma unroll
        for (int b = 0; b < UB; ++b) {
            const int u = u0 + b;
            if (u >= units) break;
            const bool is_q = u < heads;
            const bool is_v = u >= heads + kv_heads;
            if (!is_v) {
                float scale = 1.f;
                if (q_weight) {
                    float ss = 0.f;
#pragma unroll
                    for (int j = 0; j < NPL; ++j) ss = fmaf(a[b][j], a[b][j], ss);
                    ss = wave_sum(ss);
                    scale = head_norm_scale(ss, head_dim, eps);
                }
#pragma unroll
                for (int j = 0; j < NPL; ++j) {
                    const int i = lane + j * WAVE;
                    if (i < head_dim) row[i] = q_weight ? a[b][j] * scale * (is_q ? wq[j] : wk[j]) : a[b][j];
                }
                wave_lds_sync();
#pragma unroll
                for (int j = 0; j < NPL; ++j) {
                    const int i = lane + j * WAVE;
                    if (i < n_freq) rotate_pair(row, i, n_freq, interleaved, sn_tab[i], cs_tab[i]);
                }
            } else {
#pragma unroll
                for (int j = 0; j < NPL; ++j) {
                    const int i = lane + j * WAVE;
                    if (i < head_dim) row[i] = a[b][j];
                }
            }
            wave_lds_sync();
            if (is_q) {
                T* dst = q_out + ((size_t)t * heads + u) * head_dim;
                for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, i, row[i]);
            } else if (write_kv && page >= 0 && page < n_pages) {      // never write outside the pool
                const int kvh = is_v ? u - heads - kv_heads : u - heads;
                if (is_v && v_transposed) {
                    T* dst = v_cache + ((size_t)page * kv_heads + kvh) * page_size * head_dim + (pos % page_size);
                    for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, (size_t)i * page_size, row[i]);
                } else {
                    T* cache = is_v ? v_cache : k_cache;
                    T* dst = cache + (((size_t)page * kv_heads + kvh) * page_size + (pos % page_size)) * head_dim;
                    for (int i = lane; i < head_dim; i += WAVE) store_f32<T>(dst, i, row[i]);
                }
            }
            wave_lds_sync();           // the row is read out before the next unit overwrites it
        }
    }
}

template <typename T>
static void launch_rope_token(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                              const float* inv_freq, int n_freq, int interleaved, const int32_t* positions,
                              const int32_t* row_of_token, const int32_t* block_table, int table_stride,
                              int page_size, T* q_out, T* k_cache, T* v_cache, int write_kv, int n_tokens, int heads,
                              int kv_heads, int head_dim, int n_pages, int v_transposed, hipStream_t s) {
#define ROPE_TOKEN(NPL, UB)                                                                                          \
    k_qk_norm_rope_store_token<T, NPL, UB><<<n_tokens, ROPE_WAVES * WAVE, 0, s>>>(                                   \
        qkv, q_weight, k_weight, eps, inv_freq, n_freq, interleaved, positions, row_of_token, block_table, table_stride,         \
        page_size, q_out, k_cache, v_cache, write_kv, n_tokens, heads, kv_heads, head_dim, n_pages, v_transposed)
    if (head_dim <= 64)
        ROPE_TOKEN(1, 4);
    else if (head_dim <= 128)
        ROPE_TOKEN(2, 4);
    else if (head_dim <= 256)
        ROPE_TOKEN(4, 2);
    else
        ROPE_TOKEN(8, 1);
#undef ROPE_TOKEN
}

// From this many tokens on a launch takes the kernel with a block per token: its table of sines
// and cosines costs each block a fixed 10 us or so, which the kernel with a wave per head passes
// at about 400 tokens (40 heads of 64: 8 us at 256 tokens, 13 at 512, 43 at 2,048 against 22)
#ifndef ROPE_TOKEN_KERNEL_FROM
#define ROPE_TOKEN_KERNEL_FROM 400
#endif

extern "C" int imparo_qk_norm_rope_store(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                                         const float* inv_freq, int n_freq, int interleaved,
                                         const int32_t* positions, const int32_t* row_of_token,
                                         const int32_t* block_table, int table_stride, int page_size,
                                         void* q_out, void* k_cache, void* v_cache, int dtype, int write_kv,
                                         int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                                         int v_transposed, imparo_stream stream) {
    if (!qkv || !positions || !q_out) return IMPARO_BAD_ARGUMENT;
    if (write_kv && (!row_of_token || !block_table || !k_cache || !v_cache)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim > ROPE_MAX_HEAD_DIM)
        return IMPARO_BAD_ARGUMENT;
    if (n_freq < 0 || 2 * n_freq > head_dim || (n_freq > 0 && !inv_freq)) return IMPARO_BAD_ARGUMENT;
    if (page_size <= 0 || table_stride < 0 || n_pages < 0) return IMPARO_BAD_ARGUMENT;
    if ((q_weight == nullptr) != (k_weight == nullptr)) return IMPARO_BAD_ARGUMENT;
    if (n_tokens == 0) return IMPARO_OK;
    const long long total = (long long)n_tokens * (heads + 2 * kv_heads);
    const unsigned blocks = (unsigned)((total + ROPE_WAVES - 1) / ROPE_WAVES);
    hipStream_t s = (hipStream_t)stream;
    if (n_tokens >= ROPE_TOKEN_KERNEL_FROM && (dtype == IMPARO_F32 || dtype == IMPARO_BF16)) {
        if (dtype == IMPARO_F32)
            launch_rope_token<float>(qkv, q_weight, k_weight, eps, inv_freq, n_freq, interleaved, positions, row_of_token,
                                     block_table, table_stride, page_size, (float*)q_out, (float*)k_cache,
                                     (float*)v_cache, write_kv, n_tokens, heads, kv_heads, head_dim, n_pages,
                                     v_transposed, s);
        else
            launch_rope_token<bf16_t>(qkv, q_weight, k_weight, eps, inv_freq, n_freq, interleaved, positions, row_of_token,
                                      block_table, table_stride, page_size, (bf16_t*)q_out, (bf16_t*)k_cache,
                                      (bf16_t*)v_cache, write_kv, n_tokens, heads, kv_heads, head_dim, n_pages,
                                      v_transposed, s);
        return launch_status();
    }
    if (dtype == IMPARO_F32)
        k_qk_norm_rope_store<float><<<blocks, ROPE_WAVES * WAVE, 0, s>>>(
            qkv, q_weight, k_weight, eps, inv_freq, n_freq, interleaved, positions, row_of_token, block_table, table_stride,
            page_size, (float*)q_out, (float*)k_cache, (float*)v_cache, write_kv, n_tokens, heads, kv_heads,
            head_dim, n_pages, v_transposed);
    else if (dtype == IMPARO_BF16)
        k_qk_norm_rope_store<bf16_t><<<blocks, ROPE_WAVES * WAVE, 0, s>>>(
            qkv, q_weight, k_weight, eps, inv_freq, n_freq, interleaved, positions, row_of_token, block_table, table_stride,
            page_size, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, write_kv, n_tokens, heads, kv_heads,
            head_dim, n_pages, v_transposed);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}
