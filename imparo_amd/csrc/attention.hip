// Causal grouped-query attention over the paged cache.
//
// k_attention_wave: one wave per (token, head). Keys are walked in chunks of 64
// aligned at absolute multiples of 64, one key per lane for the scores, one
// output dimension per lane for the weighted sum, online softmax in float32.
// The order of every sum depends only on the query's position, so the result
// does not depend on how a prompt was cut or what else is in the batch.
#include "common.h"
#include "api.h"

#define ATT_MAX_HEAD_DIM 512
#define ATT_WAVES 4

template <typename T> struct Vec16;
template <> struct Vec16<float> { static constexpr int N = 4; };
template <> struct Vec16<bf16_t> { static constexpr int N = 8; };

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const T* __restrict__ k, int head_dim);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ q, const float* __restrict__ k, int head_dim) {
    float s = 0.f;
    for (int i = 0; i < head_dim; i += 4) {
        const float4 kv = *reinterpret_cast<const float4*>(k + i);
        s += q[i] * kv.x;
        s += q[i + 1] * kv.y;
        s += q[i + 2] * kv.z;
        s += q[i + 3] * kv.w;
    }
    return s;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const float* __restrict__ q, const bf16_t* __restrict__ k, int head_dim) {
    float s = 0.f;
    for (int i = 0; i < head_dim; i += 8) {
        const uint4 kv = *reinterpret_cast<const uint4*>(k + i);
        const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s += q[i + 2 * j] * __uint_as_float(w[j] << 16);
            s += q[i + 2 * j + 1] * __uint_as_float(w[j] & 0xffff0000u);
        }
    }
    return s;
}

template <typename T>
__global__ void k_attention_wave(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                 T* __restrict__ out, const int32_t* __restrict__ positions,
                                 const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ block_table,
                                 int table_stride, int page_size, int n_tokens, int heads, int kv_heads, int head_dim,
                                 int n_pages, float scale, int window, int v_transposed) {
    __shared__ float q_rows[ATT_WAVES][ATT_MAX_HEAD_DIM];
    __shared__ float probs[ATT_WAVES][WAVE];
    __shared__ long long v_off[ATT_WAVES][WAVE];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const long long id = (long long)blockIdx.x * ATT_WAVES + wave;
    if (id >= (long long)n_tokens * heads) return;
    const int t = (int)(id / heads);
    const int h = (int)(id - (long long)t * heads);
    const int kvh = h / (heads / kv_heads);
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int32_t* table = block_table + (size_t)row_of_token[t] * table_stride;

    float* qr = q_rows[wave];
    const T* qsrc = q + ((size_t)t * heads + h) * head_dim;
    for (int i = lane; i < head_dim; i += WAVE) qr[i] = load_f32<T>(qsrc, i);
    wave_lds_sync();

    constexpr int DPL = ATT_MAX_HEAD_DIM / WAVE;
    float acc[DPL];
#pragma unroll
    for (int j = 0; j < DPL; ++j) acc[j] = 0.f;
    float m = -INFINITY, l = 0.f;

    for (int c = (lo / WAVE) * WAVE; c <= pos; c += WAVE) {
        const int p = c + lane;
        const bool valid = p >= lo && p <= pos;
        float s = -INFINITY;
        long long off = -1;
        if (valid) {
            const int page = table[p / page_size];
            if (page >= 0 && page < n_pages) {
                off = (((long long)page * kv_heads + kvh) * page_size + (p % page_size)) * head_dim;
                s = dot_row<T>(qr, k_cache + off, head_dim) * scale;
                if (v_transposed)
                    off = ((long long)page * kv_heads + kvh) * page_size * head_dim + (p % page_size);
            }
        }
        const float m_new = fmaxf(m, wave_max(s));
        const float pe = (off >= 0) ? expf(s - m_new) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + wave_sum(pe);
        m = m_new;
        probs[wave][lane] = pe;
        v_off[wave][lane] = off;
        wave_lds_sync();
        const int n_keys = min(WAVE, pos - c + 1);
#pragma unroll
        for (int j = 0; j < DPL; ++j) acc[j] *= corr;
        for (int kk = 0; kk < n_keys; ++kk) {
            const long long vo = v_off[wave][kk];
            if (vo < 0) continue;           // uniform over the wave
            const float pk = probs[wave][kk];
            const T* vrow = v_cache + vo;
#pragma unroll
            for (int j = 0; j < DPL; ++j) {
                const int d = lane + j * WAVE;
                if (d < head_dim) acc[j] += pk * load_f32<T>(vrow, v_transposed ? (size_t)d * page_size : (size_t)d);
            }
        }
        wave_lds_sync();
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* dst = out + ((size_t)t * heads + h) * head_dim;
#pragma unroll
    for (int j = 0; j < DPL; ++j) {
        const int d = lane + j * WAVE;
        if (d < head_dim) store_f32<T>(dst, d, acc[j] * inv);
    }
}

static int check_attention_args(const void* q, const void* k_cache, const void* v_cache, void* out,
                                const int32_t* positions, const int32_t* row_of_token, const int32_t* block_table,
                                int table_stride, int page_size, int n_tokens, int heads, int kv_heads, int head_dim,
                                int n_pages, int window) {
    if (!q || !k_cache || !v_cache || !out || !positions || !row_of_token || !block_table) return IMPARO_BAD_ARGUMENT;
    if (n_tokens < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0) return IMPARO_BAD_ARGUMENT;
    if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > ATT_MAX_HEAD_DIM) return IMPARO_BAD_ARGUMENT;
    if (page_size <= 0 || table_stride <= 0 || n_pages <= 0 || window < 0) return IMPARO_BAD_ARGUMENT;
    return IMPARO_OK;
}

extern "C" int imparo_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                                const int32_t* positions, const int32_t* row_of_token,
                                const int32_t* block_table, int table_stride, int page_size,
                                int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                                float scale, int window, int v_transposed, imparo_stream stream) {
    const int bad = check_attention_args(q, k_cache, v_cache, out, positions, row_of_token, block_table, table_stride,
                                         page_size, n_tokens, heads, kv_heads, head_dim, n_pages, window);
    if (bad) return bad;
    if (n_tokens == 0) return IMPARO_OK;
    const long long total = (long long)n_tokens * heads;
    const unsigned blocks = (unsigned)((total + ATT_WAVES - 1) / ATT_WAVES);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == IMPARO_F32)
        k_attention_wave<float><<<blocks, ATT_WAVES * WAVE, 0, s>>>(
            (const float*)q, (const float*)k_cache, (const float*)v_cache, (float*)out, positions, row_of_token,
            block_table, table_stride, page_size, n_tokens, heads, kv_heads, head_dim, n_pages, scale, window, v_transposed);
    else if (dtype == IMPARO_BF16)
        k_attention_wave<bf16_t><<<blocks, ATT_WAVES * WAVE, 0, s>>>(
            (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, positions, row_of_token,
            block_table, table_stride, page_size, n_tokens, heads, kv_heads, head_dim, n_pages, scale, window,
            v_transposed);
    else
        return IMPARO_BAD_ARGUMENT;
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_attention() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_attention_wave<float>)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
