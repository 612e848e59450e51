// Per-head RMS norm + NeoX rotation of q and k, and the write of k and v into
// the paged cache, in one launch over every (token, head) of the fused qkv row.
#include "common.h"
#include "api.h"

#define ROPE_MAX_HEAD_DIM 512
#define ROPE_WAVES 4

// The arithmetic both kernels below share, written with explicit fused operations so that
// the two compile to the same roundings: which of them a token meets depends on how many
// tokens came with it, and its results must not.
// The sum over a wave's lanes, nearest lanes first (1, 2, 4, ... apart): the kernel below that gives a lane
// four neighbouring elements adds them in this same order, inside the lane first.
__device__ __forceinline__ float wave_sum_near_first(float v) {
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) v += __shfl_xor(v, off, WAVE);
    return v;
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
            ss = wave_sum_near_first(ss);
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
                    ss = wave_sum_near_first(ss);
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

// The same again for heads of 64 that are rotated whole (every LFM2 checkpoint): a lane takes four
// neighbouring elements of a head, sixteen lanes a head, so a wave has four heads at a time and
// nothing goes through LDS but the block's sines and cosines. The partner of an element is sixteen
// lanes' worth away (i, i + 32: the lane 8 further in its group) or beside it in the lane (2i, 2i + 1).
// Sums and products are taken in the order and with the roundings of the kernels above.
// (e0^2 + e1^2) + (e2^2 + e3^2), every square and every sum rounded on its own: what four lanes with one
// element each arrive at after two steps of the sum above. (The compiler would otherwise fuse a square
// into the sum that follows it; the *_rn functions of the HIP headers are plain operators and do not stop it.)
__device__ __forceinline__ float squares_of_four(const float (&e)[4]) {
#pragma clang fp contract(off)
    const float s0 = e[0] * e[0], s1 = e[1] * e[1], s2 = e[2] * e[2], s3 = e[3] * e[3];
    const float a = s0 + s1, b = s2 + s3;
    return a + b;
}
template <typename T> __device__ __forceinline__ void store4(T* dst, const float (&v)[4]);
template <> __device__ __forceinline__ void store4<float>(float* dst, const float (&v)[4]) {
    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* dst, const float (&v)[4]) {
    union { bf16_t h[4]; uint2 u; } o;
#pragma unroll
    for (int j = 0; j < 4; ++j) o.h[j] = f32_to_bf16(v[j]);
    *reinterpret_cast<uint2*>(dst) = o.u;
}

template <typename T, int ROUNDS>
__global__ __launch_bounds__(ROPE_WAVES * WAVE) void k_qk_norm_rope_store_token64(
    const float* __restrict__ qkv, const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps,
    const float* __restrict__ inv_freq, int interleaved, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ row_of_token, const int32_t* __restrict__ block_table, int table_stride,
    int page_size, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int write_kv,
    int heads, int kv_heads, int n_pages, int v_transposed) {
    constexpr int D = 64, HALF = 32;
    __shared__ float sn_tab[HALF], cs_tab[HALF];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = threadIdx.x / WAVE;
    const int l16 = lane & 15, sub = lane >> 4;
    const int units = heads + 2 * kv_heads;
    const int t = blockIdx.x;
    const int pos = positions[t];
    int page = -1;
    if (write_kv) page = block_table[(size_t)row_of_token[t] * table_stride + pos / page_size];
    if (threadIdx.x < HALF) rotation_of(pos, inv_freq[threadIdx.x], sn_tab[threadIdx.x], cs_tab[threadIdx.x]);
    float wq[4], wk[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        wq[j] = q_weight ? q_weight[4 * l16 + j] : 1.f;
        wk[j] = k_weight ? k_weight[4 * l16 + j] : 1.f;
    }
    const float* src = qkv + (size_t)t * units * D + 4 * l16;
    // all of the wave's rows are asked for before the first is used
    float4 rows[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int u = (r * ROPE_WAVES + wave) * 4 + sub;
        rows[r] = *reinterpret_cast<const float4*>(src + (size_t)min(u, units - 1) * D);
    }
    __syncthreads();
    // element j of this lane: the pair it belongs to, and whether it is the pair's second element
    float sn[4], cs[4];
    bool second[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int pair = interleaved ? 2 * l16 + (j >> 1) : 4 * (l16 & 7) + j;
        sn[j] = sn_tab[pair];
        cs[j] = cs_tab[pair];
        second[j] = interleaved ? (j & 1) : (l16 >= 8);
    }
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        const int u = (r * ROPE_WAVES + wave) * 4 + sub;
        const bool is_q = u < heads;
        const bool is_v = u >= heads + kv_heads;
        const float e[4] = {rows[r].x, rows[r].y, rows[r].z, rows[r].w};
        // (every lane takes part in the exchanges, also those of a value head or past the last unit)
        float ss = squares_of_four(e);
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) ss += __shfl_xor(ss, off, WAVE);
        const float scale = head_norm_scale(ss, D, eps);
        float n[4], partner[4], o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) n[j] = q_weight ? e[j] * scale * (is_q ? wq[j] : wk[j]) : e[j];
#pragma unroll
        for (int j = 0; j < 4; ++j) partner[j] = interleaved ? n[j ^ 1] : __shfl_xor(n[j], 8, WAVE);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float x0 = second[j] ? partner[j] : n[j], x1 = second[j] ? n[j] : partner[j];
            const float turned = second[j] ? fmaf(x0, sn[j], x1 * cs[j]) : fmaf(x0, cs[j], -(x1 * sn[j]));
            o[j] = is_v ? e[j] : turned;
        }
        if (u >= units) continue;
        if (is_q) {
            store4<T>(q_out + ((size_t)t * heads + u) * D + 4 * l16, o);
        } else if (write_kv && page >= 0 && page < n_pages) {        // never write outside the pool
            const int kvh = is_v ? u - heads - kv_heads : u - heads;
            if (is_v && v_transposed) {
                T* dst = v_cache + (((size_t)page * kv_heads + kvh) * D + 4 * l16) * page_size + (pos % page_size);
#pragma unroll
                for (int j = 0; j < 4; ++j) store_f32<T>(dst, (size_t)j * page_size, o[j]);
            } else {
                T* cache = is_v ? v_cache : k_cache;
                store4<T>(cache + (((size_t)page * kv_heads + kvh) * page_size + (pos % page_size)) * D + 4 * l16, o);
            }
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
    const int units = heads + 2 * kv_heads;
    // heads of 64 rotated whole, vectors aligned, up to 96 units a token: four elements a lane
    const bool vectors = ((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)v_cache |
                          (uintptr_t)q_weight | (uintptr_t)k_weight) % 16 == 0;
    if (head_dim == 64 && n_freq == 32 && vectors && units <= 96) {
#define ROPE_TOKEN64(ROUNDS)                                                                                        \
    k_qk_norm_rope_store_token64<T, ROUNDS><<<n_tokens, ROPE_WAVES * WAVE, 0, s>>>(                                  \
        qkv, q_weight, k_weight, eps, inv_freq, interleaved, positions, row_of_token, block_table, table_stride,     \
        page_size, q_out, k_cache, v_cache, write_kv, heads, kv_heads, n_pages, v_transposed)
        const int rounds = (units + 4 * ROPE_WAVES - 1) / (4 * ROPE_WAVES);
        if (rounds <= 1) ROPE_TOKEN64(1);
        else if (rounds == 2) ROPE_TOKEN64(2);
        else if (rounds == 3) ROPE_TOKEN64(3);
        else if (rounds == 4) ROPE_TOKEN64(4);
        else ROPE_TOKEN64(6);
#undef ROPE_TOKEN64
        return;
    }
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

// From this many tokens on a launch takes the kernel with a block per token (48 heads of 64, a wave per
// head against a block per token: 3.8 against 4.1 us at 16 tokens, 4.2 against 4.3 at 64, 5.3 against 4.5
// at 128, 8.5 against 4.9 at 256, 15 us at 2,048)
#ifndef ROPE_TOKEN_KERNEL_FROM
#define ROPE_TOKEN_KERNEL_FROM 96
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

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_rope_cache() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_qk_norm_rope_store<float>)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
