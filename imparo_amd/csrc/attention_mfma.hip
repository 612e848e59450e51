// Matrix-core attention over the paged bfloat16 cache: a split-KV kernel for
// single decoded tokens and a tiled kernel for prompt portions.
//
// Both are built on one wave-level step over a tile of 16 keys for up to 16
// queries, arranged so that nothing has to move between lanes:
//   S^T[key][query] = K . Q^T      A = K rows (8-byte loads), B = Q^T in registers
//   O^T[dim][query] += V^T . P^T   A = V^T (the cache keeps V transposed inside a
//                                  page, so 4 consecutive keys of one dimension
//                                  are one 8-byte load), B = P^T
// In the 16x16 result layout a lane holds column lane%16 and rows 4*(lane/16)+i:
// every value a lane holds belongs to query lane%16, and that is also the B
// operand layout, so the softmax weights feed the second product as they are.
// Cache layouts: K [page, kv head, slot, dim], V [page, kv head, dim, slot].
#include "common.h"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <mutex>
#include "api.h"

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define DEC_SPLIT 256     // keys per decode split, aligned at absolute multiples
#define MFMA_WAVES 4

template <int ND>
struct WaveState {
    f32x4 o[ND];   // O^T rows dt*16 + 4*(lane/16) + i of query lane%16
    s16x4 q[ND];   // Q^T operand: dims dk*16 + 4*(lane/16) + i of query lane%16
    float m, l;
};

struct Paged {
    const bf16_t* __restrict__ k;
    const bf16_t* __restrict__ v;
    const int32_t* __restrict__ table;
    int page_size, kv_heads, kvh, n_pages;
    int page_shift;     // page_size is a power of two: divisions by it are shifts
};

__device__ __forceinline__ short pack_bf16(float f) { return (short)f32_to_bf16(f); }

template <int ND>
__device__ __forceinline__ void load_q(WaveState<ND>& st, const bf16_t* __restrict__ qrow, bool valid, int lane) {
    const int g = lane >> 4;
#pragma unroll
    for (int dk = 0; dk < ND; ++dk) {
        st.q[dk] = valid ? *reinterpret_cast<const s16x4*>(qrow + dk * 16 + 4 * g) : s16x4{0, 0, 0, 0};
        st.o[dk] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.m = -INFINITY;
    st.l = 0.f;
}

// ---------------------------------------------------------------- decode
// The decode kernel walks the keys in tiles of 32 with the 16x16x32 product, so that every
// lane loads 16 bytes at a time (half as many memory instructions as with tiles of 16):
//   S^T: two products of 16 keys x 16 queries per 32 head dims. Which key an output row
//        stands for is free to choose: row m of product t is key 8*(m/4) + 4*t + m%4, so
//        that the 8 scores a lane ends up with (rows 4*(lane/16)+i of both products) are
//        the 8 consecutive keys 8*(lane/16) .. +7,
//   O^T: one product per 16 head dims over the 32 keys, whose B operand wants exactly
//        those 8 consecutive keys per lane, and whose A operand is 16 bytes of a V^T row.
// A head size that is no multiple of 32 pads the last product over head dims with zeros.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
union Frag8 {
    uint4 u;
    bf16x8 v;
};

template <int ND>
struct DecodeState {
    static constexpr int NK = (ND + 1) / 2;      // products of 32 over the head dims
    f32x4 o[ND];        // O^T rows dt*16 + 4*(lane/16) + i of query lane%16
    Frag8 q[NK];        // Q^T operand: dims dk*32 + 8*(lane/16) + j of query lane%16
    float m, l;
};

template <int ND>
struct DecodeTile {
    Frag8 k[2][(ND + 1) / 2];
    Frag8 v[ND];
};

__device__ __forceinline__ uint4 zero_unless(bool keep, uint4 v) {
    return make_uint4(keep ? v.x : 0u, keep ? v.y : 0u, keep ? v.z : 0u, keep ? v.w : 0u);
}

// Issues the loads of the tile starting at key_base (a multiple of 32). [lo_all, hi_all] are
// the live keys any query of the wave may read: addresses are clamped into it (what lies
// outside is forced to zero before use). No load sits under a branch.
template <int ND>
__device__ __forceinline__ void decode_load(DecodeTile<ND>& r, const Paged& kv, int key_base, int lo_all, int hi_all,
                                            int lane) {
    constexpr int D = ND * 16, NK = (ND + 1) / 2;
    const int c = lane & 15, g = lane >> 4;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int key = min(max(key_base + 8 * (c >> 2) + 4 * t + (c & 3), lo_all), hi_all);
        int page = kv.table[key >> kv.page_shift];
        page = min(max(page, 0), kv.n_pages - 1);
        const bf16_t* krow = kv.k + (((size_t)page * kv.kv_heads + kv.kvh) * kv.page_size + (key & (kv.page_size - 1))) * D;
#pragma unroll
        for (int dk = 0; dk < NK; ++dk)          // dims beyond D: read the row's last 8 again, zeroed in decode_tile
            r.k[t][dk].u = *reinterpret_cast<const uint4*>(krow + min(dk * 32 + 8 * g, D - 8));
    }
    const int kgc = min(max(key_base + 8 * g, lo_all & ~7), hi_all & ~7);
    int vpage = kv.table[kgc >> kv.page_shift];
    vpage = min(max(vpage, 0), kv.n_pages - 1);
    const bf16_t* vbase = kv.v + ((size_t)vpage * kv.kv_heads + kv.kvh) * kv.page_size * D + (kgc & (kv.page_size - 1));
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
        r.v[dt].u = *reinterpret_cast<const uint4*>(vbase + (size_t)(dt * 16 + c) * kv.page_size);
}

// One softmax step over a loaded tile of 32 keys. [lo_q, hi_q] is the key range of this
// lane's query. `full`: every key of the tile is inside every query's range.
template <int ND>
__device__ __forceinline__ void decode_tile(DecodeState<ND>& st, const DecodeTile<ND>& r, int key_base, int lo_q,
                                            int hi_q, int lo_all, int hi_all, bool full, float scale, int lane) {
    constexpr int D = ND * 16, NK = (ND + 1) / 2;
    const int g = lane >> 4;
    // ---- scores of keys kg .. kg+7: sv[4*t + i] from product t, row 4*g + i
    f32x4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        s[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dk = 0; dk < NK; ++dk) {
            Frag8 a = r.k[t][dk];
            if (dk * 32 + 32 > D) a.u = zero_unless(dk * 32 + 8 * g < D, a.u);
            s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, st.q[dk].v, s[t], 0, 0, 0);
        }
    }
    const int kg = key_base + 8 * g;
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const bool ok = full || (kg + j >= lo_q && kg + j <= hi_q);
        sv[j] = ok ? s[j >> 2][j & 3] * scale : -INFINITY;
        mx = fmaxf(mx, sv[j]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
    const float m_new = fmaxf(st.m, mx);
    const float corr = (st.m == -INFINITY) ? 0.f : __expf(st.m - m_new);
    union {
        uint4 u;
        bf16x8 v;
        bf16_t h[8];
    } pb;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float p = (sv[j] == -INFINITY) ? 0.f : __expf(sv[j] - m_new);
        pb.h[j] = f32_to_bf16(p);
        psum += bf16_to_f32(pb.h[j]);             // the denominator sums what the product uses
    }
    psum += __shfl_xor(psum, 16, WAVE);
    psum += __shfl_xor(psum, 32, WAVE);
    st.l = st.l * corr + psum;
    st.m = m_new;
    // ---- weighted values
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
        union {
            uint4 u;
            bf16x8 v;
            bf16_t h[8];
        } a;
        a.u = r.v[dt].u;
        if (!full) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                if (kg + j < lo_all || kg + j > hi_all) a.h[j] = 0;   // stale or foreign memory: never multiplied
        }
        st.o[dt] = st.o[dt] * corr;
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, pb.v, st.o[dt], 0, 0, 0);
    }
}

// grid (split, kv head x passes of 16 query heads, decode row). The four waves
// of a block take the split's key tiles in turn, each with the loads of its
// tiles in flight before the first product; their partial results meet in LDS
// and are merged in wave order; one partial (max, sum, O) per split goes to
// scratch for the merge kernel. With a single split the block writes the
// normalised result itself and no merge follows.
// FROM_QKV: the step's rows come as the fused projection's float32 rows [token, (heads + 2 kv_heads) x D]
// instead of finished queries, and their keys and values are not in the cache yet. Every block norms and
// rotates its own queries (the work of one wave over 16 heads; the sines and cosines once a block in
// LDS); the block whose split holds the row's own position also norms and rotates the new key, weighs
// it and the new value in from registers (the cached keys end one position earlier), and, for a layer
// that owns its cache, writes both into their page: the launch that would do all this ahead of the
// attention is gone. Head sizes of 64 and 128 rotated whole, where both elements of a pair (i, i + D/2)
// or (2i, 2i + 1) sit in one lane.
struct FromQkv {
    const float* qkv;
    const float* q_weight;      // per-head norm weights [D], or null: no norm
    const float* k_weight;
    const float* inv_freq;      // [D / 2], or null: no rotation
    bf16_t* k_out;              // the caches again, to write: null for a layer that reads another's cache
    bf16_t* v_out;
    float eps;
    int interleaved;
};

// One head's 8 x NK elements of a lane (dims dk*32 + 8*g + j): asked for early (`head_elements`, with the
// norm's weights), then normed, rotated and rounded to bfloat16 (`normed_rotated`) once the block's sines
// and cosines are there. All lanes with the same lane % 16 share a head: the sum of squares crosses
// lanes 16 and 32 apart. The norm's weights are read from LDS.
template <int ND>
struct HeadElements {
    float e[(ND + 1) / 2][8];
};
template <int ND>
__device__ __forceinline__ void head_elements(HeadElements<ND>& h, const float* src, int g) {
    constexpr int NK = (ND + 1) / 2;
#pragma unroll
    for (int dk = 0; dk < NK; ++dk) {
        const float4 a = *reinterpret_cast<const float4*>(src + dk * 32 + 8 * g);
        const float4 b = *reinterpret_cast<const float4*>(src + dk * 32 + 8 * g + 4);
        h.e[dk][0] = a.x, h.e[dk][1] = a.y, h.e[dk][2] = a.z, h.e[dk][3] = a.w;
        h.e[dk][4] = b.x, h.e[dk][5] = b.y, h.e[dk][6] = b.z, h.e[dk][7] = b.w;
    }
}
template <int ND>
__device__ __forceinline__ void normed_rotated(Frag8 (&out)[(ND + 1) / 2], HeadElements<ND>& h, const float* weight,
                                               float eps, bool rotate, int interleaved, const float* sn_tab,
                                               const float* cs_tab, bool valid, int g) {
    constexpr int D = ND * 16, NK = (ND + 1) / 2;
    static_assert(D % 64 == 0, "pairs inside a lane");
    auto& e = h.e;
    if (weight) {                      // (in LDS)
        float ss = 0.f;
#pragma unroll
        for (int dk = 0; dk < NK; ++dk)
#pragma unroll
            for (int j = 0; j < 8; ++j) ss = fmaf(e[dk][j], e[dk][j], ss);
        ss += __shfl_xor(ss, 16, WAVE);
        ss += __shfl_xor(ss, 32, WAVE);
        const float scale = head_norm_scale(ss, D, eps);
#pragma unroll
        for (int dk = 0; dk < NK; ++dk)
#pragma unroll
            for (int j = 0; j < 8; ++j) e[dk][j] = e[dk][j] * scale * weight[dk * 32 + 8 * g + j];
    }
    if (rotate) {
        if (interleaved) {
#pragma unroll
            for (int dk = 0; dk < NK; ++dk)
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    const int i = dk * 16 + 4 * g + j / 2;
                    const float x0 = e[dk][j], x1 = e[dk][j + 1], sn = sn_tab[i], cs = cs_tab[i];
                    e[dk][j] = fmaf(x0, cs, -(x1 * sn));
                    e[dk][j + 1] = fmaf(x0, sn, x1 * cs);
                }
        } else {
#pragma unroll
            for (int dk = 0; dk < NK / 2; ++dk)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int i = dk * 32 + 8 * g + j;
                    const float x0 = e[dk][j], x1 = e[dk + NK / 2][j], sn = sn_tab[i], cs = cs_tab[i];
                    e[dk][j] = fmaf(x0, cs, -(x1 * sn));
                    e[dk + NK / 2][j] = fmaf(x0, sn, x1 * cs);
                }
        }
    }
#pragma unroll
    for (int dk = 0; dk < NK; ++dk) {
        out[dk].u = make_uint4(f32x2_to_bf16x2(e[dk][0], e[dk][1]), f32x2_to_bf16x2(e[dk][2], e[dk][3]),
                               f32x2_to_bf16x2(e[dk][4], e[dk][5]), f32x2_to_bf16x2(e[dk][6], e[dk][7]));
        out[dk].u = zero_unless(valid, out[dk].u);
    }
}

template <int ND, bool FROM_QKV>
__global__ __launch_bounds__(MFMA_WAVES * 64, ND <= 4 ? 4 : 2) void k_attn_decode(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ seg_start, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ block_table, int table_stride, int page_size, int heads, int kv_heads, int n_pages,
    float scale, int window, int n_splits, FromQkv fq) {
    constexpr int D = ND * 16, NK = (ND + 1) / 2;
    constexpr int TILES = DEC_SPLIT / (MFMA_WAVES * 32);   // tiles a wave takes at most
    __shared__ float sm[MFMA_WAVES][16], sl[MFMA_WAVES][16];
    __shared__ float so[MFMA_WAVES][16][D + 1];
    __shared__ float sn_tab[FROM_QKV ? D / 2 : 1], cs_tab[FROM_QKV ? D / 2 : 1];
    __shared__ __attribute__((aligned(16))) float qw_tab[FROM_QKV ? D : 1], kw_tab[FROM_QKV ? D : 1];
    __shared__ __attribute__((aligned(16))) float k_raw[FROM_QKV ? D : 1], v_raw[FROM_QKV ? D : 1];
    const int split = blockIdx.x, ri = blockIdx.z;
    const int G = heads / kv_heads, passes = (G + 15) / 16;
    const int kvh = blockIdx.y / passes, pass = blockIdx.y % passes;
    const int row = rows[ri];
    const int t = seg_start[row];
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int last = FROM_QKV ? pos - 1 : pos;              // the last key that is in the cache
    const int k_begin = max(split * DEC_SPLIT, lo & ~31);
    const int k_end = min((split + 1) * DEC_SPLIT, last + 1);
    const bool own = FROM_QKV && split == pos / DEC_SPLIT;  // this block weighs the row's own key in
    if (k_begin >= k_end && !own) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int hq = pass * 16 + c;               // query head inside the group
    const bool qvalid = hq < G;
    const int head = kvh * G + min(hq, G - 1);
    DecodeState<ND> st;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    st.m = -INFINITY;
    st.l = 0.f;
    Paged kv{k_cache, v_cache, block_table + (size_t)row * table_stride, page_size, kv_heads, kvh, n_pages,
             __ffs(page_size) - 1};
    const int hi_q = qvalid ? last : -1;
    // (a block with the row's own key only: one clamped tile is loaded and none is used)
    const int lo_c = min(lo, max(last, 0)), last_c = max(last, 0);
    DecodeTile<ND> regs[TILES];
#pragma unroll
    for (int j = 0; j < TILES; ++j)             // past the split's end: clamped addresses, never used
        decode_load<ND>(regs[j], kv, k_begin + (wave + j * MFMA_WAVES) * 32, lo_c, last_c, lane);
    if (!FROM_QKV) {
        const bf16_t* qrow = q + ((size_t)t * heads + head) * D;
#pragma unroll
        for (int dk = 0; dk < NK; ++dk) {
            const int d = dk * 32 + 8 * g;
            st.q[dk].u = zero_unless(qvalid && d < D, *reinterpret_cast<const uint4*>(qrow + min(d, D - 8)));
        }
    }
    const int units = heads + 2 * kv_heads;
    if constexpr (FROM_QKV) {
        // The tiles' loads are on their way; so is the query's row, before anything waits. Meanwhile the
        // block's sines and cosines are worked out and the norms' weights go to LDS.
        HeadElements<ND> qh;
        head_elements<ND>(qh, fq.qkv + ((size_t)t * units + head) * D, g);
        if (fq.inv_freq && (int)threadIdx.x < D / 2)
            rotation_of(pos, fq.inv_freq[threadIdx.x], sn_tab[threadIdx.x], cs_tab[threadIdx.x]);
        if (fq.q_weight && (int)threadIdx.x >= 128 && (int)threadIdx.x < 128 + D / 2) {     // (another wave's lanes)
            const int i = (int)threadIdx.x - 128;
            qw_tab[2 * i] = fq.q_weight[2 * i], qw_tab[2 * i + 1] = fq.q_weight[2 * i + 1];
            kw_tab[2 * i] = fq.k_weight[2 * i], kw_tab[2 * i + 1] = fq.k_weight[2 * i + 1];
        }
        if (own && wave == 1 && lane < D / 2) {      // the row's new key and value wait in LDS for the first wave
            const int u = lane < D / 4 ? heads + kvh : heads + kv_heads + kvh, at = 4 * (lane % (D / 4));
            const float4 x = *reinterpret_cast<const float4*>(fq.qkv + ((size_t)t * units + u) * D + at);
            *reinterpret_cast<float4*>((lane < D / 4 ? k_raw : v_raw) + at) = x;
        }
        __syncthreads();
        normed_rotated<ND>(st.q, qh, fq.q_weight ? qw_tab : nullptr, fq.eps, fq.inv_freq != nullptr, fq.interleaved,
                           sn_tab, cs_tab, qvalid, g);
    }
#pragma unroll
    for (int j = 0; j < TILES; ++j) {
        const int kb = k_begin + (wave + j * MFMA_WAVES) * 32;
        if (kb < k_end) {
            const bool full = kb >= lo && kb + 31 <= last;
            decode_tile<ND>(st, regs[j], kb, lo, hi_q, lo, last, full, scale, lane);
        }
    }
    if constexpr (FROM_QKV) {
        if (own && wave == 0) {
            // the row's own key and value, from the projection's row: every lane holds the key's dims
            // dk*32 + 8*g + j (the same for all 16 heads) and the value's dims dt*16 + 4*g + i
            Frag8 kf[NK];
            HeadElements<ND> kh;
            head_elements<ND>(kh, k_raw, g);
            float4 vnew[ND];
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) vnew[dt] = *reinterpret_cast<const float4*>(v_raw + dt * 16 + 4 * g);
            normed_rotated<ND>(kf, kh, fq.k_weight ? kw_tab : nullptr, fq.eps, fq.inv_freq != nullptr, fq.interleaved,
                               sn_tab, cs_tab, true, g);
            bf16_t vb[ND][4];
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const float4 v4 = vnew[dt];
                vb[dt][0] = f32_to_bf16(v4.x), vb[dt][1] = f32_to_bf16(v4.y);
                vb[dt][2] = f32_to_bf16(v4.z), vb[dt][3] = f32_to_bf16(v4.w);
            }
            float dot = 0.f;
#pragma unroll
            for (int dk = 0; dk < NK; ++dk)
#pragma unroll
                for (int j = 0; j < 8; ++j) dot = fmaf((float)st.q[dk].v[j], (float)kf[dk].v[j], dot);
            dot += __shfl_xor(dot, 16, WAVE);
            dot += __shfl_xor(dot, 32, WAVE);
            if (qvalid) {
                const float sc = dot * scale;
                const float m_new = fmaxf(st.m, sc);
                const float corr = (st.m == -INFINITY) ? 0.f : __expf(st.m - m_new);
                const float p = bf16_to_f32(f32_to_bf16(__expf(sc - m_new)));    // rounded as the tiles' weights are
                st.l = st.l * corr + p;
                st.m = m_new;
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) st.o[dt][i] = fmaf(p, bf16_to_f32(vb[dt][i]), st.o[dt][i] * corr);
            }
            const int page = kv.table[pos >> kv.page_shift];
            if (fq.k_out && pass == 0 && c == 0 && page >= 0 && page < n_pages) {      // never outside the pool
                const int slot = pos & (page_size - 1);
                bf16_t* kdst = fq.k_out + (((size_t)page * kv_heads + kvh) * page_size + slot) * D + 8 * g;
#pragma unroll
                for (int dk = 0; dk < NK; ++dk) *reinterpret_cast<uint4*>(kdst + dk * 32) = kf[dk].u;
                bf16_t* vdst = fq.v_out + ((size_t)page * kv_heads + kvh) * page_size * D + slot;
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) vdst[(size_t)(dt * 16 + 4 * g + i) * page_size] = vb[dt][i];
            }
        }
    }
    if (g == 0) {
        sm[wave][c] = st.m;
        sl[wave][c] = st.l;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt)
#pragma unroll
        for (int i = 0; i < 4; ++i) so[wave][c][dt * 16 + 4 * g + i] = st.o[dt][i];
    __syncthreads();
    for (int e = threadIdx.x; e < 16 * D; e += MFMA_WAVES * 64) {
        const int qc = e / D, d = e - qc * D;
        if (pass * 16 + qc >= G) continue;
        float ms = sm[0][qc];
#pragma unroll
        for (int w = 1; w < MFMA_WAVES; ++w) ms = fmaxf(ms, sm[w][qc]);
        float acc = 0.f, ls = 0.f;
#pragma unroll
        for (int w = 0; w < MFMA_WAVES; ++w) {
            const float f = (sm[w][qc] == -INFINITY) ? 0.f : __expf(sm[w][qc] - ms);
            acc += so[w][qc][d] * f;
            ls += sl[w][qc] * f;
        }
        const int head_out = kvh * G + pass * 16 + qc;
        if (n_splits == 1) {
            out[((size_t)t * heads + head_out) * D + d] = f32_to_bf16(ls > 0.f ? acc / ls : 0.f);
            continue;
        }
        const size_t slot = ((size_t)ri * heads + head_out) * n_splits + split;
        part_o[slot * D + d] = acc;
        if (d == 0) {
            part_ml[slot * 2] = ms;
            part_ml[slot * 2 + 1] = ls;
        }
    }
}

// One wave per (decode row, head): merges the splits in split order. Lane s
// first fetches split s's (max, sum), so the weights of up to 64 splits are
// known after one round trip; the partial outputs then come eight splits at a
// time, all loads of a group issued before the first is used, and are added in
// split order.
__global__ void k_attn_decode_merge(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                    bf16_t* __restrict__ out, const int32_t* __restrict__ rows,
                                    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ positions,
                                    int heads, int head_dim, int n_splits, int window) {
    // A lane holds four neighbouring elements of the head, head_dim / 4 lanes a split's output, so the wave
    // takes several splits side by side (4 at head size 64), each lane GROUP of its splits' loads in flight at
    // once: a wave that fetches split after split makes one trip to memory after the other, and at 128 splits
    // (32,768 keys) the kernel was nothing but those trips (15 us; 4.7 at 16 splits, which is what a launch costs).
    constexpr int GROUP = 8;
    const int ri = blockIdx.x / heads, head = blockIdx.x % heads;
    const int lane = threadIdx.x;
    const int lanes_a_split = head_dim / 4, side = WAVE / lanes_a_split;   // splits side by side
    const int sub = lane / lanes_a_split, d = (lane % lanes_a_split) * 4;
    const bool works = sub < side;
    const int t = seg_start[rows[ri]];
    const int pos = positions[t];
    const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
    const int s_lo = (lo & ~15) / DEC_SPLIT, s_hi = pos / DEC_SPLIT;
    const size_t base = ((size_t)ri * heads + head) * n_splits;
    float ms = -INFINITY;
    for (int s0 = s_lo; s0 <= s_hi; s0 += WAVE) {
        const int s = s0 + lane;
        ms = fmaxf(ms, s <= s_hi ? part_ml[(base + s) * 2] : -INFINITY);
    }
    ms = wave_max(ms);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    float ls = 0.f;
    for (int s0 = s_lo; s0 <= s_hi; s0 += WAVE) {        // lane i holds the weight of split s0 + i
        const int s = s0 + lane;
        float wgt = 0.f, l = 0.f;
        if (s <= s_hi) {
            const float m = part_ml[(base + s) * 2];
            wgt = (m == -INFINITY) ? 0.f : __expf(m - ms);
            l = part_ml[(base + s) * 2 + 1] * wgt;
        }
        ls += l;
        const int n_here = min(WAVE, s_hi - s0 + 1);
        for (int k0 = 0; k0 < n_here; k0 += GROUP * side) {
            float4 v[GROUP];
#pragma unroll
            for (int i = 0; i < GROUP; ++i) {            // past the last split: the last again, weighing nothing
                const int k = min(k0 + i * side + min(sub, side - 1), n_here - 1);
                v[i] = *reinterpret_cast<const float4*>(part_o + (base + s0 + k) * head_dim + d);
            }
#pragma unroll
            for (int i = 0; i < GROUP; ++i) {
                const int k = k0 + i * side + sub;
                const float wk = __shfl(wgt, min(k, WAVE - 1), WAVE);
                const bool on = works && k < n_here;
                acc[0] += on ? v[i].x * wk : 0.f;
                acc[1] += on ? v[i].y * wk : 0.f;
                acc[2] += on ? v[i].z * wk : 0.f;
                acc[3] += on ? v[i].w * wk : 0.f;
            }
        }
    }
    ls = wave_sum(ls);
    // the sums of the splits side by side, added in the order of the sides
    float total[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < side; ++k) {
#pragma unroll
        for (int c = 0; c < 4; ++c) total[c] += __shfl(acc[c], (lane % lanes_a_split) + k * lanes_a_split, WAVE);
    }
    if (sub != 0) return;
    const float inv = ls > 0.f ? 1.0f / ls : 0.f;
    uint2 packed;
    packed.x = f32x2_to_bf16x2(total[0] * inv, total[1] * inv);
    packed.y = f32x2_to_bf16x2(total[2] * inv, total[3] * inv);
    *reinterpret_cast<uint2*>(out + ((size_t)t * heads + head) * head_dim + d) = packed;
}

// ---------------------------------------------------------------- prompt portions
// grid (tile of 64 queries, head). A block's four waves take 16 consecutive
// queries each. Keys go by in tiles of 64: the block stages the K rows and the
// V^T rows of a tile in LDS once (next tile's loads in flight meanwhile), each
// wave multiplies its queries against the four 16-key sub-tiles, runs one
// softmax update over the 64 scores and adds the weighted values. Rows are
// padded to 144 bytes in LDS so that the 8-byte operand reads of 16 rows fall
// on distinct banks.
#define PF_KEYS 64
#define PF_LD_K(D) ((D) + 8)
#define PF_LD_V (PF_KEYS + 8)

// Later tiles of a prompt have more keys to walk, and blocks whose numbers differ by the number
// of CUs tend to share a CU: every other run of 256 blocks (counted along x, then y) takes its
// blocks in reverse, so that a long walk sits beside a short one. The reversal is inside a run
// (the last run may be shorter), so every (tile, y) is still taken exactly once whatever the grid.
__device__ __forceinline__ void snake_block(int& tile, int& by) {
    const int gx = (int)gridDim.x, total = gx * (int)gridDim.y;
    int linear = (int)blockIdx.y * gx + (int)blockIdx.x;
    const int run = linear / 256;
    if (run & 1) {
        const int first = run * 256, last = min(first + 256, total) - 1;
        linear = first + (last - linear);
    }
    by = linear / gx;
    tile = linear - by * gx;
}

template <int ND>
__global__ __launch_bounds__(MFMA_WAVES * 64) void k_attn_prefill(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int32_t* __restrict__ rows, int n_rows,
    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ block_table, int table_stride, int page_size, int heads, int kv_heads, int n_pages,
    float scale, int window) {
    constexpr int D = ND * 16;
    constexpr int LDK = PF_LD_K(D);
    const int page_shift = __ffs(page_size) - 1;          // a power of two: divisions by it are shifts
    __shared__ __attribute__((aligned(16))) bf16_t ks[2][PF_KEYS * LDK];
    __shared__ __attribute__((aligned(16))) bf16_t vs[2][D * PF_LD_V];
    int tile, by, row = -1;
    snake_block(tile, by);
    for (int i = 0; i < n_rows; ++i) {
        const int r = rows[i];
        const int nt = (seg_len[r] + 63) >> 6;
        if (tile < nt) {
            row = r;
            break;
        }
        tile -= nt;
    }
    if (row < 0) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int len = seg_len[row];
    const int head = by;
    const int kvh = head / (heads / kv_heads);
    const int t0 = seg_start[row];
    const int pos0 = positions[t0];
    const int32_t* table = block_table + (size_t)row * table_stride;

    // the block's key range: from the lowest key its first query may read to its last query's position
    const int blk_first = pos0 + tile * 64;
    const int blk_last = pos0 + min(len, tile * 64 + 64) - 1;
    const int blk_lo = window > 0 ? max(0, blk_first + 1 - window) : 0;

    // this wave's queries
    const int q_first = tile * 64 + wave * 16;
    const bool wave_on = q_first < len;
    const int qi = q_first + c;
    const bool qvalid = qi < len;
    const int pos_q = pos0 + qi;
    const int pos_first = pos0 + q_first;
    const int pos_last = pos0 + min(len, q_first + 16) - 1;
    const int lo_q = window > 0 ? max(0, pos_q + 1 - window) : 0;
    const int hi_q = qvalid ? pos_q : -1;
    const int lo_all = window > 0 ? max(0, pos_first + 1 - window) : 0;
    const int lo_max = window > 0 ? max(0, pos_last + 1 - window) : 0;
    WaveState<ND> st;
    load_q<ND>(st, q + ((size_t)(t0 + min(qi, len - 1)) * heads + head) * D, qvalid && wave_on, lane);
    const float scale_log2 = scale * 1.44269504088896340736f;

    // staging: K tile = 64 keys x D/8 pieces of 16 bytes; V^T tile = D rows x 8 pieces of 8 keys
    constexpr int K_PIECES = PF_KEYS * (D / 8), V_PIECES = D * (PF_KEYS / 8);
    constexpr int K_PER = (K_PIECES + 255) / 256, V_PER = (V_PIECES + 255) / 256;
    uint4 kr[K_PER], vr[V_PER];
    auto stage_load = [&](int kb) {
#pragma unroll
        for (int j = 0; j < K_PER; ++j) {
            const int p = tid + j * 256;
            const int key = min(max(kb + p / (D / 8), blk_lo), blk_last);      // a live key: address always valid
            int page = table[key >> page_shift];
            page = min(max(page, 0), n_pages - 1);
            kr[j] = (p < K_PIECES)
                        ? *reinterpret_cast<const uint4*>(k_cache + (((size_t)page * kv_heads + kvh) * page_size +
                                                                     (key & (page_size - 1))) * D + (p % (D / 8)) * 8)
                        : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < V_PER; ++j) {
            const int p = tid + j * 256;
            const int d = p / (PF_KEYS / 8), kg = kb + (p % (PF_KEYS / 8)) * 8;   // 8 keys kg .. kg+7, one page
            const int kgc = min(max(kg, blk_lo & ~7), blk_last & ~7);
            int page = table[kgc >> page_shift];
            page = min(max(page, 0), n_pages - 1);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (p < V_PIECES)
                v = *reinterpret_cast<const uint4*>(v_cache + (((size_t)page * kv_heads + kvh) * D + d) * page_size +
                                                    (kgc & (page_size - 1)));
            // values of keys outside the live range are zero, never stale memory
            if (kg < blk_lo || kg + 7 > blk_last) {
                uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (kg + e < blk_lo || kg + e > blk_last) w[e >> 1] &= (e & 1) ? 0x0000ffffu : 0xffff0000u;
                v = make_uint4(w[0], w[1], w[2], w[3]);
            }
            vr[j] = v;
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int j = 0; j < K_PER; ++j) {
            const int p = tid + j * 256;
            if (p < K_PIECES) *reinterpret_cast<uint4*>(&ks[buf][(p / (D / 8)) * LDK + (p % (D / 8)) * 8]) = kr[j];
        }
#pragma unroll
        for (int j = 0; j < V_PER; ++j) {
            const int p = tid + j * 256;
            if (p < V_PIECES)
                *reinterpret_cast<uint4*>(&vs[buf][(p / (PF_KEYS / 8)) * PF_LD_V + (p % (PF_KEYS / 8)) * 8]) = vr[j];
        }
    };

    const int kb_first = blk_lo & ~(PF_KEYS - 1);
    stage_load(kb_first);
    stage_store(0);
    __syncthreads();
    int buf = 0;
    for (int kb = kb_first; kb <= blk_last; kb += PF_KEYS) {
        const int kn = kb + PF_KEYS;
        if (kn <= blk_last) stage_load(kn);
        // this wave's part of the tile: keys lo_all .. pos_last
        if (wave_on && kb <= pos_last && kb + PF_KEYS - 1 >= lo_all) {
            const bool full = kb >= lo_max && kb + PF_KEYS - 1 <= pos_first;
            f32x4 sc[4];
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                sc[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
                const bf16_t* krow = &ks[buf][(kt * 16 + c) * LDK + 4 * g];
#pragma unroll
                for (int dk = 0; dk < ND; ++dk) {
                    const s16x4 a = *reinterpret_cast<const s16x4*>(krow + dk * 16);
                    sc[kt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, st.q[dk], sc[kt], 0, 0, 0);
                }
            }
            // sc[kt][i] = score of key kb + 16 kt + 4 g + i for query lane%16. The running maximum
            // st.m is kept in units of log2(e), so that every weight is one exp2 of a difference.
            float mx = -INFINITY;
            if (full) {                                   // most tiles: nothing to mask (the same for the whole wave)
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        sc[kt][i] *= scale_log2;
                        mx = fmaxf(mx, sc[kt][i]);
                    }
            } else {
#pragma unroll
                for (int kt = 0; kt < 4; ++kt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int kp = kb + kt * 16 + 4 * g + i;
                        sc[kt][i] = (kp >= lo_q && kp <= hi_q) ? sc[kt][i] * scale_log2 : -INFINITY;
                        mx = fmaxf(mx, sc[kt][i]);
                    }
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float m_new = fmaxf(st.m, mx);
            const float corr = (st.m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(st.m - m_new);
            const float m_sub = (m_new == -INFINITY) ? 0.f : m_new;        // exp2(-inf - 0) = 0: masked keys
            s16x4 pb[4];
            float psum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; ++kt) {
                union {
                    uint32_t u[2];
                    s16x4 v;
                } pk;
#pragma unroll
                for (int i = 0; i < 4; i += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(sc[kt][i] - m_sub), p1 = __builtin_amdgcn_exp2f(sc[kt][i + 1] - m_sub);
                    pk.u[i >> 1] = f32x2_to_bf16x2(p0, p1);
                    // the denominator sums what the product uses
                    psum += __uint_as_float(pk.u[i >> 1] << 16) + __uint_as_float(pk.u[i >> 1] & 0xffff0000u);
                }
                pb[kt] = pk.v;
            }
            psum += __shfl_xor(psum, 16, WAVE);
            psum += __shfl_xor(psum, 32, WAVE);
            st.l = st.l * corr + psum;
            st.m = m_new;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                st.o[dt] = st.o[dt] * corr;
                const bf16_t* vrow = &vs[buf][(dt * 16 + c) * PF_LD_V + 4 * g];
#pragma unroll
                for (int kt = 0; kt < 4; ++kt) {
                    const s16x4 a = *reinterpret_cast<const s16x4*>(vrow + kt * 16);
                    st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, pb[kt], st.o[dt], 0, 0, 0);
                }
            }
        }
        if (kn <= blk_last) stage_store(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if (!qvalid || !wave_on) return;
    const float inv = st.l > 0.f ? 1.0f / st.l : 0.f;
    bf16_t* dst = out + ((size_t)(t0 + qi) * heads + head) * D + 4 * g;
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
        s16x4 v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = pack_bf16(st.o[dt][i] * inv);
        *reinterpret_cast<s16x4*>(dst + dt * 16) = v;
    }
}

// ---------------------------------------------------------------- prompt portions, head sizes in steps of 32
// The same walk with the 16x16x32 product and more work per staged tile. A wave takes 32
// queries of one head as two halves of 16 that share every K and V^T fragment it reads from
// LDS; a block's four waves are four heads that share a kv head (or two heads x two runs of
// 32 queries, or one head x four runs, as the group size allows), so a tile of 64 keys is
// fetched and staged once for all of them. Per 32 head dims, S^T of 16 keys x 16 queries is
// one product; a lane's scores of the two products over keys 16t .. 16t+15 (t = 0, 1) of a
// group of 32 keys are keys 16t + 4*(lane/16) + i, and those eight are the lane's eight
// K-slots of the second product's B operand as they are. Its A operand, 16 bytes of a V^T
// row, must hold the same eight keys: the V^T tile is staged with its keys in that order
// (key k of a group of 32 at 8*((k%16)/4) + 4*(k/16) + k%4).
#define PX_KEYS 64

// (Two blocks per CU for head sizes up to 64: within 256 registers a wave the compiler keeps the
// products' results in vector registers, where the softmax wants them, not in the accumulator file.)
// HALVES: 2 for 32 queries a wave; 1 for 16, twice the waves, when a launch has too few to fill the SIMDs twice.
// PAGE_TILE: pages of at least 64 positions, so that a tile of 64 keys lies in one page. One look at the
// block table a tile then serves every thread, and what a thread reads of a tile is at a fixed place
// inside the page: a quarter of the instructions of the general staging, which was a quarter to a
// third of the kernel's time.
template <int ND, int HALVES, bool PAGE_TILE>
__global__ __launch_bounds__(MFMA_WAVES * 64, ND <= 4 ? 2 : 1) void k_attn_prefill_x32(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int32_t* __restrict__ rows, int n_rows,
    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ block_table, int table_stride, int page_size, int heads, int kv_heads, int n_pages,
    float scale, int window, int heads_per_block, float* __restrict__ part_o, float* __restrict__ part_ml) {
    constexpr int D = ND * 16, NK = ND / 2;
    // Rows of K lie their length + 32 bytes apart: the fragment reads (row lane % 16, 16-byte piece lane / 16) then
    // meet no bank conflict at any head size (with 16 bytes of padding each read takes 8 cycles instead of 4; counted
    // with SQ_LDS_BANK_CONFLICT on reads alone). V^T rows keep 16 bytes: 32 would free its reads too but make the
    // staging stores of its reordered keys collide instead, and the kernel gains nothing more from it (measured).
    constexpr int LDK = D + 16, LDV = PX_KEYS + 8;
    static_assert(ND % 2 == 0, "head sizes in steps of 32");
    const int page_shift = __ffs(page_size) - 1;
    __shared__ __attribute__((aligned(16))) bf16_t ks[2][PX_KEYS * LDK];
    __shared__ __attribute__((aligned(16))) bf16_t vs[2][D * LDV];
    constexpr int QW = 16 * HALVES;                       // queries of a wave
    const int runs = MFMA_WAVES / heads_per_block;        // runs of QW queries per block
    const int qt = QW * runs;                             // queries per block and head
    int tile, by, row = -1;
    snake_block(tile, by);
    for (int i = 0; i < n_rows; ++i) {
        const int r = rows[i];
        const int nt = (seg_len[r] + qt - 1) / qt;
        if (tile < nt) {
            row = r;
            break;
        }
        tile -= nt;
    }
    if (row < 0) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int len = seg_len[row];
    const int head = by * heads_per_block + wave % heads_per_block;
    const int kvh = (by * heads_per_block) / (heads / kv_heads);
    const int t0 = seg_start[row];
    const int pos0 = positions[t0];
    const int32_t* table = block_table + (size_t)row * table_stride;

    // the block's key range: from the lowest key its first query may read to its last query's position;
    // with splits (gridDim.z > 1: few queries over long contexts) block z takes the z-th part of its tiles
    // of keys and leaves (max, sum, unnormalised output) per query for the merge kernel
    const int blk_first = pos0 + tile * qt;
    int blk_last = pos0 + min(len, tile * qt + qt) - 1;
    int blk_lo = window > 0 ? max(0, blk_first + 1 - window) : 0;
    const int n_splits = (int)gridDim.z, split = (int)blockIdx.z;
    if (n_splits > 1) {
        const int first_tile = blk_lo / PX_KEYS, tiles_all = blk_last / PX_KEYS - first_tile + 1;
        const int per = (tiles_all + n_splits - 1) / n_splits;
        blk_lo = max(blk_lo, (first_tile + split * per) * PX_KEYS);
        blk_last = min(blk_last, (first_tile + (split + 1) * per) * PX_KEYS - 1);
    }
    const bool has_keys = blk_lo <= blk_last;
    if (!has_keys) blk_lo = blk_last = max(blk_first, 0);       // nothing to add: one masked tile, a partial of zero weight

    // this wave's queries: q_first + 16 h + c for the halves h
    const int q_first = tile * qt + (wave / heads_per_block) * QW;
    const bool wave_on = q_first < len;
    const int pos_first = pos0 + q_first;
    const int pos_last = pos0 + min(len, q_first + QW) - 1;
    const int lo_all = window > 0 ? max(0, pos_first + 1 - window) : 0;
    const int lo_max = window > 0 ? max(0, pos_last + 1 - window) : 0;
    int lo_q[HALVES], hi_q[HALVES];
    bool qvalid[HALVES];
    Frag8 qf[HALVES][NK];
    f32x4 o[HALVES][ND];
    float m_run[HALVES];
    // The sums of the weights come out of the matrix pipe too: one more product per group of 32 keys whose
    // "values" are all ones leaves each query's sum in every row of its column. It sums the weights as the
    // value products use them, rounded to bfloat16, and takes 32 additions and two exchanges a tile off
    // the vector ALUs, which are what bounds this kernel.
    f32x4 l_acc[HALVES];
    Frag8 ones;
    ones.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
#pragma unroll
    for (int h = 0; h < HALVES; ++h) {
        const int qi = q_first + 16 * h + c;
        qvalid[h] = qi < len;
        const int pos_q = pos0 + qi;
        lo_q[h] = max(window > 0 ? max(0, pos_q + 1 - window) : 0, blk_lo);
        hi_q[h] = (qvalid[h] && has_keys) ? min(pos_q, blk_last) : -1;
        const bf16_t* qrow = q + ((size_t)(t0 + min(qi, len - 1)) * heads + head) * D + 8 * g;
#pragma unroll
        for (int dk = 0; dk < NK; ++dk)
            qf[h][dk].u = zero_unless(qvalid[h] && wave_on, *reinterpret_cast<const uint4*>(qrow + 32 * dk));
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) o[h][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[h] = -INFINITY;
        l_acc[h] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const float scale_log2 = scale * 1.44269504088896340736f;

    // Staging: K tile = 64 keys x D/8 pieces of 16 bytes; V^T tile = D rows x 8 pieces of 8 keys; with
    // head sizes in steps of 32 the 256 threads take a whole number of pieces each. A piece's
    // page comes out of the block table first and its data from that page: two trips to memory
    // in a row. So the pages of a tile are asked for a tile ahead of its data, the data a tile
    // ahead of its use, and no load sits under a branch (past the last tile they read the
    // last tile again): the waits then fall where the values are needed and nowhere else. With long
    // contexts the keys come from HBM and take longer than a tile's arithmetic: two register sets,
    // so that a tile's data is asked for two tiles before it goes to LDS.
    constexpr int K_PER = PX_KEYS * (D / 8) / 256, V_PER = D * (PX_KEYS / 8) / 256;
    static_assert(K_PER * 256 == PX_KEYS * (D / 8) && V_PER * 256 == D * (PX_KEYS / 8), "whole pieces per thread");
    const size_t page_elems = (size_t)kv_heads * page_size * D;      // of one page of K (or V) over all kv heads
    // (the compiler's own vector type: an array of HIP's uint4 stays in memory)
    u32x4 kr_a[K_PER], vr_a[V_PER], kr_b[K_PER], vr_b[V_PER];
    int kpage[K_PER], vpage[V_PER];
    const int kb_last = blk_last & ~(PX_KEYS - 1);
    // PAGE_TILE: where in a page this thread's pieces of a tile lie that starts at the page's first position
    unsigned k_at[K_PER], v_at[V_PER];
#pragma unroll
    for (int j = 0; j < K_PER; ++j) {
        const int pc = tid + j * 256;
        k_at[j] = (unsigned)(kvh * page_size + pc / (D / 8)) * D + (pc % (D / 8)) * 8;
    }
#pragma unroll
    for (int j = 0; j < V_PER; ++j) {
        const int pc = tid + j * 256;
        v_at[j] = (unsigned)(kvh * D + pc / (PX_KEYS / 8)) * page_size + (pc % (PX_KEYS / 8)) * 8;
    }
    auto load_pages = [&](int kb) __attribute__((always_inline)) {
        kb = min(kb, kb_last);
        if constexpr (PAGE_TILE) {
            kpage[0] = table[kb >> page_shift];       // the tile's page: it holds a live key, so it is there
            return;
        }
#pragma unroll
        for (int j = 0; j < K_PER; ++j) {
            const int pc = tid + j * 256;
            const int key = min(max(kb + pc / (D / 8), blk_lo), blk_last);     // a live key: address always valid
            kpage[j] = table[key >> page_shift];
        }
#pragma unroll
        for (int j = 0; j < V_PER; ++j) {
            const int pc = tid + j * 256;
            const int kgc = min(max(kb + (pc % (PX_KEYS / 8)) * 8, blk_lo & ~7), blk_last & ~7);
            vpage[j] = table[kgc >> page_shift];
        }
    };
    auto load_data = [&](int kb, u32x4 (&kr)[K_PER], u32x4 (&vr)[V_PER]) __attribute__((always_inline)) {
        kb = min(kb, kb_last);
        if constexpr (PAGE_TILE) {
            // (keys of the page outside the live range are read too: what they hold is masked, and zeroed
            // where it would be multiplied)
            const size_t base = (size_t)min(max(kpage[0], 0), n_pages - 1) * page_elems;
            const unsigned first = (unsigned)(kb & (page_size - 1));
#pragma unroll
            for (int j = 0; j < K_PER; ++j) kr[j] = *reinterpret_cast<const u32x4*>(k_cache + base + k_at[j] + first * D);
#pragma unroll
            for (int j = 0; j < V_PER; ++j) vr[j] = *reinterpret_cast<const u32x4*>(v_cache + base + v_at[j] + first);
            return;
        }
#pragma unroll
        for (int j = 0; j < K_PER; ++j) {
            const int pc = tid + j * 256;
            const int key = min(max(kb + pc / (D / 8), blk_lo), blk_last);
            const int page = min(max(kpage[j], 0), n_pages - 1);
            const unsigned in_page = (unsigned)(kvh * page_size + (key & (page_size - 1))) * D + (pc % (D / 8)) * 8;
            kr[j] = *reinterpret_cast<const u32x4*>(k_cache + (size_t)page * page_elems + in_page);
        }
#pragma unroll
        for (int j = 0; j < V_PER; ++j) {
            const int pc = tid + j * 256;
            const int d = pc / (PX_KEYS / 8);
            const int kgc = min(max(kb + (pc % (PX_KEYS / 8)) * 8, blk_lo & ~7), blk_last & ~7);   // 8 keys, one page
            const int page = min(max(vpage[j], 0), n_pages - 1);
            const unsigned in_page = (unsigned)(kvh * D + d) * page_size + (kgc & (page_size - 1));
            vr[j] = *reinterpret_cast<const u32x4*>(v_cache + (size_t)page * page_elems + in_page);
        }
    };
    // the tile whose data is in kr/vr goes to LDS: kb is its first key
    auto stage_store = [&](int kb, int buf, const u32x4 (&kr)[K_PER], const u32x4 (&vr)[V_PER]) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < K_PER; ++j) {
            const int pc = tid + j * 256;
            *reinterpret_cast<u32x4*>(&ks[buf][(pc / (D / 8)) * LDK + (pc % (D / 8)) * 8]) = kr[j];
        }
#pragma unroll
        for (int j = 0; j < V_PER; ++j) {
            const int pc = tid + j * 256;
            const int q8 = pc % (PX_KEYS / 8);
            const int kg = kb + q8 * 8;
            // values of keys outside the live range are zero, never stale memory (a tile at either
            // end of the block's range only: the same for every thread)
            uint32_t w[4] = {vr[j].x, vr[j].y, vr[j].z, vr[j].w};
            if (kb < blk_lo || kb + PX_KEYS - 1 > blk_last) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const bool dead = kg + e < blk_lo || kg + e > blk_last;
                    w[e >> 1] = dead ? (w[e >> 1] & ((e & 1) ? 0x0000ffffu : 0xffff0000u)) : w[e >> 1];
                }
            }
            // keys 8 q8 .. +7 of the tile: the first four go to 32 G + 16 (q8 % 2) + 4 t, the next four 8 further
            bf16_t* dst = &vs[buf][(pc / (PX_KEYS / 8)) * LDV + 32 * (q8 >> 2) + 16 * (q8 & 1) + 4 * ((q8 >> 1) & 1)];
            *reinterpret_cast<uint2*>(dst) = make_uint2(w[0], w[1]);
            *reinterpret_cast<uint2*>(dst + 8) = make_uint2(w[2], w[3]);
        }
    };

    // One tile: LDS buffer `buf` holds it and `have` the next tile's data, asked for two tiles ago, which goes
    // to the other LDS buffer once this tile is done; the set is then free and takes the loads of the tile
    // three further on (the other set holds the tile in between).
    auto tile_step = [&](int kb, int buf, u32x4 (&kr_have)[K_PER], u32x4 (&vr_have)[V_PER]) __attribute__((always_inline)) {
        // this wave's part of the tile: keys lo_all .. pos_last
        if (wave_on && kb <= pos_last && kb + PX_KEYS - 1 >= lo_all) {
            const bool full = kb >= lo_max && kb + PX_KEYS - 1 <= pos_first && kb >= blk_lo && kb + PX_KEYS - 1 <= blk_last;
            f32x4 sc[HALVES][4];
#pragma unroll
            for (int s16 = 0; s16 < 4; ++s16) {
#pragma unroll
                for (int h = 0; h < HALVES; ++h) sc[h][s16] = f32x4{0.f, 0.f, 0.f, 0.f};
                const bf16_t* krow = &ks[buf][(s16 * 16 + c) * LDK + 8 * g];
#pragma unroll
                for (int dk = 0; dk < NK; ++dk) {
                    Frag8 kf;
                    kf.u = *reinterpret_cast<const uint4*>(krow + dk * 32);
#pragma unroll
                    for (int h = 0; h < HALVES; ++h)
                        sc[h][s16] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[h][dk].v, sc[h][s16], 0, 0, 0);
                }
            }
            // sc[h][s16][i] = score of key kb + 16 s16 + 4 g + i for query (h, lane%16), unscaled. The
            // running maximum is kept unscaled too: a weight is one fused multiply-add and one exp2,
            // exp2((score - max) * scale * log2 e). The vector ALUs are what this kernel is bound by.
            Frag8 pb[HALVES][2];
#pragma unroll
            for (int h = 0; h < HALVES; ++h) {
                float mx = -INFINITY;
                if (full) {                               // most tiles: nothing to mask (the same for the whole wave)
#pragma unroll
                    for (int s16 = 0; s16 < 4; ++s16)
#pragma unroll
                        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sc[h][s16][i]);
                } else {
#pragma unroll
                    for (int s16 = 0; s16 < 4; ++s16)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int kp = kb + s16 * 16 + 4 * g + i;
                            sc[h][s16][i] = (kp >= lo_q[h] && kp <= hi_q[h]) ? sc[h][s16][i] : -INFINITY;
                            mx = fmaxf(mx, sc[h][s16][i]);
                        }
                }
                mx = fmaxf(mx, __shfl_xor(mx, 16, WAVE));
                mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
                const float m_new = fmaxf(m_run[h], mx);
                const float m_sub = (m_new == -INFINITY) ? 0.f : m_new * scale_log2;   // exp2(-inf - 0) = 0: masked keys
#pragma unroll
                for (int s16 = 0; s16 < 4; ++s16) {
                    uint32_t pk[2];
#pragma unroll
                    for (int i = 0; i < 4; i += 2) {
                        const float p0 = __builtin_amdgcn_exp2f(fmaf(sc[h][s16][i], scale_log2, -m_sub));
                        const float p1 = __builtin_amdgcn_exp2f(fmaf(sc[h][s16][i + 1], scale_log2, -m_sub));
                        pk[i >> 1] = f32x2_to_bf16x2(p0, p1);
                    }
                    // K-slots 4 t + i of group G, s16 = 2 G + t
                    if (s16 & 1) {
                        pb[h][s16 >> 1].u.z = pk[0];
                        pb[h][s16 >> 1].u.w = pk[1];
                    } else {
                        pb[h][s16 >> 1].u.x = pk[0];
                        pb[h][s16 >> 1].u.y = pk[1];
                    }
                }
                // the old sums shrink by exp2((old max - new max) * scale): by 1, and nothing to do, for
                // every query whose maximum stood (the whole wave mostly, once the walk is under way)
                if (__any(m_new != m_run[h])) {
                    const float corr = (m_run[h] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run[h] - m_new) * scale_log2);
                    l_acc[h] = l_acc[h] * corr;
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt) o[h][dt] = o[h][dt] * corr;
                }
                m_run[h] = m_new;
#pragma unroll
                for (int G = 0; G < 2; ++G)
                    l_acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pb[h][G].v, l_acc[h], 0, 0, 0);
            }
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const bf16_t* vrow = &vs[buf][(dt * 16 + c) * LDV + 8 * g];
#pragma unroll
                for (int G = 0; G < 2; ++G) {
                    Frag8 vf;
                    vf.u = *reinterpret_cast<const uint4*>(vrow + 32 * G);
#pragma unroll
                    for (int h = 0; h < HALVES; ++h)
                        o[h][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pb[h][G].v, o[h][dt], 0, 0, 0);
                }
            }
        }
        stage_store(min(kb + PX_KEYS, kb_last), buf ^ 1, kr_have, vr_have);
        load_data(kb + 3 * PX_KEYS, kr_have, vr_have);      // with the pages asked for a tile ago
        load_pages(kb + 4 * PX_KEYS);
        __syncthreads();
    };
    const int kb_first = blk_lo & ~(PX_KEYS - 1);
    load_pages(kb_first);
    load_data(kb_first, kr_a, vr_a);
    load_pages(kb_first + PX_KEYS);
    load_data(kb_first + PX_KEYS, kr_b, vr_b);
    load_pages(kb_first + 2 * PX_KEYS);
    stage_store(kb_first, 0, kr_a, vr_a);
    load_data(kb_first + 2 * PX_KEYS, kr_a, vr_a);
    load_pages(kb_first + 3 * PX_KEYS);
    __syncthreads();
    for (int kb = kb_first; kb <= blk_last; kb += 2 * PX_KEYS) {
        tile_step(kb, 0, kr_b, vr_b);
        if (kb + PX_KEYS > blk_last) break;
        tile_step(kb + PX_KEYS, 1, kr_a, vr_a);
    }
    if (!wave_on) return;
    if (n_splits > 1) {
#pragma unroll
        for (int h = 0; h < HALVES; ++h) {
            if (!qvalid[h]) continue;
            const size_t slot = ((size_t)(t0 + q_first + 16 * h + c) * heads + head) * n_splits + split;
            if (g == 0) {
                part_ml[slot * 2] = m_run[h];               // of unscaled scores; -inf: no key, weight zero
                part_ml[slot * 2 + 1] = l_acc[h][0];
            }
            float* dst = part_o + slot * D + 4 * g;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
                *reinterpret_cast<float4*>(dst + dt * 16) = make_float4(o[h][dt][0], o[h][dt][1], o[h][dt][2], o[h][dt][3]);
        }
        return;
    }
#pragma unroll
    for (int h = 0; h < HALVES; ++h) {
        if (!qvalid[h]) continue;
        const float inv = l_acc[h][0] > 0.f ? 1.0f / l_acc[h][0] : 0.f;
        bf16_t* dst = out + ((size_t)(t0 + q_first + 16 * h + c) * heads + head) * D + 4 * g;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) {
            s16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = pack_bf16(o[h][dt][i] * inv);
            *reinterpret_cast<s16x4*>(dst + dt * 16) = v;
        }
    }
}

// Merges the parts of the kernel above for the launch's portion rows, in the order of the parts: weights
// exp2((max_s - max) * scale * log2 e), as the kernel itself weighs its tiles. A lane holds four
// neighbouring elements of a head, so head_dim / 4 lanes hold a head and a wave several heads; GROUP parts
// at a time, every load of a group asked for before the first is used and none under a branch (past the
// last part the last is read again and weighs nothing): a wave that fetches part after part makes one trip
// to memory after the other, and the kernel is nothing but those trips.
template <int GROUP>
__global__ void k_attn_prefill_merge(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                     bf16_t* __restrict__ out, const int32_t* __restrict__ rows, int n_rows,
                                     const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
                                     int heads, int head_dim, int n_splits, float scale) {
    int tok = blockIdx.x, t = -1;
    for (int i = 0; i < n_rows; ++i) {                   // the tok-th token of the listed rows
        const int r = rows[i];
        if (tok < seg_len[r]) {
            t = seg_start[r] + tok;
            break;
        }
        tok -= seg_len[r];
    }
    if (t < 0) return;
    const int lanes_a_head = head_dim / 4, heads_a_wave = 64 / lanes_a_head;
    const int lane = threadIdx.x & 63, wave = blockIdx.y * (blockDim.x / 64) + (threadIdx.x >> 6);
    const int sub = lane / lanes_a_head, d = (lane % lanes_a_head) * 4;
    const int head = wave * heads_a_wave + sub;
    if (sub >= heads_a_wave || head >= heads) return;
    const size_t base = ((size_t)t * heads + head) * n_splits;
    const float scale_log2 = scale * 1.44269504088896340736f;
    float ms = -INFINITY;
    for (int s0 = 0; s0 < n_splits; s0 += GROUP) {
        float2 ml[GROUP];
#pragma unroll
        for (int j = 0; j < GROUP; ++j)
            ml[j] = *reinterpret_cast<const float2*>(part_ml + (base + min(s0 + j, n_splits - 1)) * 2);
#pragma unroll
        for (int j = 0; j < GROUP; ++j) ms = fmaxf(ms, ml[j].x);
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f}, ls = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += GROUP) {
        float2 ml[GROUP];
        float4 o[GROUP];
#pragma unroll
        for (int j = 0; j < GROUP; ++j) {
            const size_t at = base + min(s0 + j, n_splits - 1);
            ml[j] = *reinterpret_cast<const float2*>(part_ml + at * 2);
            o[j] = *reinterpret_cast<const float4*>(part_o + at * head_dim + d);
        }
#pragma unroll
        for (int j = 0; j < GROUP; ++j) {                // in the order of the parts
            // a part without keys has maximum -inf and an output that was never a sum: weight zero, never multiplied
            const bool counts = s0 + j < n_splits && ml[j].x != -INFINITY;
            const float wgt = counts ? __builtin_amdgcn_exp2f((ml[j].x - ms) * scale_log2) : 0.f;
            ls += counts ? ml[j].y * wgt : 0.f;
            acc[0] += counts ? o[j].x * wgt : 0.f;
            acc[1] += counts ? o[j].y * wgt : 0.f;
            acc[2] += counts ? o[j].z * wgt : 0.f;
            acc[3] += counts ? o[j].w * wgt : 0.f;
        }
    }
    const float inv = ls > 0.f ? 1.0f / ls : 0.f;
    uint2 packed;
    packed.x = (uint32_t)f32_to_bf16(acc[0] * inv) | ((uint32_t)f32_to_bf16(acc[1] * inv) << 16);
    packed.y = (uint32_t)f32_to_bf16(acc[2] * inv) | ((uint32_t)f32_to_bf16(acc[3] * inv) << 16);
    *reinterpret_cast<uint2*>(out + ((size_t)t * heads + head) * head_dim + d) = packed;
}

// ---------------------------------------------------------------- entry points
static int check_common(const void* q, const void* k_cache, const void* v_cache, const void* out, const int32_t* rows,
                        const int32_t* seg_start, const int32_t* positions, const int32_t* block_table,
                        int table_stride, int page_size, int heads, int kv_heads, int head_dim, int n_pages, int window) {
    if (!q || !k_cache || !v_cache || !out || !rows || !seg_start || !positions || !block_table)
        return IMPARO_BAD_ARGUMENT;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0) return IMPARO_BAD_ARGUMENT;
    if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > 128) return IMPARO_BAD_ARGUMENT;
    if (page_size < 16 || (page_size & (page_size - 1)) != 0) return IMPARO_BAD_ARGUMENT;
    if (table_stride <= 0 || n_pages <= 0 || window < 0) return IMPARO_BAD_ARGUMENT;
    return IMPARO_OK;
}

#define DISPATCH_ND(nd, CALL)                                                                                        \
    switch (nd) {                                                                                                    \
        case 1: { constexpr int ND = 1; CALL; } break;                                                               \
        case 2: { constexpr int ND = 2; CALL; } break;                                                               \
        case 3: { constexpr int ND = 3; CALL; } break;                                                               \
        case 4: { constexpr int ND = 4; CALL; } break;                                                               \
        case 5: { constexpr int ND = 5; CALL; } break;                                                               \
        case 6: { constexpr int ND = 6; CALL; } break;                                                               \
        case 7: { constexpr int ND = 7; CALL; } break;                                                               \
        case 8: { constexpr int ND = 8; CALL; } break;                                                               \
        default: return IMPARO_BAD_ARGUMENT;                                                                         \
    }

// The two numbers of these kernels' geometry that a caller sizes things by: a decode row's keys are
// split in runs of this many (the partial results' buffers hold one entry per run), and prompt
// portions are counted in tiles of this many queries (n_tiles of imparo_attention_prefill).
extern "C" int imparo_attention_decode_split() { return DEC_SPLIT; }
extern "C" int imparo_attention_prefill_tile() { return 64; }

static int attention_decode_launch(const void* q, const void* k_cache, const void* v_cache, void* out,
                                   float* part_o, float* part_ml, const int32_t* rows, int n_rows,
                                   const int32_t* seg_start, const int32_t* positions,
                                   const int32_t* block_table, int table_stride, int page_size,
                                   int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                   int n_splits, hipStream_t s, const FromQkv* from_qkv = nullptr) {
    const int G = heads / kv_heads;
    // the merge moves four elements of a head in one access
    if (n_splits > 1 && (((uintptr_t)part_o & 15) || ((uintptr_t)out & 7))) return IMPARO_BAD_ARGUMENT;
    dim3 grid(n_splits, kv_heads * ((G + 15) / 16), n_rows);
    if (from_qkv) {
#define DECODE_FROM_QKV(ND)                                                                                          \
    k_attn_decode<ND, true><<<grid, MFMA_WAVES * 64, 0, s>>>(                                                        \
        nullptr, (const bf16_t*)k_cache, (const bf16_t*)v_cache, part_o, part_ml, (bf16_t*)out, rows, seg_start,     \
        positions, block_table, table_stride, page_size, heads, kv_heads, n_pages, scale, window, n_splits, *from_qkv)
        if (head_dim == 64) DECODE_FROM_QKV(4);
        else if (head_dim == 128) DECODE_FROM_QKV(8);
        else return IMPARO_BAD_ARGUMENT;
#undef DECODE_FROM_QKV
    } else {
        DISPATCH_ND(head_dim / 16, (k_attn_decode<ND, false><<<grid, MFMA_WAVES * 64, 0, s>>>(
            (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, part_o, part_ml, (bf16_t*)out, rows,
            seg_start, positions, block_table, table_stride, page_size, heads, kv_heads, n_pages, scale, window,
            n_splits, FromQkv{})));
    }
    if (launch_status()) return IMPARO_LAUNCH_FAILED;
    if (n_splits == 1) return IMPARO_OK;
    k_attn_decode_merge<<<n_rows * heads, 64, 0, s>>>(part_o, part_ml, (bf16_t*)out, rows, seg_start, positions, heads,
                                                      head_dim, n_splits, window);
    return launch_status();
}

extern "C" int imparo_attention_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                                       float* part_o, float* part_ml, const int32_t* rows, int n_rows,
                                       const int32_t* seg_start, const int32_t* positions,
                                       const int32_t* block_table, int table_stride, int page_size,
                                       int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                       int n_splits, imparo_stream stream) {
    const int bad = check_common(q, k_cache, v_cache, out, rows, seg_start, positions, block_table, table_stride,
                                 page_size, heads, kv_heads, head_dim, n_pages, window);
    if (bad) return bad;
    if (!part_o || !part_ml || n_rows < 0 || n_splits <= 0 || n_splits > 65535) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    if (n_rows > 65535) return IMPARO_BAD_ARGUMENT;
    return attention_decode_launch(q, k_cache, v_cache, out, part_o, part_ml, rows, n_rows, seg_start, positions,
                                   block_table, table_stride, page_size, heads, kv_heads, head_dim, n_pages, scale,
                                   window, n_splits, (hipStream_t)stream);
}

// Which head sizes and rotations imparo_attention_decode_qkv takes: 64 or 128, rotated whole or not at all.
extern "C" int imparo_attention_decode_qkv_takes(int head_dim, int n_freq) {
    return (head_dim == 64 || head_dim == 128) && (n_freq == 0 || 2 * n_freq == head_dim);
}
// ... and for how many rows it is the faster way: every block of a row's splits makes the row's queries
// again, which a launch of its own does once (measured at 4,096 keys: 18.9 against 16.7 + 4.6 us for 8
// rows, 6 us a layer slower for 64). With many splits a row the repeated work adds up: whole decode steps
// of 1 to 16 rows at 4,096 to 32,768 keys are 1 to 3 % faster with the one launch up to 16 rows x 64 splits
// and 8 x 128, and 1.3 % slower at 16 x 128.
extern "C" int imparo_attention_decode_qkv_pays(int n_rows, int n_splits) {
    return n_rows <= 16 && (long long)n_rows * n_splits <= 1024;
}

extern "C" int imparo_attention_decode_qkv(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                                           const float* inv_freq, int n_freq, int interleaved, void* k_cache,
                                           void* v_cache, int write_kv, void* out, float* part_o, float* part_ml,
                                           const int32_t* rows, int n_rows, const int32_t* seg_start,
                                           const int32_t* positions, const int32_t* block_table, int table_stride,
                                           int page_size, int heads, int kv_heads, int head_dim, int n_pages,
                                           float scale, int window, int n_splits, imparo_stream stream) {
    const int bad = check_common(qkv, k_cache, v_cache, out, rows, seg_start, positions, block_table, table_stride,
                                 page_size, heads, kv_heads, head_dim, n_pages, window);
    if (bad) return bad;
    if (!part_o || !part_ml || n_rows < 0 || n_splits <= 0 || n_splits > 65535) return IMPARO_BAD_ARGUMENT;
    if (!imparo_attention_decode_qkv_takes(head_dim, n_freq) || (n_freq > 0 && !inv_freq)) return IMPARO_BAD_ARGUMENT;
    if ((q_weight == nullptr) != (k_weight == nullptr) || (q_weight && !(eps > 0.f))) return IMPARO_BAD_ARGUMENT;
    if (((uintptr_t)qkv | (uintptr_t)q_weight | (uintptr_t)k_weight | (uintptr_t)k_cache) % 16 != 0)
        return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    if (n_rows > 65535) return IMPARO_BAD_ARGUMENT;
    const FromQkv fq{qkv, q_weight, k_weight, n_freq > 0 ? inv_freq : nullptr, write_kv ? (bf16_t*)k_cache : nullptr,
                     write_kv ? (bf16_t*)v_cache : nullptr, eps, interleaved};
    return attention_decode_launch(nullptr, k_cache, v_cache, out, part_o, part_ml, rows, n_rows, seg_start, positions,
                                   block_table, table_stride, page_size, heads, kv_heads, head_dim, n_pages, scale,
                                   window, n_splits, (hipStream_t)stream, &fq);
}

// ---------------------------------------------------------------- decode without a workspace argument
// The splits' partial results live in an array of this library's own instead of a buffer the caller
// brings, so that the call allocates nothing. Every GPU holds its own copy of the array at its own
// address: the address is asked for once per device, with that device current, and kept. In host code
// the array's name is only a stand-in for the symbol, never a device address; kernels and copies get
// the kept pointer.
static __device__ __align__(256) float scratch[IMPARO_STATIC_SCRATCH_BYTES / sizeof(float)];

static constexpr int SCRATCH_DEVICES = 64;
static std::mutex scratch_mutex;
static std::atomic<float*> scratch_of_device[SCRATCH_DEVICES];

static int static_scratch(float** ptr) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SCRATCH_DEVICES) return IMPARO_LAUNCH_FAILED;
    float* p = scratch_of_device[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> hold(scratch_mutex);
        p = scratch_of_device[dev].load(std::memory_order_acquire);
        if (!p) {
            void* address = nullptr;
            if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess || !address) {
                (void)hipGetLastError();
                return IMPARO_LAUNCH_FAILED;
            }
            p = static_cast<float*>(address);
            scratch_of_device[dev].store(p, std::memory_order_release);
        }
    }
    *ptr = p;
    return IMPARO_OK;
}

extern "C" int imparo_attention_decode_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                              const int32_t* rows, int n_rows,
                                              const int32_t* seg_start, const int32_t* positions,
                                              const int32_t* block_table, int table_stride, int page_size,
                                              int heads, int kv_heads, int head_dim, int n_pages, float scale,
                                              int window, int n_splits, imparo_stream stream) {
    const int bad = check_common(q, k_cache, v_cache, out, rows, seg_start, positions, block_table, table_stride,
                                 page_size, heads, kv_heads, head_dim, n_pages, window);
    if (bad) return bad;
    if (n_rows < 0 || n_splits <= 0 || n_splits > 65535) return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0) return IMPARO_OK;
    if (n_rows > 65535) return IMPARO_BAD_ARGUMENT;
    // [rows, heads, splits, head_dim] partial outputs, then, at the next multiple of 64 floats,
    // [rows, heads, splits, 2] maxima and sums
    const unsigned long long slots = (unsigned long long)n_rows * heads * n_splits;
    const unsigned long long o_floats = (slots * head_dim + 63) / 64 * 64;
    if ((o_floats + slots * 2) * sizeof(float) > IMPARO_STATIC_SCRATCH_BYTES) {
        fprintf(stderr, "imparo_attention_decode_static: %d rows x %d heads x %d splits of head size %d need %llu bytes "
                        "for partial results, the library's own buffer holds %llu; use imparo_attention_decode with a "
                        "workspace, or fewer rows a call\n", n_rows, heads, n_splits, head_dim,
                (o_floats + slots * 2) * (unsigned long long)sizeof(float), (unsigned long long)IMPARO_STATIC_SCRATCH_BYTES);
        return IMPARO_SCRATCH_TOO_SMALL;
    }
    float* base = nullptr;
    const int st = static_scratch(&base);
    if (st) return st;
    // nothing here has to start at zero: the merge reads a (row, head, split) only if this call's
    // first kernel wrote it
    return attention_decode_launch(q, k_cache, v_cache, out, base, base + o_floats, rows, n_rows, seg_start, positions,
                                   block_table, table_stride, page_size, heads, kv_heads, head_dim, n_pages, scale,
                                   window, n_splits, (hipStream_t)stream);
}

// How the prompt kernel for head sizes in steps of 32 lays a launch out: heads of a kv head to a block,
// 16 or 32 queries a wave, queries of a head per block.
struct PrefillShape {
    int hpb, qt;
    bool wide;
    long long blocks;
};
static PrefillShape prefill_shape(int n_tiles, int heads, int kv_heads, long long context_bound) {
    PrefillShape p;
    // four heads of a kv head to a block where the group allows it, else more runs of queries
    const int group = heads / kv_heads;
    p.hpb = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
    // 32 queries a wave where that still leaves twice as many waves as SIMDs (n_tiles x 64 queries x heads at most)
    // and the contexts are long: measured with 32 heads of 64 and 2,048 queries, 16 a wave are 9% faster
    // on a fresh prompt, as fast at 4,096 keys and 5 to 9% slower from 16k on
    p.wide = (long long)n_tiles * 2 * heads >= 2048 && context_bound >= 8192;
    // n_tiles counts tiles of 64 queries per row: a row has at most that many blocks of 64 queries or more,
    // and 64 / qt times as many of fewer (blocks past a row's last find no tile and leave)
    p.qt = (p.wide ? 32 : 16) * (MFMA_WAVES / p.hpb);
    p.blocks = (long long)n_tiles * (p.qt < 64 ? 64 / p.qt : 1) * (heads / p.hpb);
    return p;
}

// Into how many parts the keys of a launch of prompt portions are cut (1: none). Few queries over a
// long context leave the chip idle (512 queries of 16 heads are 128 blocks, each walking all the keys:
// 474 us over 30,000 keys, 144 us in 8 parts): up to 8 parts, towards four blocks per CU, at least
// 1,024 keys of the longest context each; the caller brings room for the parts' results
// ([tokens, heads, parts, head size] and [.., 2] floats).
extern "C" int imparo_attention_prefill_splits(int n_tiles, int heads, int kv_heads, int head_dim, int max_context) {
    if (n_tiles <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || head_dim % 32 != 0) return 1;
    const PrefillShape p = prefill_shape(n_tiles, heads, kv_heads, max_context);
    // Blocks of 32 queries a wave over long contexts: three of them fit a CU (registers), and a wave there
    // waits for its tiles a third of the time, so the chip wants two full rounds of them, 1,536 blocks.
    // Measured with 2,048 queries of 32 heads (512 blocks) in 3 parts: as fast at 8k keys, 6 % faster at
    // 16k, 9 to 10 % from 24k on; 4,096 queries (1,024 blocks) in 2 parts 7 % faster at 32k.
    if (p.wide && max_context >= 12288) {
        if (p.blocks >= 1536) return 1;
        return (int)std::max<long long>(
            1, std::min<long long>({8, (1536 + p.blocks - 1) / p.blocks, (long long)max_context / 4096}));
    }
    const long long blocks = p.blocks * (p.wide ? 2 : 1);       // a block of 32 queries a wave counts as two
    if (blocks >= 1024 || max_context < 2048) return 1;
    return (int)std::max<long long>(1, std::min<long long>({8, 1024 / blocks, max_context / 1024}));
}

extern "C" int imparo_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                        float* part_o, float* part_ml, int n_splits,
                                        const int32_t* rows, int n_rows, int n_tiles,
                                        const int32_t* seg_start, const int32_t* seg_len, const int32_t* positions,
                                        const int32_t* block_table, int table_stride, int page_size,
                                        int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                        imparo_stream stream) {
    const int bad = check_common(q, k_cache, v_cache, out, rows, seg_start, positions, block_table, table_stride,
                                 page_size, heads, kv_heads, head_dim, n_pages, window);
    if (bad) return bad;
    if (!seg_len || n_rows < 0 || n_tiles < 0 || heads > 65535) return IMPARO_BAD_ARGUMENT;
    if (n_splits < 1 || n_splits > 64 || (n_splits > 1 && (!part_o || !part_ml || head_dim % 32 != 0)))
        return IMPARO_BAD_ARGUMENT;
    // the merge moves four elements of a head in one access
    if (n_splits > 1 && (((uintptr_t)part_o & 15) || ((uintptr_t)part_ml & 7) || ((uintptr_t)out & 7)))
        return IMPARO_BAD_ARGUMENT;
    if (n_rows == 0 || n_tiles == 0) return IMPARO_OK;
    hipStream_t s = (hipStream_t)stream;
    if (head_dim % 32 == 0) {
        const PrefillShape p = prefill_shape(n_tiles, heads, kv_heads, (long long)table_stride * page_size);
        const int hpb = p.hpb;
        const bool wide = p.wide;
        dim3 grid32((unsigned)(n_tiles * (p.qt < 64 ? 64 / p.qt : 1)), heads / hpb, n_splits);
#define PREFILL_X32_GO(ND, HALVES, PAGE_TILE)                                                                       \
    k_attn_prefill_x32<ND, HALVES, PAGE_TILE><<<grid32, MFMA_WAVES * 64, 0, s>>>(                                    \
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, rows, n_rows, seg_start,     \
        seg_len, positions, block_table, table_stride, page_size, heads, kv_heads, n_pages, scale, window, hpb,      \
        part_o, part_ml)
#define PREFILL_X32(ND)                                                                                              \
    if (wide && page_size >= PX_KEYS) PREFILL_X32_GO(ND, 2, true);                                                   \
    else if (wide) PREFILL_X32_GO(ND, 2, false);                                                                     \
    else if (page_size >= PX_KEYS) PREFILL_X32_GO(ND, 1, true);                                                      \
    else PREFILL_X32_GO(ND, 1, false)
        switch (head_dim / 32) {
            case 1: PREFILL_X32(2); break;
            case 2: PREFILL_X32(4); break;
            case 3: PREFILL_X32(6); break;
            default: PREFILL_X32(8);
        }
#undef PREFILL_X32
#undef PREFILL_X32_GO
        if (launch_status()) return IMPARO_LAUNCH_FAILED;
        if (n_splits == 1) return IMPARO_OK;
        // a block of four waves per token, each wave as many heads as its lanes hold; tokens past the portions'
        // last find none and leave
        const int heads_a_block = 4 * (64 / (head_dim / 4));
        dim3 merge_grid((unsigned)n_tiles * 64, (unsigned)((heads + heads_a_block - 1) / heads_a_block));
#define MERGE(GROUP)                                                                                              \
    k_attn_prefill_merge<GROUP><<<merge_grid, 256, 0, s>>>(part_o, part_ml, (bf16_t*)out, rows, n_rows, seg_start, \
                                                           seg_len, heads, head_dim, n_splits, scale)
        if (n_splits <= 2) MERGE(2);
        else if (n_splits <= 4) MERGE(4);
        else MERGE(8);
#undef MERGE
        return launch_status();
    }
    dim3 grid(n_tiles, heads);
    DISPATCH_ND(head_dim / 16, (k_attn_prefill<ND><<<grid, MFMA_WAVES * 64, 0, s>>>(
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, rows, n_rows, seg_start,
        seg_len, positions, block_table, table_stride, page_size, heads, kv_heads, n_pages, scale, window)));
    return launch_status();
}

// Asks the runtime about one kernel of this file, which makes it load the file's code onto the
// current device (it loads a file's kernels when one of them is first used; a stream under capture
// cannot do that).
int imparo_load_code_attention_mfma() {
    hipFuncAttributes attributes;
    return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&k_attn_decode_merge)) == hipSuccess ? IMPARO_OK
                                                                                              : IMPARO_LAUNCH_FAILED;
}
