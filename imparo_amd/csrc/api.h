// C entry points of the gfx950 kernel library. Every pointer is device memory
// unless named host_*. Every entry validates its sizes, launches on `stream`
// and returns IMPARO_OK (0), IMPARO_BAD_ARGUMENT (1, nothing launched) or
// IMPARO_LAUNCH_FAILED (2). dtype codes: 0 = float32, 1 = bfloat16.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* imparo_stream;

// The hash of the sources this library was built from, as the build computed it.
const char* imparo_hip_source_hash();

// Loads the code of every kernel file onto the current device. The runtime would load each file's
// code when one of its kernels is first launched, which a stream under graph capture cannot do: call
// this once per device before the first capture.
int imparo_load_code(void);

// x[t, :] = table[ids[t], :] as float32.
int imparo_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* x,
                        int n_tokens, int width, int vocab, imparo_stream stream);

// ids[dst[i]] = src[src_index[i]] for i < n, clamped into [0, vocab): token ids sampled by the
// step before that are still on the device. The caller guarantees dst[i] < len(ids) and
// src_index[i] < len(src).
int imparo_place_tokens(int32_t* ids, const int32_t* dst, const int32_t* src, const int32_t* src_index,
                        int n, int vocab, imparo_stream stream);

// Row-wise RMS norm. For output row i the source row is rows ? rows[i] : i.
// If delta is given the row is x + delta[0] + delta[1] + ... first (n_delta
// slices, each [n_x_rows, width], added in order); with write_back (rows must
// be null) the sum is stored to x. out[i, :] = v * rsqrt(mean(v^2) + eps) * weight.
int imparo_rms_norm(float* x, const float* delta, int n_delta, int n_x_rows, const int32_t* rows, const float* weight,
                    void* out, int out_dtype, int n_rows, int width, float eps, int write_back,
                    imparo_stream stream);

// Y[m, n] = X[m, k] . W[n, k]^T (+ bias[n], float32, may be null), float32
// accumulate. X and W share `dtype`. epilogue 0: Y is [m, n]. epilogue 1
// (SwiGLU): W's rows alternate gate, up; Y is [m, n/2] with
// Y[m, j] = silu(y[m, 2j]) * y[m, 2j+1].
// `slices` > 1 (only the number imparo_gemm_slices gives, float32 out, epilogue 0): K is cut into
// that many slices and Y is [slices, m, n], slice s holding the sum over its part of K (the bias
// in slice 0); the consumer adds the slices in order.
int imparo_gemm(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                int m, int n, int k, int epilogue, int slices, imparo_stream stream);
int imparo_gemm_slices(int m, int n, int k, int dtype);
// epilogue 2 (float32 out, `slices` 1): Y[m, n] += the product (+ bias), each element of Y read where it
// is stored. Only for shapes for which imparo_gemm_adds gives 1 (many rows, a K the tile kernel takes).
int imparo_gemm_adds(int m, int n, int k, int dtype);
// imparo_gemm with the kernel named by the caller instead of chosen by the library: for tests and
// measurements, so that every kernel can be met at any shape (the numbers are listed in gemm.hip).
// Nothing in the library keeps the choice: it is this call's argument.
int imparo_gemm_variant(const void* x, const void* w, const float* bias, void* y, int dtype, int out_dtype,
                        int m, int n, int k, int epilogue, int slices, int variant, imparo_stream stream);

// Per (token, head): RMS norm over the head (weight null: none), NeoX rotation
// with angles pos * inv_freq[i] over the first 2*n_freq dims (n_freq 0: none): pair i is dims
// (i, i + n_freq), or with `interleaved` dims (2i, 2i + 1).
// qkv is float32 [n_tokens, (heads + 2*kv_heads) * head_dim]; q goes to q_out
// [n_tokens, heads, head_dim], k and v into the paged cache at each token's
// position: page = table[row_of_token[t] * table_stride + pos / page_size].
// Cache layout [n_pages, kv_heads, page_size, head_dim]; with v_transposed the V
// cache is [n_pages, kv_heads, head_dim, page_size]. write_kv 0 skips the cache.
int imparo_qk_norm_rope_store(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                              const float* inv_freq, int n_freq, int interleaved,
                              const int32_t* positions, const int32_t* row_of_token,
                              const int32_t* block_table, int table_stride, int page_size,
                              void* q_out, void* k_cache, void* v_cache, int dtype, int write_kv,
                              int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                              int v_transposed, imparo_stream stream);

// Causal grouped-query attention over the paged cache; one query per (token,
// head); keys lo..pos with lo = max(0, pos + 1 - window) (window 0: all keys).
int imparo_attention(const void* q, const void* k_cache, const void* v_cache, void* out, int dtype,
                     const int32_t* positions, const int32_t* row_of_token,
                     const int32_t* block_table, int table_stride, int page_size,
                     int n_tokens, int heads, int kv_heads, int head_dim, int n_pages,
                     float scale, int window, int v_transposed, imparo_stream stream);

// Matrix-core attention, bfloat16, V cache transposed, page_size a power of two
// >= 16, head_dim a multiple of 16 up to 128.
// Decode: one query token per listed row (rows[i] indexes seg_start); the key
// range is split in pieces of 256 keys whose partial results go through
// part_o [n_rows, heads, n_splits, head_dim] and part_ml [n_rows, heads,
// n_splits, 2]; n_splits >= ceil(longest context / 256).
int imparo_attention_decode_split(void);      // keys per split
int imparo_attention_prefill_tile(void);      // queries per tile that n_tiles counts
int imparo_attention_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                            float* part_o, float* part_ml, const int32_t* rows, int n_rows,
                            const int32_t* seg_start, const int32_t* positions,
                            const int32_t* block_table, int table_stride, int page_size,
                            int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                            int n_splits, imparo_stream stream);

// The same for a step whose rows' keys and values are not in the cache yet: qkv is the fused
// projection's float32 rows [tokens, (heads + 2 kv_heads) x head_dim] (q heads, k heads, v heads). The
// launch norms each head of q and k (weights [head_dim], or both null: no norm), rotates them
// (inv_freq [n_freq] with 2 n_freq = head_dim, pairs (i, i + n_freq) or with `interleaved`
// (2i, 2i + 1); n_freq 0: no rotation), attends over the cached keys before each row's position and
// the new key, and with write_kv puts the new key and value into their page (V pages transposed).
// It replaces imparo_qk_norm_rope_store + imparo_attention_decode for such a step, in one launch less.
// Head sizes 64 and 128 (imparo_attention_decode_qkv_takes); a layer that reads another layer's cache
// finds the row's key there already and takes the two-launch form.
int imparo_attention_decode_qkv_takes(int head_dim, int n_freq);
int imparo_attention_decode_qkv_pays(int n_rows, int n_splits);   // few rows over not too many splits: the one launch is the faster way
int imparo_attention_decode_qkv(const float* qkv, const float* q_weight, const float* k_weight, float eps,
                                const float* inv_freq, int n_freq, int interleaved, void* k_cache, void* v_cache,
                                int write_kv, void* out, float* part_o, float* part_ml, const int32_t* rows,
                                int n_rows, const int32_t* seg_start, const int32_t* positions,
                                const int32_t* block_table, int table_stride, int page_size, int heads,
                                int kv_heads, int head_dim, int n_pages, float scale, int window, int n_splits,
                                imparo_stream stream);

// imparo_attention_decode for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the
// reference. The splits' partial results go through a buffer of IMPARO_STATIC_SCRATCH_BYTES that the
// library holds itself on every GPU it runs on (until the process ends) instead of part_o / part_ml;
// the call allocates and frees nothing. rows x heads x n_splits x (head_dim + 2) floats (the first
// part rounded up to 64 floats) must fit, else nothing is launched, a line on stderr says what was
// asked for, and IMPARO_SCRATCH_TOO_SMALL (3) is returned. All calls on one GPU share that GPU's
// buffer: calls that overlap there (two streams, two threads) race; calls on one stream do not.
// The buffer keeps the last call's contents; no call relies on them. The first call on a device
// looks the buffer's address up (no allocation, but not a stream operation: make it outside a capture).
#define IMPARO_STATIC_SCRATCH_BYTES (16u << 20)
int imparo_attention_decode_static(const void* q, const void* k_cache, const void* v_cache, void* out,
                                   const int32_t* rows, int n_rows,
                                   const int32_t* seg_start, const int32_t* positions,
                                   const int32_t* block_table, int table_stride, int page_size,
                                   int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                                   int n_splits, imparo_stream stream);

// Prompt portions: the listed rows' segments in tiles of 64 queries;
// n_tiles = sum over the rows of ceil(seg_len / 64). n_splits (from
// imparo_attention_prefill_splits, or 1) parts of each block's keys, merged by a
// second launch; then part_o holds [tokens, heads, n_splits, head_dim] floats
// and part_ml [tokens, heads, n_splits, 2], tokens counted over the whole batch.
// `max_context` is the bound on the contexts that imparo_attention_prefill itself goes by: what its
// block table can hold, table_stride x page_size (both lay a launch out from that one number).
int imparo_attention_prefill_splits(int n_tiles, int heads, int kv_heads, int head_dim, int max_context);
int imparo_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                             float* part_o, float* part_ml, int n_splits,
                             const int32_t* rows, int n_rows, int n_tiles,
                             const int32_t* seg_start, const int32_t* seg_len, const int32_t* positions,
                             const int32_t* block_table, int table_stride, int page_size,
                             int heads, int kv_heads, int head_dim, int n_pages, float scale, int window,
                             imparo_stream stream);

// Gated short convolution over each request's segment, continuing from its
// state slot. bcx float32 [n_tokens, 3*width] = [B | C | x]. state float32
// [n_slots, taps-1, width], oldest first. seg_start[r], seg_len[r], slot[r]
// describe request r's tokens in the batch. out[t] = C_t * (sum_k w[ch,k] *
// seq[t+k] + bias[ch]).
int imparo_short_conv(const float* bcx, const float* weight, const float* bias, const float* state,
                      const int32_t* row_of_token, const int32_t* seg_start, const int32_t* slot,
                      void* out, int out_dtype, int n_tokens, int width, int taps, int n_slots, int n_rows,
                      imparo_stream stream);

// The same for a batch in which every request brings exactly one token, output
// and state update in one launch: n_tokens == n_rows, token r belongs to row r.
int imparo_short_conv_decode(const float* bcx, const float* weight, const float* bias, float* state,
                             const int32_t* slot, void* out, int out_dtype, int n_rows, int width, int taps,
                             int n_slots, imparo_stream stream);

// The conv mixer's input projection and imparo_short_conv_decode in one launch, for at most 16
// single-token rows: x [m, k] and w [3 e, k] bfloat16, in_bias [3 e] or null, conv_w [e, taps],
// conv_b [e] or null, slot [m] (distinct). out [m, e]; the state is shifted in place.
int imparo_in_proj_conv_decode(const void* x, const void* w, const float* in_bias, const float* conv_w,
                               const float* conv_b, float* state, const int32_t* slot, void* out, int out_dtype,
                               int m, int e, int k, int taps, int n_slots, imparo_stream stream);

// The same on activations that are the residual stream times a norm's weight, each row still to be
// scaled: ssq_in [n_parts, 16] holds the partial sums of squares of the stream's rows and the launch
// multiplies B, C and x of row r by rsqrt(sum_p ssq_in[p][r] / k + eps). ssq_in null: as above.
int imparo_in_proj_conv_decode_normed(const void* x, const float* ssq_in, int n_parts, float eps, const void* w,
                                      const float* in_bias, const float* conv_w, const float* conv_b, float* state,
                                      const int32_t* slot, void* out, int out_dtype, int m, int e, int k, int taps,
                                      int n_slots, imparo_stream stream);

// Products for a step of at most 16 rows with a norm of the residual stream folded into them
// (decode_rows.hip). x [m, k] and w [n, k] bfloat16, k a multiple of 8, bias float32 [n] or null.
// With ssq_in [n_parts, 16] and eps, x is the stream times a norm's weight, each row still to be
// scaled, and row r's result is multiplied by rsqrt(sum_p ssq_in[p][r] / k + eps) at the end, in float32.
// epilogue 0: y [m, n] in out_dtype; 1: SwiGLU, y [m, n/2] (rows of w alternate gate, up);
// 2: x_io [m, n] float32 += the result, in place, and ssq_out [imparo_rows_parts(n), 16] receives the
// partial sums of squares of the new rows (entries of rows >= m are zero); with weighted_by [n] (the
// weight of the norm that reads the stream next), weighted_out [m, n] bfloat16 receives the new rows
// times it. A block sums the whole of K, in an order that depends on k alone.
int imparo_rows_parts(int n);
int imparo_rows_gemm(const void* x, const float* ssq_in, int n_parts, float eps, const void* w, const float* bias,
                     void* y, int out_dtype, float* x_io, float* ssq_out, void* weighted_out, const float* weighted_by,
                     int m, int n, int k, int epilogue, imparo_stream stream);

// state' = the last taps-1 rows of (state ++ B*x) for every request; runs after
// imparo_short_conv on the same stream.
int imparo_short_conv_state(const float* bcx, float* state, const int32_t* seg_start, const int32_t* seg_len,
                            const int32_t* slot, int n_rows, int n_tokens, int width, int taps, int n_slots,
                            imparo_stream stream);

// out[r] = smallest index of the maximum of logits[r, :]; NaN never wins.
int imparo_argmax_rows(const float* logits, int32_t* out, int n_rows, int vocab, imparo_stream stream);

// out[r] = the first index whose cumulative softmax(logits[r]/temperature[r])
// reaches uniform[r]; temperature <= 0 is argmax.
int imparo_sample_rows(const float* logits, const float* temperature, const float* uniform, int32_t* out,
                       int n_rows, int vocab, imparo_stream stream);

// Fills n float32 values (or n int32 values of the same bits) without a memset node.
int imparo_fill_f32(float* p, float value, int64_t n, imparo_stream stream);

// The fixed-size state of one slot, every site in one launch: for site i, per_slot[i] float32
// values at base[i] (a device address) + slot * per_slot[i] are set to value[i]. base, per_slot
// and value are device arrays of n_sites entries that the caller built from tensors it owns.
int imparo_fill_sites(const uint64_t* base, const int64_t* per_slot, const float* value, int n_sites, int slot,
                      imparo_stream stream);

// ---------------------------------------------------------------------------------------------
// A model's step as one call. A program is the model's run order as a list of operations over a
// float32 residual stream: the embedding, then per layer a norm, a mixer, a norm and a
// feed-forward, then the norm and head of the wanted rows. Each operation launches the kernels
// above, chosen by the batch's shape exactly as a caller of the single entry points would choose
// them; what the program saves is the caller's time between launches. The reference issues a
// step's kernels from one native routine as well
// (/root/reference/crates/imparo-model/src/lfm2/workflow_gpu.rs:317-1633).
//
// Scratch lives in regions that the caller binds: the program names them (imparo_program_region_*),
// says how many bytes of each a step needs (imparo_program_needs) and refuses to run with
// IMPARO_SCRATCH_TOO_SMALL, before any launch, when a bound region is too small for the step.
// Nothing here allocates device memory.
typedef struct ImparoProgram ImparoProgram;

// A projection Y = X . W^T (+ bias): W is [n, k] in `dtype`, bias float32 [n] or null.
typedef struct {
    const void* weight;
    const float* bias;
    int32_t dtype, n, k;
} ImparoLinearDesc;

typedef struct {
    ImparoLinearDesc qkv, out;           // fused q | k | v projection, output projection
    const float* q_norm;                 // per-head RMS norm weights [head_dim], both null: no norm
    const float* k_norm;
    float norm_eps;
    const float* inv_freq;               // [n_freq] or null
    int32_t n_freq, interleaved;
    int32_t heads, kv_heads, head_dim;
    float scale;
    int32_t window;                      // 0: every key
    void* k_cache;                       // this call's cache site
    void* v_cache;
    int32_t n_pages, v_transposed, group; // group: which of the step's block tables
    int32_t owns_cache;                  // 0: reads a cache that an earlier call of the step has written
} ImparoAttentionDesc;

typedef struct {
    ImparoLinearDesc in_proj, out_proj;
    const float* conv_weight;            // [width, taps]
    const float* conv_bias;              // [width] or null
    int32_t width, taps;
    float* state;                        // [n_slots, taps - 1, width]
    int32_t n_slots;
} ImparoShortConvDesc;

typedef struct {
    ImparoLinearDesc gate_up, down;      // gate and up rows alternate in gate_up
} ImparoSwigluDesc;

// One batch: device arrays as imparo_cache_pack lays them out (any placement), and the sizes the
// host knows. tables[g] is [n_rows, table_width] for cache group g.
#define IMPARO_MAX_GROUPS 8
typedef struct {
    const int32_t* tokens;               // [n_tokens]
    const int32_t* positions;            // [n_tokens]
    const int32_t* row_of_token;         // [n_tokens]
    const int32_t* seg_start;            // [n_rows]
    const int32_t* seg_len;              // [n_rows]
    const int32_t* slot;                 // [n_rows]
    const int32_t* single_rows;          // [n_single]: rows that bring one token
    const int32_t* portion_rows;         // [n_portion]: rows that bring more
    const int32_t* want_rows;            // [n_want]: places in the packed batch whose logits are wanted
    const int32_t* tables[IMPARO_MAX_GROUPS];
    int32_t n_groups, table_width;
    int32_t n_tokens, n_rows, n_want, n_single, n_portion;
    int32_t max_seg_len, max_context;    // longest segment; longest context after the step (a bound will do)
    int32_t portion_tiles;               // sum over the portion rows of ceil(tokens / imparo_attention_prefill_tile())
} ImparoStepArgs;

ImparoProgram* imparo_program_new(int engine_dtype, int page_size);
void imparo_program_delete(ImparoProgram* p);
// In a step of at most 16 single tokens a norm of the stream can be folded into the products around
// it (decode_rows.hip): mode 0 never, 1 where imparo_rows_fold_pays says so (the default), 2 wherever
// the operations allow. Folding changes results by rounding only.
int imparo_program_set_fold(ImparoProgram* p, int mode);
int imparo_rows_fold_pays(int m, int n, int k);
// Operations, in run order. Each returns IMPARO_OK or IMPARO_BAD_ARGUMENT (sizes that do not fit).
int imparo_program_embedding(ImparoProgram* p, const void* table, int table_dtype, int vocab, int width);
// h = norm(stream + what the last mixer or feed-forward left pending), in out_dtype; the sum goes back to the stream
int imparo_program_norm(ImparoProgram* p, const float* weight, float eps, int width, int out_dtype);
int imparo_program_attention(ImparoProgram* p, const ImparoAttentionDesc* d);
int imparo_program_short_conv(ImparoProgram* p, const ImparoShortConvDesc* d);
int imparo_program_swiglu(ImparoProgram* p, const ImparoSwigluDesc* d);
// logits = head(norm(stream + pending) at the wanted rows); the stream is left as it is
int imparo_program_head(ImparoProgram* p, const float* norm_weight, float eps, int width, const ImparoLinearDesc* head);

int imparo_program_n_regions(const ImparoProgram* p);
const char* imparo_program_region_name(const ImparoProgram* p, int region);
int imparo_program_bind(ImparoProgram* p, int region, void* ptr, int64_t bytes);
// needs[region] = bytes of each region that a step of this shape uses (0: not used)
int imparo_program_needs(ImparoProgram* p, const ImparoStepArgs* args, int64_t* needs);
// Runs the step on `stream`. *logits = where the float32 [n_want, vocab] logits are (inside the
// "logits" region), or null if nothing is wanted. IMPARO_SCRATCH_TOO_SMALL: nothing was launched,
// imparo_program_needs says what to bind. Any other failure: imparo_program_error names the operation.
int imparo_program_run(ImparoProgram* p, const ImparoStepArgs* args, float** logits, imparo_stream stream);
const char* imparo_program_error(const ImparoProgram* p);

#ifdef __cplusplus
}
#endif
