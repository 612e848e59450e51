// A model's step issued by one native call: the run order as a list of operations, each of which
// launches the kernels of this library chosen by the batch's shape. Host code only; the kernels are
// reached through the library's own C entry points, so a step issued from here and a step issued
// launch by launch by a caller of those entry points run the same kernels with the same arguments.
//
// The list mirrors the pre-norm arrangement of parts: a float32 residual stream x, a delta that the
// last mixer or feed-forward left pending on it (possibly in slices of K, added in order by the next
// norm), and the normed rows h that the next part reads
// (/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:8-15 for the arrangement,
// /root/reference/crates/imparo-model/src/lfm2/workflow_gpu.rs:317-1633 for a step issued natively).
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

#include "api.h"
#include "common.h"

namespace {

struct Region {
    std::string name;
    char* ptr = nullptr;
    int64_t bytes = 0;
};

enum OpKind { OP_EMBEDDING, OP_NORM, OP_ATTENTION, OP_SHORT_CONV, OP_SWIGLU, OP_HEAD };

struct Op {
    OpKind kind;
    // embedding
    const void* table = nullptr;
    int table_dtype = 0, vocab = 0, width = 0;
    // norm (and the head's norm)
    const float* weight = nullptr;
    float eps = 0.f;
    int out_dtype = 0;
    ImparoAttentionDesc attention{};
    ImparoShortConvDesc conv{};
    ImparoSwigluDesc swiglu{};
    ImparoLinearDesc head{};
};

inline int64_t element_size(int dtype) { return dtype == IMPARO_F32 ? 4 : 2; }

}  // namespace

struct ImparoProgram {
    int engine_dtype = IMPARO_BF16, page_size = 0;
    int fold = 1;        // norms folded into the products around them: 0 never, 1 where it pays, 2 wherever possible
    std::vector<Region> regions;
    std::vector<Op> ops;
    std::string error;
    // regions by role
    int r_residual, r_normed, r_mixer_in, r_mixer_mid, r_q, r_mixer_out, r_mixer_out_sliced, r_ffn_out, r_ffn_out_sliced,
        r_part_o, r_part_ml, r_prefill_part_o, r_prefill_part_ml, r_normed_rows, r_logits, r_fold_ssq, r_fold_weighted;

    int region(const char* name) {
        regions.push_back(Region{name});
        return (int)regions.size() - 1;
    }
};

namespace {

// One walk over the operations. A dry walk launches nothing and notes what each region must hold;
// the real walk hands out the bound memory. Both take every decision from the same code.
struct Walk {
    ImparoProgram* p;
    const ImparoStepArgs* a;
    imparo_stream stream;
    bool dry;
    std::vector<int64_t> need;
    int status = IMPARO_OK;
    int op_index = 0;
    // the residual stream, what is pending on it, the rows the next part reads
    float* x = nullptr;
    const float* pending = nullptr;
    int n_pending = 0;
    void* h = nullptr;
    int h_dtype = IMPARO_F32;
    float* logits = nullptr;
    // A step of at most 16 single tokens may fold a norm into the products around it (decode_rows.hip):
    // the product that feeds the stream adds its result there itself and leaves the new rows' partial
    // sums of squares and the rows times the next norm's weight (f_*: waiting for that norm); the norm
    // then launches nothing and hands those rows on as h, each still to be scaled (h_ssq, h_parts,
    // h_eps), which the product behind it does at its end.
    const float* f_ssq = nullptr;
    const void* f_weighted = nullptr;
    int f_parts = 0;
    const float* h_ssq = nullptr;
    int h_parts = 0;
    float h_eps = 0.f;

    Walk(ImparoProgram* p, const ImparoStepArgs* a, imparo_stream s, bool dry)
        : p(p), a(a), stream(s), dry(dry), need(p->regions.size(), 0) {}

    void* get(int region, int64_t bytes) {
        if (bytes < 1) bytes = 1;
        if (bytes > need[region]) need[region] = bytes;
        if (dry) return (void*)(uintptr_t)256;          // never read: a dry walk launches nothing
        return p->regions[region].ptr;
    }

    void fail(int code, const char* what) {
        if (status != IMPARO_OK) return;
        status = code;
        char buf[256];
        snprintf(buf, sizeof buf, "operation %d: %s %s", op_index, what,
                 code == IMPARO_BAD_ARGUMENT ? "refused its arguments" : "failed to launch");
        p->error = buf;
    }

    // runs a launch unless the walk is dry or has failed
    template <typename F>
    void launch(const char* what, F&& f) {
        if (dry || status != IMPARO_OK) return;
        const int rc = f();
        if (rc != IMPARO_OK) fail(rc, what);
    }

    struct Out {
        void* ptr;
        int slices;      // > 0: [slices, m, width] (1: plain); 0: added into the stream
    };

    // A projection of m rows, as a part's Linear runs it: in slices of K where the consumer adds
    // slices and the library says that pays, added into `into` where the library's epilogue can,
    // else plain into `region`.
    Out linear(const ImparoLinearDesc& lin, const void* in, int in_dtype, int m, int out_dtype, int region,
               int sliced_region, bool swiglu, bool sliced_ok, float* into) {
        if (in_dtype != lin.dtype) {
            fail(IMPARO_BAD_ARGUMENT, "a projection whose input is not in its weight's dtype");
            return Out{nullptr, 1};
        }
        const int width = swiglu ? lin.n / 2 : lin.n;
        if (sliced_ok && !swiglu && out_dtype == IMPARO_F32) {
            const int slices = imparo_gemm_slices(m, lin.n, lin.k, lin.dtype);
            if (slices > 1) {
                void* out = get(sliced_region, (int64_t)slices * m * width * 4);
                launch("imparo_gemm (slices of K)", [&] {
                    return imparo_gemm(in, lin.weight, lin.bias, out, lin.dtype, IMPARO_F32, m, lin.n, lin.k, 0, slices, stream);
                });
                return Out{out, slices};
            }
        }
        if (into && !swiglu && out_dtype == IMPARO_F32 && imparo_gemm_adds(m, lin.n, lin.k, lin.dtype)) {
            launch("imparo_gemm (added to the stream)", [&] {
                return imparo_gemm(in, lin.weight, lin.bias, into, lin.dtype, IMPARO_F32, m, lin.n, lin.k, 2, 1, stream);
            });
            return Out{into, 0};
        }
        void* out = get(region, (int64_t)m * width * element_size(out_dtype));
        launch("imparo_gemm", [&] {
            return imparo_gemm(in, lin.weight, lin.bias, out, lin.dtype, out_dtype, m, lin.n, lin.k, swiglu ? 1 : 0, 1, stream);
        });
        return Out{out, 1};
    }

    // what a mixer or feed-forward returned becomes the pending delta (or went into the stream already)
    void leave(const Out& out) {
        if (out.slices == 0) {
            pending = nullptr;
            n_pending = 0;
        } else {
            pending = (const float*)out.ptr;
            n_pending = out.slices;
        }
    }

    float* stream_if_nothing_pending() const { return pending ? nullptr : x; }

    // whether the operation can read rows that are still to be scaled (the stream times its norm's weight)
    bool takes_unscaled(const Op& op) const {
        auto fits = [](const ImparoLinearDesc& l) { return l.dtype == IMPARO_BF16 && l.k % 8 == 0; };
        switch (op.kind) {
            case OP_ATTENTION: return fits(op.attention.qkv);
            case OP_SWIGLU: return fits(op.swiglu.gate_up);
            case OP_SHORT_CONV: return fits(op.conv.in_proj) && op.conv.in_proj.n % 24 == 0;     // its one-launch form
            default: return false;
        }
    }

    // A product whose result goes into the stream (a mixer's output projection, a feed-forward's way
    // back). In a step of at most 16 single tokens, where the next operation is a norm and the one
    // behind it can scale its rows itself, the product adds its result to the stream and leaves what
    // folds that norm away; else it runs as a part's Linear runs it and leaves a delta pending.
    void produce(const ImparoLinearDesc& lin, const void* in, int in_dtype, int region, int sliced_region) {
        const int T = a->n_tokens;
        float* into = stream_if_nothing_pending();
        const size_t next = (size_t)op_index + 1;
        if (p->fold && into && p->engine_dtype == IMPARO_BF16 && T <= 16 && a->max_seg_len == 1 && lin.dtype == IMPARO_BF16 &&
            in_dtype == IMPARO_BF16 && lin.k % 8 == 0 && next + 1 < p->ops.size() && p->ops[next].kind == OP_NORM &&
            p->ops[next].out_dtype == IMPARO_BF16 && p->ops[next].width == lin.n && takes_unscaled(p->ops[next + 1]) &&
            (p->fold == 2 || imparo_rows_fold_pays(T, lin.n, lin.k))) {
            const int parts = imparo_rows_parts(lin.n);
            float* ssq = (float*)get(p->r_fold_ssq, (int64_t)parts * 16 * 4);
            void* weighted = get(p->r_fold_weighted, (int64_t)T * lin.n * 2);
            const float* by = p->ops[next].weight;
            launch("imparo_rows_gemm (added to the stream)", [&] {
                return imparo_rows_gemm(in, nullptr, 0, 0.f, lin.weight, lin.bias, nullptr, IMPARO_F32, into, ssq, weighted, by,
                                        T, lin.n, lin.k, 2, stream);
            });
            pending = nullptr;
            n_pending = 0;
            f_ssq = ssq;
            f_parts = parts;
            f_weighted = weighted;
            return;
        }
        leave(linear(lin, in, in_dtype, T, IMPARO_F32, region, sliced_region, false, true, into));
    }

    // A product that reads the normed rows h (a mixer's input projection, gate and up). Rows that are
    // still to be scaled go to the kernels that scale at their end.
    Out consume(const ImparoLinearDesc& lin, int out_dtype, int region, bool swiglu) {
        const int T = a->n_tokens;
        if (!h_ssq) return linear(lin, h, h_dtype, T, out_dtype, region, -1, swiglu, false, nullptr);
        const int width = swiglu ? lin.n / 2 : lin.n;
        void* out = get(region, (int64_t)T * width * element_size(out_dtype));
        launch("imparo_rows_gemm (rows scaled at the end)", [&] {
            return imparo_rows_gemm(h, h_ssq, h_parts, h_eps, lin.weight, lin.bias, out, out_dtype, nullptr, nullptr, nullptr,
                                    nullptr, T, lin.n, lin.k, swiglu ? 1 : 0, stream);
        });
        return Out{out, 1};
    }

    void embedding(const Op& op) {
        const int T = a->n_tokens;
        x = (float*)get(p->r_residual, (int64_t)T * op.width * 4);
        pending = nullptr;
        n_pending = 0;
        launch("imparo_embed_gather", [&] {
            return imparo_embed_gather(op.table, op.table_dtype, a->tokens, x, T, op.width, op.vocab, stream);
        });
    }

    void norm(const Op& op) {
        const int T = a->n_tokens;
        if (f_weighted) {          // the product before has done the add and left what this norm's readers need
            h = const_cast<void*>(f_weighted);
            h_dtype = IMPARO_BF16;
            h_ssq = f_ssq;
            h_parts = f_parts;
            h_eps = op.eps;
            f_weighted = nullptr;
            f_ssq = nullptr;
            return;
        }
        h_ssq = nullptr;
        void* out = get(p->r_normed, (int64_t)T * op.width * element_size(op.out_dtype));
        const float* delta = pending;
        const int n_delta = pending ? n_pending : 0;
        launch("imparo_rms_norm", [&] {
            return imparo_rms_norm(x, delta, n_delta, T, nullptr, op.weight, out, op.out_dtype, T, op.width, op.eps,
                                   delta ? 1 : 0, stream);
        });
        pending = nullptr;
        n_pending = 0;
        h = out;
        h_dtype = op.out_dtype;
    }

    void decode_parts(const ImparoAttentionDesc& d, float** part_o, float** part_ml, int* n_splits) {
        const int split = imparo_attention_decode_split();
        *n_splits = (a->max_context + split - 1) / split;
        if (*n_splits < 1) *n_splits = 1;
        *part_o = (float*)get(p->r_part_o, (int64_t)a->n_single * d.heads * *n_splits * d.head_dim * 4);
        *part_ml = (float*)get(p->r_part_ml, (int64_t)a->n_single * d.heads * *n_splits * 2 * 4);
    }

    void attention(const Op& op) {
        const ImparoAttentionDesc& d = op.attention;
        const int T = a->n_tokens;
        const int dt = p->engine_dtype;
        if (d.group < 0 || d.group >= a->n_groups) return fail(IMPARO_BAD_ARGUMENT, "an attention whose cache group the step has no table for");
        const int32_t* table = a->tables[d.group];
        const int stride = a->table_width;
        const Out qkv = consume(d.qkv, IMPARO_F32, p->r_mixer_in, false);
        const int64_t o_bytes = (int64_t)T * d.heads * d.head_dim * element_size(dt);
        if (dt != d.out.dtype) return fail(IMPARO_BAD_ARGUMENT, "an output projection whose weight dtype differs from the attention output's");
        const int decode_splits = std::max(1, (a->max_context + imparo_attention_decode_split() - 1) / imparo_attention_decode_split());
        if (d.v_transposed && d.owns_cache && a->n_single == T && a->n_portion == 0 && imparo_attention_decode_qkv_pays(T, decode_splits) &&
            imparo_attention_decode_qkv_takes(d.head_dim, d.n_freq)) {
            // every row brings one token: head norm, rotation and the write of the new key and value ride in the attention launch
            void* o = get(p->r_mixer_mid, o_bytes);
            float *part_o, *part_ml;
            int n_splits;
            decode_parts(d, &part_o, &part_ml, &n_splits);
            launch("imparo_attention_decode_qkv", [&] {
                return imparo_attention_decode_qkv((const float*)qkv.ptr, d.q_norm, d.k_norm, d.norm_eps, d.inv_freq, d.n_freq,
                                                   d.interleaved, d.k_cache, d.v_cache, 1, o, part_o, part_ml, a->single_rows,
                                                   a->n_single, a->seg_start, a->positions, table, stride, p->page_size,
                                                   d.heads, d.kv_heads, d.head_dim, d.n_pages, d.scale, d.window, n_splits,
                                                   stream);
            });
            return produce(d.out, o, dt, p->r_mixer_out, p->r_mixer_out_sliced);
        }
        void* q = get(p->r_q, o_bytes);
        launch("imparo_qk_norm_rope_store", [&] {
            return imparo_qk_norm_rope_store((const float*)qkv.ptr, d.q_norm, d.k_norm, d.norm_eps, d.inv_freq, d.n_freq,
                                             d.interleaved, a->positions, a->row_of_token, d.owns_cache ? table : nullptr,
                                             d.owns_cache ? stride : 0, p->page_size, q, d.owns_cache ? d.k_cache : nullptr,
                                             d.owns_cache ? d.v_cache : nullptr, dt, d.owns_cache ? 1 : 0, T, d.heads,
                                             d.kv_heads, d.head_dim, d.owns_cache ? d.n_pages : 0, d.v_transposed, stream);
        });
        void* o = get(p->r_mixer_mid, o_bytes);
        if (d.v_transposed) {
            // matrix-core kernels: single tokens split over their keys, portions tiled over their queries
            if (a->n_single) {
                float *part_o, *part_ml;
                int n_splits;
                decode_parts(d, &part_o, &part_ml, &n_splits);
                launch("imparo_attention_decode", [&] {
                    return imparo_attention_decode(q, d.k_cache, d.v_cache, o, part_o, part_ml, a->single_rows, a->n_single,
                                                   a->seg_start, a->positions, table, stride, p->page_size, d.heads,
                                                   d.kv_heads, d.head_dim, d.n_pages, d.scale, d.window, n_splits, stream);
                });
            }
            if (a->n_portion) {
                const int parts = imparo_attention_prefill_splits(a->portion_tiles, d.heads, d.kv_heads, d.head_dim, stride * p->page_size);
                float *part_o = nullptr, *part_ml = nullptr;
                if (parts > 1) {
                    part_o = (float*)get(p->r_prefill_part_o, (int64_t)T * d.heads * parts * d.head_dim * 4);
                    part_ml = (float*)get(p->r_prefill_part_ml, (int64_t)T * d.heads * parts * 2 * 4);
                }
                launch("imparo_attention_prefill", [&] {
                    return imparo_attention_prefill(q, d.k_cache, d.v_cache, o, part_o, part_ml, parts, a->portion_rows,
                                                    a->n_portion, a->portion_tiles, a->seg_start, a->seg_len, a->positions,
                                                    table, stride, p->page_size, d.heads, d.kv_heads, d.head_dim, d.n_pages,
                                                    d.scale, d.window, stream);
                });
            }
        } else {
            launch("imparo_attention", [&] {
                return imparo_attention(q, d.k_cache, d.v_cache, o, dt, a->positions, a->row_of_token, table, stride,
                                        p->page_size, T, d.heads, d.kv_heads, d.head_dim, d.n_pages, d.scale, d.window, 0,
                                        stream);
            });
        }
        produce(d.out, o, dt, p->r_mixer_out, p->r_mixer_out_sliced);
    }

    void short_conv(const Op& op) {
        const ImparoShortConvDesc& d = op.conv;
        const int T = a->n_tokens, R = a->n_rows;
        const int y_dtype = d.out_proj.dtype;
        void* y = get(p->r_mixer_mid, (int64_t)T * d.width * element_size(y_dtype));
        const bool single = a->max_seg_len == 1;
        if (single && d.in_proj.dtype == IMPARO_BF16 && T > 0 && T <= 16 && d.in_proj.n % 24 == 0 && d.in_proj.k % 8 == 0) {
            // a decode step's few rows: projection and conv in one launch
            if (h_dtype != IMPARO_BF16) return fail(IMPARO_BAD_ARGUMENT, "a conv input projection whose input is not in its weight's dtype");
            launch("imparo_in_proj_conv_decode", [&] {
                return imparo_in_proj_conv_decode_normed(h, h_ssq, h_parts, h_eps, d.in_proj.weight, d.in_proj.bias,
                                                         d.conv_weight, d.conv_bias, d.state, a->slot, y, y_dtype, T, d.width,
                                                         d.in_proj.k, d.taps, d.n_slots, stream);
            });
            return produce(d.out_proj, y, y_dtype, p->r_mixer_out, p->r_mixer_out_sliced);
        }
        const Out bcx = consume(d.in_proj, IMPARO_F32, p->r_mixer_in, false);
        if (single) {
            if (T != R) return fail(IMPARO_BAD_ARGUMENT, "a step of single tokens whose rows and tokens differ in number");
            launch("imparo_short_conv_decode", [&] {
                return imparo_short_conv_decode((const float*)bcx.ptr, d.conv_weight, d.conv_bias, d.state, a->slot, y, y_dtype, R,
                                                d.width, d.taps, d.n_slots, stream);
            });
        } else {
            launch("imparo_short_conv", [&] {
                return imparo_short_conv((const float*)bcx.ptr, d.conv_weight, d.conv_bias, d.state, a->row_of_token, a->seg_start,
                                         a->slot, y, y_dtype, T, d.width, d.taps, d.n_slots, R, stream);
            });
            launch("imparo_short_conv_state", [&] {
                return imparo_short_conv_state((const float*)bcx.ptr, d.state, a->seg_start, a->seg_len, a->slot, R, T, d.width,
                                               d.taps, d.n_slots, stream);
            });
        }
        produce(d.out_proj, y, y_dtype, p->r_mixer_out, p->r_mixer_out_sliced);
    }

    void swiglu(const Op& op) {
        const ImparoSwigluDesc& d = op.swiglu;
        // the gated hidden may lie where the mixer's input projection lay: that is dead by now
        const Out g = consume(d.gate_up, d.down.dtype, p->r_mixer_in, true);
        produce(d.down, g.ptr, d.down.dtype, p->r_ffn_out, p->r_ffn_out_sliced);
    }

    void head(const Op& op) {
        const int W = a->n_want;
        if (W == 0) return;
        void* rows = get(p->r_normed_rows, (int64_t)W * op.width * element_size(op.head.dtype));
        const float* delta = pending;
        const int n_delta = pending ? n_pending : 0;
        launch("imparo_rms_norm (wanted rows)", [&] {
            return imparo_rms_norm(x, delta, n_delta, a->n_tokens, a->want_rows, op.weight, rows, op.head.dtype, W, op.width,
                                   op.eps, 0, stream);
        });
        const Out out = linear(op.head, rows, op.head.dtype, W, IMPARO_F32, p->r_logits, -1, false, false, nullptr);
        logits = (float*)out.ptr;
    }

    void run() {
        if (a->n_tokens < 1 || a->n_rows < 1 || a->n_groups < 0 || a->n_groups > IMPARO_MAX_GROUPS)
            return fail(IMPARO_BAD_ARGUMENT, "a step without tokens, or with more cache groups than the library takes;");
        for (op_index = 0; op_index < (int)p->ops.size() && status == IMPARO_OK; ++op_index) {
            const Op& op = p->ops[op_index];
            switch (op.kind) {
                case OP_EMBEDDING: embedding(op); break;
                case OP_NORM: norm(op); break;
                case OP_ATTENTION: attention(op); break;
                case OP_SHORT_CONV: short_conv(op); break;
                case OP_SWIGLU: swiglu(op); break;
                case OP_HEAD: head(op); break;
            }
        }
    }
};

bool good_linear(const ImparoLinearDesc& l) {
    return l.weight && l.n > 0 && l.k > 0 && (l.dtype == IMPARO_F32 || l.dtype == IMPARO_BF16);
}

}  // namespace

extern "C" int imparo_load_code() {
    const int status[] = {imparo_load_code_attention(), imparo_load_code_attention_mfma(), imparo_load_code_decode_rows(), imparo_load_code_elementwise(),
                          imparo_load_code_gemm(),      imparo_load_code_rope_cache(),     imparo_load_code_sampling()};
    for (int s : status)
        if (s != IMPARO_OK) return s;
    return IMPARO_OK;
}

extern "C" ImparoProgram* imparo_program_new(int engine_dtype, int page_size) {
    if ((engine_dtype != IMPARO_F32 && engine_dtype != IMPARO_BF16) || page_size < 1) return nullptr;
    ImparoProgram* p = new ImparoProgram();
    p->engine_dtype = engine_dtype;
    p->page_size = page_size;
    // the names are those under which a caller that runs the parts one by one keeps the same buffers
    p->r_residual = p->region("residual");
    p->r_normed = p->region("normed");
    p->r_mixer_in = p->region("mixer_in");
    p->r_mixer_mid = p->region("mixer_mid");
    p->r_q = p->region("q");
    p->r_mixer_out = p->region("mixer_out");
    p->r_mixer_out_sliced = p->region("mixer_out_sliced");
    p->r_ffn_out = p->region("ffn_out");
    p->r_ffn_out_sliced = p->region("ffn_out_sliced");
    p->r_part_o = p->region("attn_part_o");
    p->r_part_ml = p->region("attn_part_ml");
    p->r_prefill_part_o = p->region("attn_prefill_part_o");
    p->r_prefill_part_ml = p->region("attn_prefill_part_ml");
    p->r_normed_rows = p->region("normed_rows");
    p->r_logits = p->region("logits");
    p->r_fold_ssq = p->region("fold_ssq");
    p->r_fold_weighted = p->region("fold_weighted");
    return p;
}

extern "C" void imparo_program_delete(ImparoProgram* p) { delete p; }

extern "C" int imparo_program_set_fold(ImparoProgram* p, int mode) {
    if (!p || mode < 0 || mode > 2) return IMPARO_BAD_ARGUMENT;
    p->fold = mode;
    return IMPARO_OK;
}

// Whether a product of m <= 16 rows over a [n, k] weight that feeds the residual stream should add its
// result there itself and fold the next norm away: one launch less, at the price of every block
// summing the whole of K (no slices of K over blocks) and of a product behind the norm that scales its
// rows at its end. Measured on whole decode steps of 1 to 16 rows at three model widths (1024, 1536,
// 2048) with everything folded, with only the products over K <= 2048 folded (the mixers' output
// projections), and with nothing folded: the second is the fastest everywhere (a step of 8 rows at
// width 1024: 0.670 ms against 0.702 and 0.718; at width 2048: 0.915 against 0.942 and 0.934); a block
// that walks a K of 4,608 or more alone takes longer than the norm's launch it saves.
extern "C" int imparo_rows_fold_pays(int m, int n, int k) {
    (void)n;
    return m <= 16 && k <= 2048;
}

extern "C" int imparo_program_embedding(ImparoProgram* p, const void* table, int table_dtype, int vocab, int width) {
    if (!p || !table || vocab < 1 || width < 1 || !p->ops.empty()) return IMPARO_BAD_ARGUMENT;
    Op op{OP_EMBEDDING};
    op.table = table;
    op.table_dtype = table_dtype;
    op.vocab = vocab;
    op.width = width;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_norm(ImparoProgram* p, const float* weight, float eps, int width, int out_dtype) {
    if (!p || !weight || width < 1 || p->ops.empty()) return IMPARO_BAD_ARGUMENT;
    Op op{OP_NORM};
    op.weight = weight;
    op.eps = eps;
    op.width = width;
    op.out_dtype = out_dtype;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_attention(ImparoProgram* p, const ImparoAttentionDesc* d) {
    if (!p || !d || p->ops.empty() || !good_linear(d->qkv) || !good_linear(d->out)) return IMPARO_BAD_ARGUMENT;
    if (d->heads < 1 || d->kv_heads < 1 || d->heads % d->kv_heads || d->head_dim < 16 || d->head_dim % 16) return IMPARO_BAD_ARGUMENT;
    if (d->qkv.n != (d->heads + 2 * d->kv_heads) * d->head_dim || d->out.k != d->heads * d->head_dim) return IMPARO_BAD_ARGUMENT;
    if (!d->k_cache || !d->v_cache || d->n_pages < 1 || d->group < 0 || d->group >= IMPARO_MAX_GROUPS) return IMPARO_BAD_ARGUMENT;
    if ((d->q_norm == nullptr) != (d->k_norm == nullptr) || (d->n_freq > 0 && !d->inv_freq)) return IMPARO_BAD_ARGUMENT;
    Op op{OP_ATTENTION};
    op.attention = *d;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_short_conv(ImparoProgram* p, const ImparoShortConvDesc* d) {
    if (!p || !d || p->ops.empty() || !good_linear(d->in_proj) || !good_linear(d->out_proj)) return IMPARO_BAD_ARGUMENT;
    if (d->width < 1 || d->taps < 2 || d->in_proj.n != 3 * d->width || d->out_proj.k != d->width || !d->conv_weight ||
        !d->state || d->n_slots < 1)
        return IMPARO_BAD_ARGUMENT;
    Op op{OP_SHORT_CONV};
    op.conv = *d;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_swiglu(ImparoProgram* p, const ImparoSwigluDesc* d) {
    if (!p || !d || p->ops.empty() || !good_linear(d->gate_up) || !good_linear(d->down)) return IMPARO_BAD_ARGUMENT;
    if (d->gate_up.n % 2 || d->down.k != d->gate_up.n / 2) return IMPARO_BAD_ARGUMENT;
    Op op{OP_SWIGLU};
    op.swiglu = *d;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_head(ImparoProgram* p, const float* norm_weight, float eps, int width,
                                   const ImparoLinearDesc* head) {
    if (!p || !norm_weight || !head || p->ops.empty() || !good_linear(*head) || head->k != width) return IMPARO_BAD_ARGUMENT;
    Op op{OP_HEAD};
    op.weight = norm_weight;
    op.eps = eps;
    op.width = width;
    op.head = *head;
    p->ops.push_back(op);
    return IMPARO_OK;
}

extern "C" int imparo_program_n_regions(const ImparoProgram* p) { return p ? (int)p->regions.size() : 0; }

extern "C" const char* imparo_program_region_name(const ImparoProgram* p, int region) {
    if (!p || region < 0 || region >= (int)p->regions.size()) return "";
    return p->regions[region].name.c_str();
}

extern "C" int imparo_program_bind(ImparoProgram* p, int region, void* ptr, int64_t bytes) {
    if (!p || region < 0 || region >= (int)p->regions.size() || bytes < 0 || (bytes > 0 && !ptr)) return IMPARO_BAD_ARGUMENT;
    if ((uintptr_t)ptr & 15) return IMPARO_BAD_ARGUMENT;       // the kernels load 16 bytes at a time
    p->regions[region].ptr = (char*)ptr;
    p->regions[region].bytes = bytes;
    return IMPARO_OK;
}

extern "C" int imparo_program_needs(ImparoProgram* p, const ImparoStepArgs* args, int64_t* needs) {
    if (!p || !args || !needs) return IMPARO_BAD_ARGUMENT;
    Walk w(p, args, nullptr, true);
    w.run();
    for (size_t i = 0; i < w.need.size(); ++i) needs[i] = w.need[i];
    return w.status;
}

extern "C" int imparo_program_run(ImparoProgram* p, const ImparoStepArgs* args, float** logits, imparo_stream stream) {
    if (!p || !args || !logits) return IMPARO_BAD_ARGUMENT;
    *logits = nullptr;
    Walk dry(p, args, nullptr, true);
    dry.run();
    if (dry.status != IMPARO_OK) return dry.status;
    for (size_t i = 0; i < dry.need.size(); ++i)
        if (dry.need[i] > p->regions[i].bytes) {
            char buf[200];
            snprintf(buf, sizeof buf, "region %s holds %lld bytes and the step needs %lld", p->regions[i].name.c_str(),
                     (long long)p->regions[i].bytes, (long long)dry.need[i]);
            p->error = buf;
            return IMPARO_SCRATCH_TOO_SMALL;
        }
    Walk w(p, args, stream, false);
    w.run();
    *logits = w.logits;
    return w.status;
}

extern "C" const char* imparo_program_error(const ImparoProgram* p) { return p ? p->error.c_str() : ""; }
