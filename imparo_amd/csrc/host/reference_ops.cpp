// Plain C++ statements of what each GPU kernel computes: float32, whole arrays, one loop per
// sum, no tiling, no cache. They exist to be compared with the kernels (tests) and share no
// code with them. Sums run in the order a reader would write them: k = 0, 1, 2, ...
// Formulas as the reference's CPU path states them: RMS norm ops.rs:6-22, linear
// ops.rs:660-674, short conv ops.rs:80-167, SiLU ops.rs:73-78, rotation ops.rs:551-569,
// attention cpu_support.rs:402-445 with softmax ops.rs:572-583, argmax ops.rs:628-640
// (all under /root/reference/crates/imparo-cpu/src or imparo-model/src).
#include "host_api.h"

#include <cmath>
#include <cstring>
#include <limits>
#include <vector>

extern "C" {

void imparo_ref_embed(const float* table, const int32_t* ids, float* x, int n_tokens, int width) {
    for (int t = 0; t < n_tokens; ++t) std::memcpy(x + (size_t)t * width, table + (size_t)ids[t] * width, sizeof(float) * width);
}

// y = x * (1 / sqrt(mean(x^2) + eps)) * w, the mean a sequential float32 sum
void imparo_ref_rms_norm(const float* x, const float* w, float eps, float* y, int rows, int width) {
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * width;
        float ss = 0.f;
        for (int i = 0; i < width; ++i) ss += xr[i] * xr[i];
        const float scale = 1.0f / std::sqrt(ss / (float)width + eps);
        for (int i = 0; i < width; ++i) y[(size_t)r * width + i] = xr[i] * scale * w[i];
    }
}

// y[m, n] = sum_k x[m, k] w[n, k] (+ bias[n]): one accumulator per output, fused multiply-adds
// in the order k = 0, 1, 2, ... -- the order the float32 GPU kernel keeps whatever its tiling
void imparo_ref_gemm(const float* x, const float* w, const float* bias, float* y, int m, int n, int k) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float acc = 0.f;
            for (int q = 0; q < k; ++q) acc = std::fmaf(x[(size_t)i * k + q], w[(size_t)j * k + q], acc);
            y[(size_t)i * n + j] = bias ? acc + bias[j] : acc;
        }
}

// out = silu(gate) * up, silu(g) = g / (1 + exp(-g)): the activation sits on the gate
void imparo_ref_swiglu(const float* gate, const float* up, float* out, int64_t count) {
    for (int64_t i = 0; i < count; ++i) out[i] = gate[i] / (1.0f + std::exp(-gate[i])) * up[i];
}

// Per (token, head): optional RMS norm over the head's dims with weight w[head_dim], then the
// rotation of pairs (i, i + n_freq): angle = position * inv_freq[i], the product in float64.
void imparo_ref_head_norm_rope(const float* x, const float* w, float eps, const int32_t* positions,
                               const float* inv_freq, int n_freq, float* y, int n_tokens, int heads, int head_dim) {
    std::vector<float> row((size_t)head_dim);
    for (int t = 0; t < n_tokens; ++t)
        for (int h = 0; h < heads; ++h) {
            const float* src = x + ((size_t)t * heads + h) * head_dim;
            float* dst = y + ((size_t)t * heads + h) * head_dim;
            if (w) {
                float ss = 0.f;
                for (int i = 0; i < head_dim; ++i) ss += src[i] * src[i];
                const float scale = 1.0f / std::sqrt(ss / (float)head_dim + eps);
                for (int i = 0; i < head_dim; ++i) row[(size_t)i] = src[i] * scale * w[i];
            } else {
                for (int i = 0; i < head_dim; ++i) row[(size_t)i] = src[i];
            }
            for (int i = 0; i < n_freq; ++i) {
                const float theta = (float)((double)positions[t] * (double)inv_freq[i]);
                const float sn = std::sin(theta), cs = std::cos(theta);
                const float x0 = row[(size_t)i], x1 = row[(size_t)(i + n_freq)];
                row[(size_t)i] = x0 * cs - x1 * sn;
                row[(size_t)(i + n_freq)] = x0 * sn + x1 * cs;
            }
            for (int i = 0; i < head_dim; ++i) dst[i] = row[(size_t)i];
        }
}

// One request whose keys and values of positions 0 .. n_keys-1 are given: the query at position
// p reads keys max(0, p + 1 - window) .. p (window 0: all from 0); kv head of head h is
// h / (heads / kv_heads); softmax with the maximum subtracted.
void imparo_ref_attention(const float* q, const float* k, const float* v, const int32_t* q_positions, float* out,
                          int n_queries, int heads, int kv_heads, int head_dim, float scale, int window) {
    const int group = heads / kv_heads;
    std::vector<float> s;
    for (int t = 0; t < n_queries; ++t) {
        const int pos = q_positions[t];
        const int lo = window > 0 ? std::max(0, pos + 1 - window) : 0;
        s.resize((size_t)(pos - lo + 1));
        for (int h = 0; h < heads; ++h) {
            const int kvh = h / group;
            const float* qr = q + ((size_t)t * heads + h) * head_dim;
            float mx = -std::numeric_limits<float>::infinity();
            for (int p = lo; p <= pos; ++p) {
                const float* kr = k + ((size_t)p * kv_heads + kvh) * head_dim;
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot += qr[d] * kr[d];
                s[(size_t)(p - lo)] = dot * scale;
                mx = std::max(mx, dot * scale);
            }
            float sum = 0.f;
            for (int p = lo; p <= pos; ++p) {
                s[(size_t)(p - lo)] = std::exp(s[(size_t)(p - lo)] - mx);
                sum += s[(size_t)(p - lo)];
            }
            float* o = out + ((size_t)t * heads + h) * head_dim;
            for (int d = 0; d < head_dim; ++d) {
                float acc = 0.f;
                for (int p = lo; p <= pos; ++p) acc += s[(size_t)(p - lo)] / sum * v[((size_t)p * kv_heads + kvh) * head_dim + d];
                o[d] = acc;
            }
        }
    }
}

// One request's segment: bcx[t] = (B | C | x), u = B * x, seq = state ++ u (state: the last
// taps-1 values of u, oldest first), conv[t][c] = sum_j w[c][j] seq[t + j][c] (tap 0 meets the
// oldest value) + bias[c], y = C * conv; the state becomes the last taps-1 rows of seq.
void imparo_ref_short_conv(const float* bcx, const float* w, const float* bias, float* state, float* y, int n_tokens,
                           int width, int taps) {
    const int hist = taps - 1;
    std::vector<float> seq((size_t)(hist + n_tokens) * width);
    std::memcpy(seq.data(), state, sizeof(float) * (size_t)hist * width);
    for (int t = 0; t < n_tokens; ++t)
        for (int c = 0; c < width; ++c)
            seq[(size_t)(hist + t) * width + c] = bcx[(size_t)t * 3 * width + c] * bcx[(size_t)t * 3 * width + 2 * width + c];
    for (int t = 0; t < n_tokens; ++t)
        for (int c = 0; c < width; ++c) {
            float acc = 0.f;
            for (int j = 0; j < taps; ++j) acc = std::fmaf(w[(size_t)c * taps + j], seq[(size_t)(t + j) * width + c], acc);
            if (bias) acc += bias[c];
            y[(size_t)t * width + c] = bcx[(size_t)t * 3 * width + width + c] * acc;
        }
    std::memcpy(state, seq.data() + (size_t)n_tokens * width, sizeof(float) * (size_t)hist * width);
}

// The smallest index at the maximum; NaN never wins; a row of NaN gives 0
void imparo_ref_argmax(const float* logits, int32_t* out, int rows, int vocab) {
    for (int r = 0; r < rows; ++r) {
        const float* row = logits + (size_t)r * vocab;
        int best = -1;
        for (int i = 0; i < vocab; ++i)
            if (row[i] == row[i] && (best < 0 || row[i] > row[best])) best = i;
        out[r] = best < 0 ? 0 : best;
    }
}

// Temperature sampling by inverse CDF: weights exp((l - max) / T) (a NaN logit weighs nothing),
// the pick is the first index whose running sum exceeds uniform * total; sums in float64.
// temperature <= 0 is the argmax.
void imparo_ref_sample(const float* logits, const float* temperature, const float* uniform, int32_t* out, int rows,
                       int vocab) {
    imparo_ref_argmax(logits, out, rows, vocab);
    for (int r = 0; r < rows; ++r) {
        if (!(temperature[r] > 0.f)) continue;
        const float* row = logits + (size_t)r * vocab;
        const float mx = row[out[r]];
        double total = 0.0;
        for (int i = 0; i < vocab; ++i) {
            const float e = std::exp((row[i] - mx) / temperature[r]);
            if (e == e) total += e;
        }
        const double target = (double)uniform[r] * total;
        double cum = 0.0;
        int pick = out[r], last = out[r];
        bool found = false;
        for (int i = 0; i < vocab && !found; ++i) {
            const float e = std::exp((row[i] - mx) / temperature[r]);
            if (!(e == e) || !(e > 0.f)) continue;
            cum += e;
            last = i;
            if (cum > target) {
                pick = i;
                found = true;
            }
        }
        out[r] = found ? pick : last;
    }
}

}  // extern "C"
