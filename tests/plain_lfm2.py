"""A plain, slow LFM2 in float32 on the CPU: whole sequences, no cache, one
function per part. It shares no code with the engine; every formula is written
from the reference's text and cites it (paths under /root/reference).

Used as the yardstick for the engine's logits in every way of cutting and
batching requests.
"""
import json
import math
import os

import numpy as np
import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- parts

def rms_norm(x, weight, eps):
    """crates/imparo-cpu/src/ops.rs:6-22 -- mean of squares over the row, scale
    = 1/sqrt(mean + eps), y = x * scale * w. No +1 offset, no bias."""
    x = x.to(torch.float32)
    mean = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    scale = 1.0 / torch.sqrt(mean + eps)
    return x * scale * weight


def linear(x, weight, bias=None):
    """crates/imparo-cpu/src/ops.rs:660-674 -- y[j] = sum_i W[j, i] x[i]; the
    weight is [n_out rows of n_in]."""
    y = x @ weight.t()
    return y if bias is None else y + bias


def silu(x):
    """crates/imparo-cpu/src/ops.rs:73-78 -- t / (1 + exp(-t))."""
    return x / (1.0 + torch.exp(-x))


def swiglu(n, w1, w3, w2):
    """crates/imparo-model/src/lfm2/workflow_cpu.rs:307-313 -- SiLU on the GATE
    (w1), times up (w3), then down (w2)."""
    return linear(silu(linear(n, w1)) * linear(n, w3), w2)


def rope_neox(x, positions, base, n_rot):
    """crates/imparo-cpu/src/ops.rs:551-569 -- dimension i pairs with i + n_rot/2;
    inv_i = base^(-2i/n_rot) in f32; theta = pos * inv (product in f64, then f32);
    x_i' = x_i cos - x_{i+half} sin; x_{i+half}' = x_i sin + x_{i+half} cos.
    x is [T, heads, D]; positions [T]."""
    half = n_rot // 2
    i = np.arange(half, dtype=np.float32)
    inv = np.power(np.float32(base), (np.float32(-2.0) * i / np.float32(n_rot)).astype(np.float32)).astype(np.float32)
    theta = (np.asarray(positions, dtype=np.float64)[:, None] * inv.astype(np.float64)[None, :]).astype(np.float32)
    cos = torch.from_numpy(np.cos(theta)).unsqueeze(1)
    sin = torch.from_numpy(np.sin(theta)).unsqueeze(1)
    out = x.clone()
    x0 = x[..., :half]
    x1 = x[..., half:n_rot]
    out[..., :half] = x0 * cos - x1 * sin
    out[..., half:n_rot] = x0 * sin + x1 * cos
    return out


def attend(q, k, v, positions, scale, window=None):
    """crates/imparo-model/src/cpu_support.rs:402-445 -- kv head of head h is
    h // (H/Hk) (contiguous groups); the query at pos sees keys lo..pos with
    lo = 0, or pos+1-w under a window; causality is the position bound, there
    is no mask tensor; softmax with max subtraction (ops.rs:572-583).
    q [T,H,D]; k, v [T,Hk,D] hold positions 0..T-1 of one request; positions
    are the queries' own absolute positions (here 0..T-1)."""
    T, H, D = q.shape
    Hk = k.shape[1]
    per_kv = H // Hk
    out = torch.zeros(T, H, D, dtype=torch.float32)
    for t in range(T):
        pos = int(positions[t])
        lo = 0 if window is None else max(0, pos + 1 - window)
        for h in range(H):
            kvh = h // per_kv
            s = (k[lo:pos + 1, kvh] @ q[t, h]) * scale
            p = torch.exp(s - s.max())
            p = p / p.sum()
            out[t, h] = p @ v[lo:pos + 1, kvh]
    return out


def short_conv(bcx, conv_w, conv_b=None, state=None):
    """crates/imparo-cpu/src/ops.rs:109-167 -- row = [B | C | x]; u = B*x;
    seq = state ++ u (state: the previous L-1 raw u rows, oldest first, zeros
    for a fresh request); conv_t = sum_k w[ch,k] seq[t+k] (tap 0 multiplies the
    OLDEST value); y_t = C_t * conv_t; state' = last L-1 rows of seq.
    The optional bias (not in the reference) is added to conv_t before C."""
    T, three_e = bcx.shape
    E = three_e // 3
    L = conv_w.shape[-1]
    w = conv_w.reshape(E, L)
    B, C, x = bcx[:, :E], bcx[:, E:2 * E], bcx[:, 2 * E:]
    u = B * x
    if state is None:
        state = torch.zeros(L - 1, E, dtype=torch.float32)
    seq = torch.cat([state, u], dim=0)
    conv = torch.zeros(T, E, dtype=torch.float32)
    for kk in range(L):
        conv = conv + w[:, kk][None, :] * seq[kk:kk + T]
    if conv_b is not None:
        conv = conv + conv_b
    return C * conv, seq[T:T + L - 1].clone()


def argmax_first(logits):
    """crates/imparo-cpu/src/ops.rs:628-640 -- the smallest index attaining the
    maximum; NaN never wins, all-NaN gives 0."""
    a = np.asarray(logits, dtype=np.float32)
    m = -np.inf
    for v in a:
        if v > m:
            m = v
    hits = np.nonzero(a == m)[0]
    return int(hits[0]) if len(hits) else 0


def ff_dim_from_config(cfg):
    """The SwiGLU width as config.json gives it: block_ff_dim (intermediate_size
    where a file has only that), two thirds of it times the multiplier rounded
    up to multiple_of unless auto-adjust is switched off."""
    if cfg.get("block_auto_adjust_ff_dim", True):
        f = int(2 * cfg.get("block_ff_dim", cfg.get("intermediate_size")) / 3)
        mult = cfg.get("block_ffn_dim_multiplier", 1.0)
        if mult is not None:
            f = int(mult * f)
        m = cfg.get("block_multiple_of", 256)
        return m * ((f + m - 1) // m)
    return cfg.get("block_ff_dim", cfg.get("intermediate_size"))


# --------------------------------------------------------------------------- model

class PlainLfm2:
    """crates/imparo-model/src/lfm2/workflow_cpu.rs:8-15,131-332 --
        x = embed[token]                                  (no scale)
        block: x = x + mixer(rms_norm(x, operator_norm))
               x = x + w2( silu(w1 n) * (w3 n) ),  n = rms_norm(x, ffn_norm)
        logits = lm_head( rms_norm(x, embedding_norm) )   (lm_head = embed when tied)
    """

    def __init__(self, model_dir):
        with open(os.path.join(model_dir, "config.json")) as f:
            self.cfg = json.load(f)
        self.w = {}
        with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(torch.float32)
        c = self.cfg
        self.E = c["hidden_size"]
        self.H = c["num_attention_heads"]
        self.Hk = c["num_key_value_heads"]
        self.D = self.E // self.H
        self.eps = c.get("norm_eps", 1e-5)
        self.theta = c.get("rope_theta", 1000000.0)
        self.bias = c.get("conv_bias", False)

    def norm_and_rotate(self, x, weight, rope_positions):
        """crates/imparo-model/src/cpu_support.rs:361-376 -- per (token, head):
        the RMS norm over the head with one weight [D] for all heads FIRST,
        then the rotation of the normed row."""
        return rope_neox(rms_norm(x, weight, self.eps), rope_positions, self.theta, self.D)

    def mixer_attention(self, i, h, positions, window, shared_kv=None, rope_positions=None):
        """Returns the mixer's output and the (k, v) it attended over; with
        `shared_kv` the layer projects only q and reads another call's k, v.
        `positions` index the request's own keys (0..T-1); `rope_positions`
        are the angles' positions when they differ from those."""
        p = f"model.layers.{i}.self_attn."
        T = h.shape[0]
        if rope_positions is None:
            rope_positions = positions
        q = linear(h, self.w[p + "q_proj.weight"]).reshape(T, self.H, self.D)
        # on q and k; v untouched (workflow_cpu.rs:209-229)
        q = self.norm_and_rotate(q, self.w[p + "q_layernorm.weight"], rope_positions)
        if shared_kv is None:
            k = linear(h, self.w[p + "k_proj.weight"]).reshape(T, self.Hk, self.D)
            v = linear(h, self.w[p + "v_proj.weight"]).reshape(T, self.Hk, self.D)
            k = self.norm_and_rotate(k, self.w[p + "k_layernorm.weight"], rope_positions)
        else:
            k, v = shared_kv
        o = attend(q, k, v, positions, 1.0 / math.sqrt(self.D), window)
        return linear(o.reshape(T, self.H * self.D), self.w[p + "out_proj.weight"]), (k, v)

    def mixer_conv(self, i, h):
        p = f"model.layers.{i}.conv."
        b = (lambda n: self.w[p + n]) if self.bias else (lambda n: None)
        bcx = linear(h, self.w[p + "in_proj.weight"], b("in_proj.bias"))
        y, _ = short_conv(bcx, self.w[p + "conv.weight"], b("conv.bias"))
        return linear(y, self.w[p + "out_proj.weight"], b("out_proj.bias"))

    def hidden(self, tokens, order=None, first_position=0):
        """`order`: list of (layer, cache_of) calls; None runs every layer once.
        cache_of names an earlier call whose k, v this call reads.
        `first_position` turns every rotation as if the sequence began there."""
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        T = tokens.shape[0]
        positions = np.arange(T)
        rope_positions = positions + first_position
        x = self.w["model.embed_tokens.weight"][tokens]
        if order is None:
            order = [(i, None) for i in range(len(self.cfg["layer_types"]))]
        kv_of_call = {}
        for c, (i, cache_of) in enumerate(order):
            kind = self.cfg["layer_types"][i]
            p = f"model.layers.{i}."
            h = rms_norm(x, self.w[p + "operator_norm.weight"], self.eps)
            if kind == "conv":
                m = self.mixer_conv(i, h)
            else:
                window = self.cfg.get("sliding_window") if kind == "sliding_attention" else None
                m, kv_of_call[c] = self.mixer_attention(i, h, positions, window,
                                                        None if cache_of is None else kv_of_call[cache_of],
                                                        rope_positions)
            x = x + m
            n = rms_norm(x, self.w[p + "ffn_norm.weight"], self.eps)
            x = x + swiglu(n, self.w[p + "feed_forward.w1.weight"], self.w[p + "feed_forward.w3.weight"],
                           self.w[p + "feed_forward.w2.weight"])
        return x

    def logits(self, tokens, order=None, first_position=0):
        """Logits [T, V] of one whole sequence from position 0."""
        x = self.hidden(tokens, order, first_position)
        head = self.w["model.embed_tokens.weight"] if self.cfg.get("tie_embedding", True) \
            else self.w["lm_head.weight"]
        return linear(rms_norm(x, self.w["model.embedding_norm.weight"], self.eps), head)

    def greedy(self, prompt, n_new):
        seq = list(prompt)
        out = []
        for _ in range(n_new):
            nxt = argmax_first(self.logits(seq)[-1].numpy())
            out.append(nxt)
            seq.append(nxt)
        return out
