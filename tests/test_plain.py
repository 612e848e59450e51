"""Pins the plain implementation by what fixes it beside the reference's text:
vectors the reference's own tests hold, special cases that reduce to a library
routine, and invariants. Each is chosen so that a plausible mistake fails it.
"""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as P


# ---------------------------------------------------------------- short conv
def _bcx(b, c, x):
    return torch.tensor([list(bb) + list(cc) + list(xx) for bb, cc, xx in zip(b, c, x)], dtype=torch.float32)


def test_conv_tap_zero_is_the_oldest_value():
    # /root/reference/crates/imparo-cpu/src/ops.rs:1207-1254: width 1, kernel 3, state [5,7],
    # b = x = c = 1 for two tokens; tap-0-only -> out [5,7], state' [1,1]; last-tap-only -> [1,1]
    bcx = _bcx([[1.0]] * 2, [[1.0]] * 2, [[1.0]] * 2)
    state = torch.tensor([[5.0], [7.0]])
    y, s = P.short_conv(bcx, torch.tensor([[[1.0, 0.0, 0.0]]]), state=state)
    assert y.flatten().tolist() == [5.0, 7.0] and s.flatten().tolist() == [1.0, 1.0]
    y, _ = P.short_conv(bcx, torch.tensor([[[0.0, 0.0, 1.0]]]), state=state)
    assert y.flatten().tolist() == [1.0, 1.0]


def test_conv_reference_native_vectors():
    # /root/reference/crates/imparo-cuda/native/tests/lfm2_ops_test.cpp:46-62: width 1, kernel 4,
    # state {11,13,17}, bcx {2,0,3, 2,0,5}, oldest-tap weights {1,0,0,0} -> out {0,0}, state' {17,6,10}
    oldest = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]])
    bcx = _bcx([[2.0], [2.0]], [[0.0], [0.0]], [[3.0], [5.0]])
    y, s = P.short_conv(bcx, oldest, state=torch.tensor([[11.0], [13.0], [17.0]]))
    assert y.flatten().tolist() == [0.0, 0.0]
    assert s.flatten().tolist() == [17.0, 6.0, 10.0]
    # same file: all-ones rows over state {5,7,9} with the oldest tap -> out {5,7}
    y, _ = P.short_conv(torch.ones(2, 3), oldest, state=torch.tensor([[5.0], [7.0], [9.0]]))
    assert y.flatten().tolist() == [5.0, 7.0]
    # lfm2_ops_test.cpp:64-72: history 2, one token {b2, c1, x3} over {5,7} -> {7,6}
    _, s = P.short_conv(_bcx([[2.0]], [[1.0]], [[3.0]]), torch.tensor([[[0.0, 0.0, 0.0]]]),
                        state=torch.tensor([[5.0], [7.0]]))
    assert s.flatten().tolist() == [7.0, 6.0]


def test_conv_c_gates_the_output_and_the_state_still_advances():
    # ops.rs:1258-1285: c = 0, b = 2, x = 3 -> out 0, state holds b*x = 6
    y, s = P.short_conv(_bcx([[2.0]], [[0.0]], [[3.0]]), torch.tensor([[[1.0, 1.0]]]),
                        state=torch.tensor([[9.0]]))
    assert y.item() == 0.0 and s.item() == 6.0


def test_conv_batch_equals_one_token_at_a_time():
    # ops.rs:1161-1203: width 4, kernel 3, 5 tokens; exact binary fractions so equality is exact
    g = torch.Generator().manual_seed(0)
    bcx = torch.randint(-8, 8, (5, 12), generator=g).float() / 4
    w = torch.randint(-8, 8, (4, 1, 3), generator=g).float() / 4
    y_all, s_all = P.short_conv(bcx, w)
    state = None
    ys = []
    for t in range(5):
        y, state = P.short_conv(bcx[t:t + 1], w, state=state)
        ys.append(y)
    assert torch.equal(torch.cat(ys), y_all) and torch.equal(state, s_all)


def test_conv_reduces_to_a_depthwise_conv1d():
    g = torch.Generator().manual_seed(1)
    T, E, L = 9, 6, 4
    bcx = torch.randn(T, 3 * E, generator=g)
    w = torch.randn(E, 1, L, generator=g)
    bias = torch.randn(E, generator=g)
    u = (bcx[:, :E] * bcx[:, 2 * E:]).t().unsqueeze(0)                    # [1, E, T]
    lib = torch.nn.functional.conv1d(torch.nn.functional.pad(u, (L - 1, 0)), w, bias, groups=E)[0].t()
    y, _ = P.short_conv(bcx, w, bias)
    torch.testing.assert_close(y, bcx[:, E:2 * E] * lib, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- attention
def test_attention_is_causal_and_scaled():
    # /root/reference/crates/imparo-model/src/cpu_support.rs:485-512
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]])
    k = torch.tensor([[[0.0, 1.0]], [[1.0, 0.0]]])
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]])
    out = P.attend(q, k, v, [0, 1], 1.0)
    assert out[0, 0].tolist() == [1.0, 0.0]
    assert abs(out[1, 0].sum().item() - 1.0) < 1e-6 and out[1, 0, 1] > out[1, 0, 0]
    # scores 0 and 1 at scale 1: weights 1/(1+e), e/(1+e); scale 0.5 changes them
    assert abs(out[1, 0, 1].item() - math.e / (1 + math.e)) < 1e-6
    half = P.attend(q, k, v, [0, 1], 0.5)
    assert abs(half[1, 0, 1].item() - math.exp(0.5) / (1 + math.exp(0.5))) < 1e-6


def test_a_window_of_one_leaves_each_token_alone():
    # cpu_support.rs:516-535
    q = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]]])
    k = torch.tensor([[[0.0, 1.0]], [[1.0, 0.0]]])
    v = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]])
    out = P.attend(q, k, v, [0, 1], 1.0, window=1)
    assert out[0, 0].tolist() == [1.0, 0.0] and out[1, 0].tolist() == [0.0, 1.0]


def test_grouped_query_heads_map_contiguously():
    # cpu_support.rs:538-557: 4 heads, 2 kv heads, v = [10, 20] -> [10, 10, 20, 20]
    q = torch.ones(1, 4, 1)
    k = torch.ones(1, 2, 1)
    v = torch.tensor([[[10.0], [20.0]]])
    assert P.attend(q, k, v, [0], 1.0).flatten().tolist() == [10.0, 10.0, 20.0, 20.0]


def test_attention_reduces_to_the_library_routine():
    g = torch.Generator().manual_seed(2)
    T, H, Hk, D = 11, 6, 2, 8
    q, k, v = torch.randn(T, H, D, generator=g), torch.randn(T, Hk, D, generator=g), torch.randn(T, Hk, D, generator=g)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1).repeat_interleave(H // Hk, 0),
        v.transpose(0, 1).repeat_interleave(H // Hk, 0), is_causal=True).transpose(0, 1)
    torch.testing.assert_close(P.attend(q, k, v, range(T), 1.0 / math.sqrt(D)), lib, rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- rotation
def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 2, 8, generator=g)
    assert torch.equal(P.rope_neox(x[:1], [0], 10000.0, 8), x[:1])
    y = P.rope_neox(x, [3, 17, 100, 4000], 10000.0, 8)
    torch.testing.assert_close(x[..., :4] ** 2 + x[..., 4:] ** 2, y[..., :4] ** 2 + y[..., 4:] ** 2,
                               rtol=1e-5, atol=1e-5)


def test_rope_pairs_i_with_i_plus_half_and_turns_the_right_way():
    # one pair (i=0, inv=1): position p turns (1, 0) to (cos p, sin p); an interleaved pairing or a
    # flipped sign fails this
    x = torch.zeros(1, 1, 4)
    x[0, 0, 0] = 1.0
    y = P.rope_neox(x, [1], 10000.0, 4)
    assert abs(y[0, 0, 0].item() - math.cos(1.0)) < 1e-6 and abs(y[0, 0, 2].item() - math.sin(1.0)) < 1e-6
    assert y[0, 0, 1].item() == 0.0 and y[0, 0, 3].item() == 0.0
    # second pair turns by base^(-2/4) = 0.01 per position
    x = torch.zeros(1, 1, 4)
    x[0, 0, 1] = 1.0
    y = P.rope_neox(x, [50], 10000.0, 4)
    assert abs(y[0, 0, 1].item() - math.cos(0.5)) < 1e-6 and abs(y[0, 0, 3].item() - math.sin(0.5)) < 1e-6


def test_rope_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(4)
    q, k = torch.randn(1, 1, 16, generator=g), torch.randn(1, 1, 16, generator=g)
    def score(m, n):
        return (P.rope_neox(q, [m], 10000.0, 16) * P.rope_neox(k, [n], 10000.0, 16)).sum().item()
    assert abs(score(5, 2) - score(105, 102)) < 1e-4 and abs(score(5, 2) - score(9, 2)) > 1e-3


# ---------------------------------------------------------------- the rest
def test_rms_norm():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 10, generator=g)
    w = torch.ones(10)
    y = P.rms_norm(x, w, 0.0)
    torch.testing.assert_close((y * y).mean(-1), torch.ones(3), rtol=1e-5, atol=1e-5)      # unit rms
    torch.testing.assert_close(P.rms_norm(7 * x, w, 0.0), y, rtol=1e-5, atol=1e-5)        # scale free
    w2 = torch.arange(10).float()
    torch.testing.assert_close(P.rms_norm(x, w2, 1e-5), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w2)
    # the weight multiplies: no +1 offset (a zero weight gives zero)
    assert torch.equal(P.rms_norm(x, torch.zeros(10), 1e-5), torch.zeros(3, 10))
    # eps is inside the root: a zero row stays zero and finite
    assert torch.equal(P.rms_norm(torch.zeros(1, 10), w, 1e-5), torch.zeros(1, 10))


def test_silu_values_and_gate_side():
    # lfm2_ops_test.cpp:83-84
    assert abs(P.silu(torch.tensor(1.0)).item() - 0.7310586) < 1e-6 and P.silu(torch.tensor(0.0)).item() == 0.0
    torch.testing.assert_close(P.silu(torch.linspace(-5, 5, 11)), torch.nn.functional.silu(torch.linspace(-5, 5, 11)))
    # SiLU is on the gate (w1): with w3 x = 1 the result is silu(w1 x); swapping the roles changes it
    n = torch.tensor([[2.0]])
    w1, w3, w2 = torch.tensor([[1.0]]), torch.tensor([[0.5]]), torch.tensor([[1.0]])
    assert abs(P.swiglu(n, w1, w3, w2).item() - (2.0 / (1 + math.exp(-2.0))) * 1.0) < 1e-6


def test_linear_is_out_by_in():
    w = torch.tensor([[1.0, 2.0, 3.0], [0.0, 1.0, 0.0]])
    assert P.linear(torch.tensor([[1.0, 1.0, 1.0]]), w).tolist() == [[6.0, 1.0]]


def test_argmax_first_max_and_nan():
    assert P.argmax_first([1.0, 3.0, 3.0, 2.0]) == 1
    assert P.argmax_first([float("nan"), 1.0, float("nan")]) == 1
    assert P.argmax_first([float("nan")] * 3) == 0
    assert P.argmax_first(np.arange(5.0)) == int(np.argmax(np.arange(5.0)))


def test_ff_dim():
    for ff, mult, want in ((12288, 256, 8192), (10240, 256, 6912), (6656, 256, 4608), (480, 64, 320)):
        assert P.ff_dim_from_config(dict(block_auto_adjust_ff_dim=True, block_ff_dim=ff, block_multiple_of=mult)) == want
    assert P.ff_dim_from_config(dict(block_auto_adjust_ff_dim=False, block_ff_dim=192)) == 192


def test_whole_model_is_causal_and_one_expert_head_cases(plain_models):
    """A later token never changes an earlier logit; and the model's greedy
    continuation is a function of the prefix."""
    m = plain_models["A"]
    toks = list(range(3, 23))
    a = m.logits(toks)
    b = m.logits(toks[:12] + [200] * 8)
    torch.testing.assert_close(a[:12], b[:12], rtol=1e-5, atol=1e-6)
    assert not torch.allclose(a[12:], b[12:], atol=1e-4)


# ---------------------------------------------------------------- the whole model's composition
# What fixes the arrangement of the parts beside the reference's text
# (/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:8-15,203-229): each case below
# fails for one plausible way of putting right parts together wrongly.

def test_only_distances_count_because_the_head_norm_comes_before_the_rotation(plain_models):
    """Turning every position by the same amount changes no logit: conv blocks
    know no positions and rotated scores depend on distances only. That holds
    only if q and k are normed first and rotated after: a per-dimension weight
    applied after the rotation scales the two halves of a pair differently and
    the score of a pair of positions then depends on where they are."""
    for name, vocab in (("A", 256), ("B", 384)):
        m = plain_models[name]
        toks = [(7 * i + 3) % vocab for i in range(24)]
        a, b = m.logits(toks), m.logits(toks, first_position=57)
        torch.testing.assert_close(a, b, rtol=2e-4, atol=2e-5)

        class RotatesFirst(type(m)):
            def norm_and_rotate(self, x, weight, rope_positions):
                return P.rms_norm(P.rope_neox(x, rope_positions, self.theta, self.D), weight, self.eps)
        wrong = RotatesFirst.__new__(RotatesFirst)
        wrong.__dict__.update(m.__dict__)
        wa, wb = wrong.logits(toks), wrong.logits(toks, first_position=57)
        assert (wa - wb).abs().max() > 50 * (a - b).abs().max()      # the mistake would show


def test_blocks_add_to_the_stream_and_the_last_norm_feeds_the_head(plain_models):
    """With every block's way back into the stream silenced (out_proj and w2
    zero) the logits are head(rms_norm(embedding, embedding_norm)): the blocks
    only ever add, nothing scales or norms the stream itself, and the head
    reads the normed stream (tied: the embedding table; untied: lm_head)."""
    import copy
    for name, vocab in (("A", 256), ("B", 384)):
        m = copy.copy(plain_models[name])
        m.w = dict(m.w)
        for k in list(m.w):
            if k.endswith("out_proj.weight") or k.endswith("out_proj.bias") or k.endswith("feed_forward.w2.weight"):
                m.w[k] = torch.zeros_like(m.w[k])
        toks = [(5 * i + 1) % vocab for i in range(9)]
        e = m.w["model.embed_tokens.weight"][toks]
        head = m.w["model.embed_tokens.weight"] if name == "A" else m.w["lm_head.weight"]
        want = torch.nn.functional.rms_norm(e, (e.shape[-1],), m.w["model.embedding_norm.weight"], m.eps) @ head.t()
        torch.testing.assert_close(m.logits(toks), want, rtol=1e-5, atol=1e-6)


def test_mixers_and_feed_forwards_read_the_normed_stream(plain_models):
    """Pre-norm: a block's mixer and feed-forward see rms_norm(x), so doubling
    the embedding table (with eps far below the rows' mean square) leaves the
    delta a part adds as it was: hidden(2 e) - hidden(e) = e. Post-norm, or a
    part fed the raw stream, would change its delta too. One part at a time,
    the other silenced, since the second part of a block sees the first's
    delta beside the stream."""
    import copy
    toks = [(11 * i + 2) % 256 for i in range(12)]
    for layer in (0, 1):                                  # a conv block, an attention block
        for silenced in ("feed_forward.w2.weight", "out_proj.weight"):
            m = copy.copy(plain_models["A"])
            m.w = dict(m.w)
            m.eps = 1e-12
            for k in list(m.w):
                if k.endswith(silenced):
                    m.w[k] = torch.zeros_like(m.w[k])
            e = m.w["model.embed_tokens.weight"][toks]
            h1 = m.hidden(toks, order=[(layer, None)])
            m.w["model.embed_tokens.weight"] = 2 * m.w["model.embed_tokens.weight"]
            h2 = m.hidden(toks, order=[(layer, None)])
            torch.testing.assert_close(h2 - h1, e, rtol=1e-4, atol=1e-6)
            assert (h1 - e).abs().max() > 1e-4          # and the part did add something, far above the tolerance


def test_a_conv_block_is_the_library_conv_between_two_gates(plain_models):
    """The conv mixer of Tiny B (biases on) from library routines: in_proj as
    F.linear, the depthwise causal conv with ITS bias as F.conv1d (so the bias
    lands on the conv's output, before the C gate), out_proj as F.linear."""
    F = torch.nn.functional
    m = plain_models["B"]
    g = torch.Generator().manual_seed(3)
    h = torch.randn(11, m.E, generator=g)
    p = "model.layers.0.conv."
    bcx = F.linear(h, m.w[p + "in_proj.weight"], m.w[p + "in_proj.bias"])
    B, C, x = bcx.split(m.E, dim=-1)                                   # in that order
    L = m.w[p + "conv.weight"].shape[-1]
    conv = F.conv1d(F.pad((B * x).t().unsqueeze(0), (L - 1, 0)), m.w[p + "conv.weight"], m.w[p + "conv.bias"],
                    groups=m.E)[0].t()
    want = F.linear(C * conv, m.w[p + "out_proj.weight"], m.w[p + "out_proj.bias"])
    torch.testing.assert_close(m.mixer_conv(0, h), want, rtol=1e-5, atol=1e-6)


def _attention_layer_input(m, layer, tokens, seed):
    """A normed input for one attention layer of a plain model, and its positions."""
    g = torch.Generator().manual_seed(seed)
    T = len(tokens)
    return torch.randn(T, m.E, generator=g), np.arange(T)


def test_values_are_not_normed_so_twice_the_values_give_twice_the_delta(plain_models):
    """/root/reference/crates/imparo-model/src/lfm2/workflow_cpu.rs:218-229 norms q and k per head and
    leaves v as projected. Doubling v_proj must then double the attention mixer's output, exactly (a
    power of two commutes with every rounding); a norm on v would swallow the factor."""
    import copy
    for name, layer in (("A", 1), ("B", 2)):
        m = copy.copy(plain_models[name])
        m.w = dict(m.w)
        h, pos = _attention_layer_input(m, layer, range(13), 4)
        once, (_, v1) = m.mixer_attention(layer, h, pos, None)
        key = f"model.layers.{layer}.self_attn.v_proj.weight"
        m.w[key] = 2 * m.w[key]
        twice, (_, v2) = m.mixer_attention(layer, h, pos, None)
        assert torch.equal(v2, 2 * v1)
        assert torch.equal(twice, 2 * once)
        assert once.abs().max() > 1e-4


def test_keys_and_queries_are_normed_so_their_projections_scale_away(plain_models):
    """workflow_cpu.rs:218-229: the RMS norm over each head of q and of k. With eps far below the heads'
    mean squares, three times k_proj (or q_proj) changes nothing; without the norm on k the scores
    would be three times as sharp and the logits would move."""
    import copy
    for name, vocab in (("A", 256), ("B", 384)):
        base = copy.copy(plain_models[name])
        base.w = dict(base.w)
        base.eps = 1e-12
        toks = [(13 * i + 5) % vocab for i in range(20)]
        want = base.logits(toks)
        for which in ("k_proj", "q_proj"):
            m = copy.copy(base)
            m.w = dict(base.w)
            for k in list(m.w):
                if k.endswith(f"self_attn.{which}.weight"):
                    m.w[k] = 3 * m.w[k]
            torch.testing.assert_close(m.logits(toks), want, rtol=1e-4, atol=1e-6)
        # the same factor on a weight that no norm follows does show: the test can fail
        m = copy.copy(base)
        m.w = dict(base.w)
        for k in list(m.w):
            if k.endswith("self_attn.v_proj.weight"):
                m.w[k] = 3 * m.w[k]
        assert (m.logits(toks) - want).abs().max() > 1e-3


def test_the_attention_mixer_is_library_attention_at_its_default_scale(plain_models):
    """workflow_cpu.rs:243 scales scores by 1/sqrt(head size), which is what
    F.scaled_dot_product_attention does when no scale is given. The mixer, from its projections to its
    output projection, against the library routine on the same normed and rotated q and k, the plain v,
    causal, each group of H/Hk neighbouring heads on one kv head (cpu_support.rs:402-445)."""
    F = torch.nn.functional
    for name, layer in (("A", 3), ("B", 4)):
        m = plain_models[name]
        T = 17
        h, pos = _attention_layer_input(m, layer, range(T), 9)
        p = f"model.layers.{layer}.self_attn."
        q = F.linear(h, m.w[p + "q_proj.weight"]).reshape(T, m.H, m.D)
        k = F.linear(h, m.w[p + "k_proj.weight"]).reshape(T, m.Hk, m.D)
        v = F.linear(h, m.w[p + "v_proj.weight"]).reshape(T, m.Hk, m.D)
        q = m.norm_and_rotate(q, m.w[p + "q_layernorm.weight"], pos)
        k = m.norm_and_rotate(k, m.w[p + "k_layernorm.weight"], pos)
        per_kv = m.H // m.Hk
        kk = k.repeat_interleave(per_kv, dim=1)
        vv = v.repeat_interleave(per_kv, dim=1)
        o = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True)
        want = F.linear(o.transpose(0, 1).reshape(T, m.H * m.D), m.w[p + "out_proj.weight"])
        got, _ = m.mixer_attention(layer, h, pos, None)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
        # another scale would show: scores of this size move the output far above the tolerance
        wrong = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                               is_causal=True, scale=1.0)
        assert (F.linear(wrong.transpose(0, 1).reshape(T, m.H * m.D), m.w[p + "out_proj.weight"]) - want
                ).abs().max() > 100 * (got - want).abs().max() + 1e-5


def test_a_block_adds_its_mixer_first_and_feeds_the_sum_to_the_feed_forward(plain_models):
    """workflow_cpu.rs:293-316: x1 = x + mixer(norm_a(x)); x2 = x1 + ffn(norm_b(x1)). One block of each
    kind, put together here from the part functions, equals what the model computes for that block; the
    other order (feed-forward first, the mixer on the sum) and the parallel form (both on x) do not."""
    for name, vocab in (("A", 256), ("B", 384)):
        m = plain_models[name]
        toks = [(3 * i + 7) % vocab for i in range(15)]
        e = m.w["model.embed_tokens.weight"][toks]
        kinds = m.cfg["layer_types"]
        for layer in (kinds.index("conv"), kinds.index("full_attention")):
            p = f"model.layers.{layer}."
            norm_a = lambda x: P.rms_norm(x, m.w[p + "operator_norm.weight"], m.eps)
            norm_b = lambda x: P.rms_norm(x, m.w[p + "ffn_norm.weight"], m.eps)
            ffn = lambda n: P.swiglu(n, m.w[p + "feed_forward.w1.weight"], m.w[p + "feed_forward.w3.weight"],
                                     m.w[p + "feed_forward.w2.weight"])
            if kinds[layer] == "conv":
                mixer = lambda h: m.mixer_conv(layer, h)
            else:
                mixer = lambda h: m.mixer_attention(layer, h, np.arange(len(toks)), None)[0]
            x1 = e + mixer(norm_a(e))
            want = x1 + ffn(norm_b(x1))
            got = m.hidden(toks, order=[(layer, None)])
            torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-7)
            f1 = e + ffn(norm_b(e))
            ffn_first = f1 + mixer(norm_a(f1))
            parallel = e + mixer(norm_a(e)) + ffn(norm_b(e))
            gap = (got - want).abs().max()
            assert (got - ffn_first).abs().max() > 1e-5 + 100 * gap
            assert (got - parallel).abs().max() > 1e-5 + 100 * gap
