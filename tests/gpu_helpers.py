"""Shared pieces of the GPU tests: engines, cached reference logits, a batch
context built by hand for tests of single kernels and parts."""
import functools
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch


def make_engine(model_dir, dtype, **kw):
    from imparo_amd.engine import Engine
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_requests", 8)
    return Engine(model_dir, dtype=dtype, **kw)


class RefCache:
    """Plain-implementation logits of whole sequences, computed once each."""

    def __init__(self, plain):
        self.plain = plain
        self._memo: Dict[Tuple, torch.Tensor] = {}

    def __call__(self, tokens, order=None) -> torch.Tensor:
        key = (tuple(tokens), None if order is None else tuple(order))
        if key not in self._memo:
            self._memo[key] = self.plain.logits(list(tokens), order)
        return self._memo[key]


def assert_picks_near_best(plain, prompt, generated, rel, what=""):
    """For runs whose rounding may turn a near-tie the other way (bfloat16): every generated
    token must be, in the plain implementation's logits of the same prefix, within `rel` of the
    largest logit magnitude below the best token. A token recomputed from a wrong prefix or a
    stale state misses by far more."""
    ref = plain.logits(list(prompt) + list(generated))
    scale = float(ref.abs().max())
    for i, tok in enumerate(generated):
        row = ref[len(prompt) - 1 + i]
        gap = float(row.max() - row[tok])
        assert gap <= rel * scale, f"{what}: token {i} ({tok}) lies {gap:.3g} below the best, allowed {rel * scale:.3g}"


def step_all(engine, rid, tokens, cuts: Sequence[int]) -> torch.Tensor:
    """Feeds `tokens` as request `rid` in portions of the sizes in `cuts`
    (repeated as needed), wanting every position; returns [T, V] on the CPU."""
    from imparo_amd.engine import StepEntry
    outs, at, i = [], 0, 0
    while at < len(tokens):
        n = min(cuts[i % len(cuts)], len(tokens) - at)
        outs.append(engine.step([StepEntry(rid, tokens[at:at + n], list(range(n)))]).cpu())
        at += n
        i += 1
    return torch.cat(outs)


def mixed_schedule(rng, lengths, max_live=4, sizes=(1, 1, 1, 2, 2, 3, 5, 9, 16, 40)):
    """A schedule of steps: each step gives some live requests a portion or
    one token. Returns [(step entries [(rid, lo, hi)], ends [rid])]."""
    waiting = list(range(len(lengths)))
    fed = {}
    steps = []
    while waiting or fed:
        while waiting and len(fed) < max_live and (not fed or rng.random() < 0.6):
            fed[waiting.pop(0)] = 0
        entries, ends = [], []
        for rid in sorted(fed):
            if rng.random() < 0.25 and len(fed) > 1:
                continue                                  # left out of this step, goes on later
            left = lengths[rid] - fed[rid]
            n = min(left, rng.choice(sizes))
            entries.append((rid, fed[rid], fed[rid] + n))
            fed[rid] += n
            if fed[rid] == lengths[rid]:
                ends.append(rid)
        for rid in ends:
            del fed[rid]
        if entries:
            steps.append((entries, ends))
    return steps


def peak_pages(steps, page_size: int) -> int:
    """The most pages a schedule of mixed_schedule holds at any time (a request
    holds ceil(fed / page_size) pages from its first step to its end)."""
    held, peak = {}, 0
    for entries, ends in steps:
        for rid, lo, hi in entries:
            held[rid] = -(-hi // page_size)
        peak = max(peak, sum(held.values()))
        for rid in ends:
            del held[rid]
    return peak


def hand_context(segments: Sequence[Tuple[int, int]], page_size: int, n_pages: int, dtype, device,
                 kv_sites: Dict[int, Tuple[int, int]] = None, fixed_sites: Dict[int, Tuple[int, ...]] = None,
                 n_slots: int = 8, tables: List[List[int]] = None, slots: List[int] = None,
                 v_transposed: bool = False):
    """A StepContext for rows given as (start position, number of tokens).
    kv_sites: site -> (kv_heads, head_dim); fixed_sites: site -> state shape.
    Pages are handed out in order unless `tables` gives them."""
    from imparo_amd.parts.base import StepContext, Workspace

    class Storage:
        pass
    st = Storage()
    st.paged, st.fixed = {}, {}
    for site, (hk, d) in (kv_sites or {}).items():
        v_shape = (n_pages, hk, d, page_size) if v_transposed else (n_pages, hk, page_size, d)
        st.paged[site] = dict(k=torch.zeros(n_pages, hk, page_size, d, dtype=dtype, device=device),
                              v=torch.zeros(v_shape, dtype=dtype, device=device))
    for site, shape in (fixed_sites or {}).items():
        st.fixed[site] = torch.zeros((n_slots,) + tuple(shape), dtype=torch.float32, device=device)
    R = len(segments)
    pos, row, start, length = [], [], [], []
    t = 0
    for r, (p0, n) in enumerate(segments):
        pos += list(range(p0, p0 + n))
        row += [r] * n
        start.append(t)
        length.append(n)
        t += n
    if tables is None:
        tables, nxt = [], 0
        for p0, n in segments:
            k = (p0 + n + page_size - 1) // page_size
            tables.append(list(range(nxt, nxt + k)))
            nxt += k
        assert nxt <= n_pages
    P = max(len(tb) for tb in tables)
    tab = np.full((R, P), -1, dtype=np.int32)
    for r, tb in enumerate(tables):
        tab[r, :len(tb)] = tb
    i32 = lambda a: torch.tensor(np.asarray(a, dtype=np.int32), device=device)
    ctx = StepContext(
        n_tokens=t, n_rows=R, positions=i32(pos), row_of_token=i32(row), seg_start=i32(start),
        seg_len=i32(length), slot=i32(slots if slots is not None else list(range(R))),
        block_tables={0: i32(tab)}, page_size=page_size, dtype=dtype, workspace=Workspace(device),
        storage=st, group_of_site={s: 0 for s in (kv_sites or {})},
        max_seg_len=max(length), max_context=max(p0 + n for p0, n in segments), host_seg_len=list(length))
    dec = [r for r, n in enumerate(length) if n == 1]
    pre = [r for r, n in enumerate(length) if n > 1]
    lists = i32(dec + pre)
    ctx.single_rows, ctx.n_single_rows = lists[:len(dec)], len(dec)
    ctx.portion_rows, ctx.n_portion_rows = lists[len(dec):], len(pre)
    return ctx
