"""Command line, in the manner of the reference's tools.

  forward   explicit token ids in, top logits out, with the reference's
            instruments: --repeat, --decode, --split, --cobatch, --scramble-kv
            (/root/reference/crates/imparo-model/src/bin/imparo-forward.rs:1036-1186)
  generate  continuous batching over prompts given as ids; -m/--model,
            -c/--ctx, -np/--parallel as the reference's server spells them
            (/root/reference/crates/imparo-server/src/main.rs:181-231);
            --max-tokens and --temperature are its request fields (:1849-1872)
  random    a configuration and a seed -> a model folder
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _fnv1a(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for b in data:
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def _top10(row) -> str:
    import torch
    vals, idx = torch.topk(row, min(10, row.shape[0]))
    return " ".join(f"{int(i)}:{float(v):.4f}" for v, i in zip(vals, idx))


def _pool_sizing(a, default_tokens: int) -> dict:
    """How the cache pools are sized: --num-pages, --kv-gb, or enough for the run."""
    if a.num_pages is not None and a.kv_gb is not None:
        raise SystemExit("give one of --num-pages and --kv-gb")
    if a.num_pages is not None:
        return dict(num_pages=a.num_pages)
    if a.kv_gb is not None:
        return dict(kv_budget_bytes=int(a.kv_gb * (1 << 30)))
    return dict(max_tokens=default_tokens)


def cmd_forward(a) -> int:
    import torch
    from .engine import Engine, StepEntry
    from .kernels import ops
    tokens = [int(t) for t in a.tokens]
    cap = a.ctx or (len(tokens) + a.decode + 64)
    n_conv = max(1, a.cobatch)
    sizing = _pool_sizing(a, (cap // a.page_size + 2) * a.page_size * n_conv)
    eng = Engine(a.model, dtype=a.dtype, page_size=a.page_size, max_requests=max(2, n_conv),
                 max_step_tokens=max(len(tokens) * n_conv, 1), **sizing)

    def argmax(row) -> int:
        out = torch.empty(1, dtype=torch.int32, device=row.device)
        return int(ops.argmax_rows(row.view(1, -1), out).cpu()[0])

    def run_once(cuts: List[int], tag: str):
        """Prompt in portions cut at `cuts`, then --decode greedy steps."""
        bounds = [0] + [c for c in cuts if 0 < c < len(tokens)] + [len(tokens)]
        logits = None
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            logits = eng.step([StepEntry(tag, tokens[lo:hi], [hi - lo - 1] if hi == len(tokens) else [])])
        final = logits[0].clone()
        trail, hashes = [], []
        row = final
        for _ in range(a.decode):
            nxt = argmax(row)
            trail.append(nxt)
            row = eng.step([StepEntry(tag, [nxt], [0])])[0]
            hashes.append(_fnv1a(row.cpu().numpy().tobytes()))
        eng.release(tag)
        return final, trail, hashes

    status = 0
    if a.cobatch:
        # B conversations: the prompt cut to B lengths, decoded alone then together
        B = a.cobatch
        lens = [max(1, len(tokens) * (i + 1) // B) for i in range(B)]
        alone = []
        for i, n in enumerate(lens):
            row = eng.step([StepEntry(f"alone{i}", tokens[:n], [n - 1])])[0]
            rows = []
            for _ in range(a.decode):
                nxt = argmax(row)
                row = eng.step([StepEntry(f"alone{i}", [nxt], [0])])[0].clone()
                rows.append((nxt, row))
            alone.append(rows)
            eng.release(f"alone{i}")
        first = eng.step([StepEntry(f"co{i}", tokens[:n], [n - 1]) for i, n in enumerate(lens)])
        cur = [argmax(first[i]) for i in range(B)]
        worst = 0.0
        for s in range(a.decode):
            out = eng.step([StepEntry(f"co{i}", [cur[i]], [0]) for i in range(B)])
            for i in range(B):
                nxt, ref = alone[i][s]
                if nxt != cur[i]:
                    print(f"cobatch: row {i} step {s}: token {cur[i]} together, {nxt} alone")
                    status = 1
                worst = max(worst, float((out[i] - ref).abs().max()))
            cur = [argmax(out[i]) for i in range(B)]
        print(f"cobatch {B} rows x {a.decode} steps: max |logit delta| together vs alone = {worst:.3e}")
        return status

    series = a.split if a.split else [0]
    base = None
    for rep in range(max(a.repeat, 1)):
        for cut in (series if len(series) > 1 else [series[0]]):
            final, trail, hashes = run_once([cut] if cut else [], f"rep{rep}")
            print(f"rep {rep} split {cut}: top10 {_top10(final)}")
            if a.decode:
                print(f"  trail {' '.join(map(str, trail))}")
                print(f"  hash {_fnv1a(b''.join(h.to_bytes(8, 'little') for h in hashes)):016x}")
            if base is None:
                base = (final, trail)
            else:
                delta = float((final - base[0]).abs().max())
                print(f"  max |delta| to the first run: {delta:.3e}")
                if trail != base[1]:
                    status = 1
    if a.scramble_kv:
        eng2 = Engine(a.model, dtype=a.dtype, page_size=a.page_size, max_requests=2,
                      max_step_tokens=max(len(tokens), 1), **_pool_sizing(a, (cap // a.page_size + 2) * a.page_size))
        eng2.cache.scramble(seed=1)
        row = eng2.step([StepEntry("s", tokens, [len(tokens) - 1])])[0]
        delta = float((row - base[0]).abs().max())
        print(f"scramble-kv: max |delta| to identity placement: {delta:.3e}")
        status = status or int(delta != 0.0)
    return status


def cmd_generate(a) -> int:
    from .engine.scheduler import generate
    prompts = [_ids(p) for p in a.input_ids]
    t0 = time.time()
    out = generate(a.model, prompts, max_tokens=a.max_tokens, temperature=a.temperature, seed=a.seed,
                   stop_token_ids=None if a.stop_token_ids is None else _ids(a.stop_token_ids),
                   dtype=a.dtype, ctx=a.ctx, parallel=a.parallel, max_batch_tokens=a.max_batch_tokens,
                   page_size=a.page_size, num_pages=a.num_pages,
                   kv_budget_bytes=None if a.kv_gb is None else int(a.kv_gb * (1 << 30)))
    dt = time.time() - t0
    for i, ids in enumerate(out):
        print(json.dumps({"index": i, "output_ids": ids}))
    n = sum(len(o) for o in out)
    print(f"[imparo] {n} tokens in {dt:.3f} s ({n / dt:.1f} tok/s incl. load)", file=sys.stderr)
    return 0


def cmd_random(a) -> int:
    import torch
    from .weights import write_random_model
    with open(a.config) as f:
        cfg = json.load(f)
    write_random_model(cfg, a.seed, a.out, dtype=torch.float32 if a.store == "float32" else torch.bfloat16)
    print(a.out)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="imparo_amd", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)

    def common(p):
        p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
        p.add_argument("-c", "--ctx", type=int, default=None, help="most tokens one request may hold")
        p.add_argument("--page-size", type=int, default=64)
        p.add_argument("--num-pages", type=int, default=None,
                       help="pages in every cache pool (a small number makes requests wait or be recomputed)")
        p.add_argument("--kv-gb", type=float, default=None, help="memory for the paged caches, in GiB")

    f = sub.add_parser("forward", help="run explicit token ids and print top logits")
    common(f)
    f.add_argument("--repeat", type=int, default=1, help="run the same forward N times (determinism)")
    f.add_argument("--decode", type=int, default=0, help="then N greedy single-token steps; prints the trail")
    f.add_argument("--split", type=lambda s: [int(x) for x in s.split(",")], default=None,
                   help="K[,K2...]: prefix up to K first, then the tail; 0 is the cold forward")
    f.add_argument("--cobatch", type=int, default=0, help="B conversations alone, then together (needs --decode)")
    f.add_argument("--scramble-kv", action="store_true", help="repeat with permuted page placement and compare")
    f.add_argument("model")
    f.add_argument("tokens", nargs="+")
    f.set_defaults(fn=cmd_forward)

    g = sub.add_parser("generate", help="generate from prompts given as token ids")
    common(g)
    g.add_argument("-m", "--model", required=True)
    g.add_argument("-np", "--parallel", type=int, default=64, help="requests that decode at once")
    g.add_argument("--input-ids", action="append", required=True, help="one prompt: ids separated by commas or spaces")
    g.add_argument("--max-tokens", type=int, default=16)
    g.add_argument("--temperature", type=float, default=0.0)
    g.add_argument("--seed", type=int, default=0)
    g.add_argument("--stop-token-ids", default=None,
                   help='ids that end a reply unsent, e.g. "7,2" ("" for none; default: the model\'s eos_token_id)')
    g.add_argument("--max-batch-tokens", type=int, default=2048, help="token budget of one step")
    g.set_defaults(fn=cmd_generate)

    r = sub.add_parser("random", help="write a model folder with random weights")
    r.add_argument("--config", required=True, help="a config.json to take the sizes from")
    r.add_argument("--seed", type=int, default=0)
    r.add_argument("--out", required=True)
    r.add_argument("--store", default="bfloat16", choices=["bfloat16", "float32"])
    r.set_defaults(fn=cmd_random)

    a = ap.parse_args(argv)
    if a.cmd == "forward" and a.cobatch and not a.decode:
        ap.error("--cobatch follows --decode N")
    return a.fn(a)
