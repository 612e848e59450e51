#!/usr/bin/env python3
"""Benchmark: decode tokens per second of the LFM2-1.2B shape on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the whole batch through the engine's own loop, as
generation runs it: step function, sampling kernel, the sampled tokens fed to
the next step on the device and read back by the host one step late (while the
GPU runs that next step).
Default: batch 8, every request's context ending at 4096 tokens, random
bfloat16 weights (seed 2), synthetic token ids uniform over the vocabulary.
The JSON line also carries a 2,048-token prefill, the decode step's HBM
roofline, and decode at batch 1 and 64. Every figure is the median of three
measurements taken in turn.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

LFM2_1_2B = dict(
    architectures=["Lfm2ForCausalLM"], model_type="lfm2", vocab_size=65536, hidden_size=2048,
    num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
    layer_types=["full_attention" if i in (2, 5, 8, 10, 12, 14) else "conv" for i in range(16)],
    block_auto_adjust_ff_dim=True, block_ff_dim=12288, block_multiple_of=256, block_ffn_dim_multiplier=1.0,
    conv_L_cache=3, conv_bias=False, rope_theta=1000000.0, tie_embedding=True, norm_eps=1e-5,
    max_position_embeddings=128000,
)


def model_numbers(cfg):
    """Matrix parameters per token (layers, head) and cache bytes per token, from the configuration."""
    from imparo_amd.config import Lfm2Config
    c = Lfm2Config.from_dict(cfg)
    E, F, D, H, Hk, L = c.hidden_size, c.ff_dim, c.head_dim, c.num_attention_heads, c.num_key_value_heads, c.conv_L_cache
    n_attn = sum(t != "conv" for t in c.layer_types)
    n_conv = len(c.layer_types) - n_attn
    attn = (H + 2 * Hk) * D * E + E * H * D
    conv = 3 * E * E + E * E
    ffn = 3 * E * F
    layer_params = n_attn * (attn + ffn) + n_conv * (conv + ffn)
    head_params = c.vocab_size * E
    return dict(cfg=c, layer_params=layer_params, head_params=head_params, n_attn=n_attn, n_conv=n_conv,
                kv_bytes_per_token=n_attn * 2 * Hk * D * 2, conv_state_bytes=n_conv * (L - 1) * E * 4,
                attn_flops_per_pair=n_attn * 4 * H * D)


def decode_run(engine, sampler, batch, context, steps, warmup, vocab, seed):
    """Fills `batch` requests up to context - steps - warmup tokens, then times `steps` decode steps."""
    import torch
    from imparo_amd.engine import DeviceToken, StepEntry
    g = torch.Generator().manual_seed(seed)
    start = context - steps - warmup
    ids = [f"d{i}" for i in range(batch)]
    last = None
    for i, rid in enumerate(ids):                      # prompts in 2,048-token portions
        prompt = torch.randint(0, vocab, (start,), generator=g).tolist()
        for lo in range(0, start, 2048):
            hi = min(start, lo + 2048)
            out = engine.step([StepEntry(rid, prompt[lo:hi], [hi - lo - 1] if hi == start else [])])
        last = out.clone() if last is None else torch.cat([last, out])
    temps, unis = [0.0] * batch, [0.0] * batch
    picked = sampler.pick_async(last, temps, unis)

    def one_step(picked):
        logits = engine.step([StepEntry(rid, [DeviceToken(picked.on_device, i)], [0]) for i, rid in enumerate(ids)])
        following = sampler.pick_async(logits, temps, unis)
        picked.tokens()                                # the step before's tokens, read while this one runs
        return following

    for _ in range(warmup):
        picked = one_step(picked)
    picked.tokens()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        picked = one_step(picked)
    picked.tokens()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    for rid in ids:
        engine.release(rid)
    return dt


def prefill_run(engine, tokens, vocab, reps, seed):
    """Seconds of each of `reps` whole prompts of `tokens` tokens (one step each, fresh tokens each time)."""
    import torch
    from imparo_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    times = []
    for r in range(reps + 1):
        prompt = torch.randint(0, vocab, (tokens,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry("p", prompt, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        engine.release("p")
        if r > 0:                                      # the first run sizes the workspace
            times.append(dt)
    return times


def small_steps(engine, vocab, seed):
    """Steps whose kernels take about as long as a caller needs to issue them: eight decoding
    requests beside a 32-token portion of a prompt, and a 128-token prompt alone; neither is a
    captured graph. For each: `ms`, a step as the engine runs it, one after the other; `gpu_ms`, its
    kernels back to back (the step is queued while the GPU is still busy with something else, then
    timed between two events); `host_ms`, what the host needs to check, pack and issue it when the
    GPU is idle. A step is bound by the host where ms is well above gpu_ms."""
    import torch
    from imparo_amd.engine import StepEntry
    g = torch.Generator().manual_seed(seed)
    draw = lambda n: torch.randint(0, vocab, (n,), generator=g).tolist()
    busy_a = torch.randn(4096, 4096, device=engine.device, dtype=torch.bfloat16)

    def keep_gpu_busy():                       # a few milliseconds of work that has nothing to do with the step
        for _ in range(24):
            torch.mm(busy_a, busy_a)

    def measure(make_step, after_step, reps=12):
        for _ in range(3):
            make_step()
            after_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            make_step()
            after_step()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) / reps
        gpu, host = [], []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            make_step()
            host.append(time.perf_counter() - t0)
            after_step()
            keep_gpu_busy()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            make_step()
            e1.record()
            after_step()
            torch.cuda.synchronize()
            gpu.append(e0.elapsed_time(e1) * 1e-3)
        return {"ms": round(wall * 1e3, 4), "gpu_ms": round(median(gpu) * 1e3, 4), "host_ms": round(median(host) * 1e3, 4)}

    out = {}
    ids = [f"s{i}" for i in range(8)]
    for rid in ids:
        engine.step([StepEntry(rid, draw(600), [])])
    portion = draw(32)

    def mixed():
        engine.step([StepEntry(rid, [7], [0]) for rid in ids] + [StepEntry("sp", portion, [31])])

    def mixed_after():
        if engine.length("sp") >= 1024:
            engine.release("sp")
        if engine.length(ids[0]) >= 1500:
            for rid in ids:
                engine.release(rid)
                engine.step([StepEntry(rid, draw(600), [])])

    out["mixed_small"] = dict(measure(mixed, mixed_after), decode_rows=8, portion_tokens=32)
    for rid in ids + ["sp"]:
        engine.release(rid)
    prompt = draw(128)
    out["prefill_128"] = dict(measure(lambda: engine.step([StepEntry("s128", prompt, [127])]),
                                      lambda: engine.release("s128")), tokens=128)
    return out


def median(xs):
    xs = sorted(xs)
    n = len(xs)
    return xs[n // 2] if n % 2 else 0.5 * (xs[n // 2 - 1] + xs[n // 2])


def percentile(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(q * len(xs)))]


def shape(hidden, heads, block_ff_dim):
    """The layer sizes of the smaller LFM2 checkpoints: same layout as the 1.2B, other widths."""
    cfg = dict(LFM2_1_2B)
    cfg.update(hidden_size=hidden, num_attention_heads=heads, block_ff_dim=block_ff_dim)
    return cfg


LFM2_700M = shape(1536, 24, 10240)
LFM2_350M = shape(1024, 16, 6656)


def build_engine(cfg, seed, dtype, **kw):
    """Random weights of `cfg` drawn from `seed`, written to a temporary folder, loaded, and the folder removed."""
    from imparo_amd import write_random_model
    from imparo_amd.engine import Engine
    tmp = tempfile.mkdtemp(prefix="imparo_bench_")
    try:
        write_random_model(cfg, seed, tmp)
        return Engine(tmp, dtype=dtype, page_size=64, **kw)
    finally:
        for f in os.listdir(tmp):
            os.remove(os.path.join(tmp, f))
        os.rmdir(tmp)


class StepClock:
    """Stands between the scheduler and the engine and notes, for every step, what it fed and a GPU
    event at its start: the time from one step's event to the next is that step's time on the GPU
    (the host runs a step ahead, so nothing waits for the notes)."""

    def __init__(self, engine, weight_bytes, head_bytes, kv_bytes_per_token, flops_per_token):
        self._engine = engine
        self._held = {}                  # request -> tokens in the cache
        self.notes = []                  # (event, decode rows, prompt tokens, bytes to read, flops)
        self._sizes = (weight_bytes, head_bytes, kv_bytes_per_token, flops_per_token)

    def __getattr__(self, name):
        return getattr(self._engine, name)

    def step(self, entries):
        import torch
        weight_bytes, head_bytes, kv_bytes, flops_per_token = self._sizes
        rows = sum(1 for e in entries if len(e.tokens) == 1)
        fed = sum(len(e.tokens) for e in entries)
        for e in entries:
            self._held[e.request] = self._held.get(e.request, 0) + len(e.tokens)
        # every weight once (the head only if a row asks for logits), the cache of the requests in the step
        to_read = (weight_bytes + (head_bytes if any(e.want for e in entries) else 0)
                   + kv_bytes * sum(self._held[e.request] for e in entries))
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        self.notes.append((ev, rows, fed - rows, to_read, flops_per_token * fed))
        return self._engine.step(entries)

    def release(self, request_id):
        self._held.pop(request_id, None)
        return self._engine.release(request_id)

    def by_kind(self, hbm_peak_gbs, flops_peak):
        """Step times by what a step fed: single tokens only, or portions of prompts as well."""
        import torch
        end = torch.cuda.Event(enable_timing=True)
        end.record()
        torch.cuda.synchronize()
        events = [n[0] for n in self.notes] + [end]
        kinds = {"decode_only": [], "mixed": []}
        for i, (_, rows, prompt_tokens, to_read, flops) in enumerate(self.notes):
            ms = events[i].elapsed_time(events[i + 1])
            kinds["mixed" if prompt_tokens else "decode_only"].append((ms, rows, prompt_tokens, to_read, flops))
        out = {}
        for kind, steps in kinds.items():
            if not steps:
                continue
            times = [t[0] for t in steps]
            out[kind] = {
                "steps": len(steps), "p50_ms": round(percentile(times, 0.5), 3), "p90_ms": round(percentile(times, 0.9), 3),
                "max_ms": round(max(times), 3), "mean_rows": round(sum(t[1] for t in steps) / len(steps), 1),
                "mean_prompt_tokens": round(sum(t[2] for t in steps) / len(steps), 1),
                # what the step had to read / its time / the HBM peak; what it had to compute / its time / the MFMA peak
                "hbm_frac_p50": round(percentile([t[3] / (t[0] * 1e-3) / 1e9 / hbm_peak_gbs for t in steps], 0.5), 4),
                "mfma_frac_p50": round(percentile([t[4] / (t[0] * 1e-3) / flops_peak for t in steps], 0.5), 4),
            }
        return out


def serving_workload(dtype, engine=None):
    """Continuous batching: 32 requests, prompts of 64..3072 tokens, replies of 32..512 tokens, in 4
    waves of 8 (a wave every 48 steps), 512-token portions beside decoded tokens. LFM2-700M shape.
    The decode steps' graphs are captured before the clock starts (Scheduler.warm), as a server
    would do at start-up. Returns the record."""
    import numpy as np
    import torch
    from imparo_amd.engine.scheduler import Scheduler
    from imparo_amd.sampling import Sampler, SamplingParams
    cfg = LFM2_700M
    nums = model_numbers(cfg)
    elem = 2 if dtype == "bfloat16" else 4
    if engine is None:
        engine = build_engine(cfg, 3, dtype, max_tokens=32 * (3072 + 512 + 64), max_requests=32)
    engine = StepClock(engine, nums["layer_params"] * elem, nums["head_params"] * elem,
                       nums["kv_bytes_per_token"] * elem // 2, 2.0 * nums["layer_params"])
    sampler = Sampler(engine.device)
    rng = np.random.default_rng(3)
    jobs = [(i, rng.integers(0, cfg["vocab_size"], size=int(rng.integers(64, 3073))).tolist(), int(rng.integers(32, 513)))
            for i in range(32)]
    sched = Scheduler(engine, sampler.pick, max_batch_tokens=2048, max_running=32, portion=512,
                      pick_async=sampler.pick_async)
    t_warm = time.perf_counter()
    warmed = sched.warm(3072 + 512)
    torch.cuda.synchronize()
    t_warm = time.perf_counter() - t_warm
    t0 = time.perf_counter()
    steps = 0
    while jobs or sched.has_work():
        if jobs and steps % 48 == 0:
            for i, prompt, n in jobs[:8]:
                sched.add(i, prompt, SamplingParams(max_tokens=n, stop_token_ids=()))
            jobs = jobs[8:]
        sched.step()
        steps += 1
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    done = sched.finished
    n_prompt = sum(len(r.prompt) for r in done.values())
    n_out = sum(len(r.generated) for r in done.values())
    assert len(done) == 32 and all(r.finish_reason == "length" for r in done.values())
    c = nums["cfg"]
    return {
        "metric": "continuous batching, LFM2-700M shape: generated tok/s over the whole run", "value": round(n_out / dt, 1),
        "unit": "tok/s", "n_gpus": 1, "seconds": round(dt, 3), "steps": steps, "prompt_tokens": n_prompt,
        "generated_tokens": n_out, "all_tokens_per_s": round((n_prompt + n_out) / dt, 1),
        "preemptions": sum(r.preemptions for r in done.values()), "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, random weights (seed 3)",
        "graphs_captured_before_the_clock": warmed, "seconds_to_capture_them": round(t_warm, 3),
        "step_times": engine.by_kind(HBM_PEAK_GBS, MFMA_PEAK["bf16" if dtype == "bfloat16" else "fp32"]),
        "config": {"model": "LFM2-700M shape", "requests": 32, "waves": 4, "portion": 512, "max_batch_tokens": 2048,
                   "hidden_size": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "ff_dim": c.ff_dim, "layers": c.num_hidden_layers}}


def long_workload(dtype, requests, prompt_len, portion=2048, quiet=False, engine=None):
    """Long contexts: `requests` concurrent requests, each a prompt of `prompt_len` tokens fed in
    portions of `portion` tokens (2,048), then 128 decoded tokens each. LFM2-350M shape. Returns the record."""
    import torch
    from imparo_amd.engine import DeviceToken, StepEntry
    from imparo_amd.sampling import Sampler
    cfg = LFM2_350M
    if engine is None:
        engine = build_engine(cfg, 4, dtype, max_tokens=requests * (prompt_len + 128 + 64), max_requests=requests)
    sampler = Sampler(engine.device)
    g = torch.Generator().manual_seed(4)
    ids = list(range(requests))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    last = []
    for rid in ids:
        prompt = torch.randint(0, cfg["vocab_size"], (prompt_len,), generator=g).tolist()
        out = None
        for lo in range(0, prompt_len, portion):
            hi = min(prompt_len, lo + portion)
            out = engine.step([StepEntry(rid, prompt[lo:hi], [hi - lo - 1] if hi == prompt_len else [])])
        last.append(out.clone())                   # (the engine's next step writes its logits where these lie)
        if rid % 8 == 7 and not quiet:
            print(f"[bench] {rid + 1} of {requests} prompts are in the cache", file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    zeros = [0.0] * requests
    picked = sampler.pick_async(torch.cat(last), zeros, zeros)
    for _ in range(128 - 1):
        logits = engine.step([StepEntry(rid, [DeviceToken(picked.on_device, i)], [0]) for i, rid in enumerate(ids)])
        following = sampler.pick_async(logits, zeros, zeros)
        picked.tokens()
        picked = following
    picked.tokens()
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    pages_used = engine.cache.groups[0].pool.n_pages - engine.free_pages()[0]
    for rid in ids:
        engine.release(rid)
    nums = model_numbers(cfg)
    step_bytes = ((nums["layer_params"] + nums["head_params"]) * 2
                  + requests * ((prompt_len + 64) * nums["kv_bytes_per_token"] + nums["conv_state_bytes"]))
    return {
        "metric": "long contexts, LFM2-350M shape: decode tok/s with every request at its full context",
        "value": round(requests * 127 / (t2 - t1), 1), "unit": "tok/s", "n_gpus": 1,
        "prefill_tok_s": round(requests * prompt_len / (t1 - t0), 1), "prefill_seconds": round(t1 - t0, 3),
        "decode_ms_per_step": round((t2 - t1) / 127 * 1e3, 3),
        "decode_hbm_frac": round(step_bytes / ((t2 - t1) / 127) / 1e9 / HBM_PEAK_GBS, 4),
        "dtype": "bf16" if dtype == "bfloat16" else "fp32",
        "data": "synthetic token ids, random weights (seed 4)",
        "config": {"model": "LFM2-350M shape", "requests": requests, "prompt_len": prompt_len, "portion": portion,
                   "decode_tokens": 128, "hidden_size": 1024, "heads": 16, "kv_heads": 8, "ff_dim": 4608, "layers": 16,
                   "cache_pages_used": pages_used}}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64 and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="run only the 2,048-token prefill (for profiling)")
    ap.add_argument("--workload", default="decode", choices=["decode", "serving", "long"],
                    help="decode: the headline line (default). serving: continuous batching of 32 requests in 4 "
                         "waves (LFM2-700M shape). long: 64 requests of 32,768-token prompts, then 128 tokens "
                         "each (LFM2-350M shape). The last two print a line of their own")
    ap.add_argument("--requests", type=int, default=64, help="--workload long: concurrent requests")
    ap.add_argument("--prompt-len", type=int, default=32768, help="--workload long: tokens per prompt")
    ap.add_argument("--portion", type=int, default=2048, help="--workload long: tokens of a prompt per step")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.workload == "serving":
        print(json.dumps(serving_workload(args.dtype)), flush=True)
        return 0
    if args.workload == "long":
        print(json.dumps(long_workload(args.dtype, args.requests, args.prompt_len, args.portion)), flush=True)
        return 0

    import torch
    from imparo_amd.sampling import Sampler

    cfg = dict(LFM2_1_2B)
    full_layers = cfg["num_hidden_layers"]
    if args.layers is not None and args.layers < full_layers:
        cfg["num_hidden_layers"] = args.layers
        cfg["layer_types"] = cfg["layer_types"][:args.layers]
    nums = model_numbers(cfg)
    c = nums["cfg"]
    print(f"[bench] writing random weights ({(nums['layer_params'] + nums['head_params']) / 1e9:.2f} B parameters) ...",
          file=sys.stderr, flush=True)
    further = not (args.no_points or args.prefill_only)
    # the pools hold the largest point: 256 requests at the context (which also holds 8 at 32,768)
    biggest = max(args.batch, 256 if further else 1)
    engine = build_engine(cfg, 2, args.dtype, max_tokens=biggest * (args.context + 64), max_requests=biggest,
                          max_step_tokens=32768 if further else 8192)
    sampler = Sampler(engine.device)
    elem = 2 if args.dtype == "bfloat16" else 4
    peak = MFMA_PEAK["bf16" if args.dtype == "bfloat16" else "fp32"]
    if args.prefill_only:
        pts = prefill_run(engine, 2048, c.vocab_size, 5, 3)
        print(json.dumps({"prefill_ms": round(median(pts) * 1e3, 3), "tokens": 2048,
                          "all_ms": [round(t * 1e3, 3) for t in pts]}), flush=True)
        return 0

    def step_bytes(batch, steps, context=None):
        """Bytes one decode step has to read: every weight once, the cache of the live requests."""
        mean_ctx = (context or args.context) - steps / 2
        return ((nums["layer_params"] + nums["head_params"]) * elem
                + batch * (mean_ctx * nums["kv_bytes_per_token"] * elem / 2 + nums["conv_state_bytes"]))

    def prefill_flops(T):
        return 2.0 * T * nums["layer_params"] + 2.0 * nums["head_params"] + nums["attn_flops_per_pair"] * T * (T + 1) / 2

    # Every figure of the headline and of the points at batch 1 and 64 is the median of PASSES measurements
    # taken in turn (batch 8, batch 1, batch 64, prefill, and again), so that a slow moment of the machine
    # does not fall on one of them alone. A decode measurement is W warmup steps and exactly K timed steps,
    # each time on freshly filled contexts.
    PASSES = 3
    points_steps = max(8, args.steps // 2)
    widths = [args.batch] + ([] if args.no_points else [b for b in (1, 64) if b != args.batch])
    seconds = {b: [] for b in widths}
    prefills = []
    T = 2048
    for p in range(PASSES):
        for b in widths:
            k = args.steps if b == args.batch else points_steps
            w = args.warmup if b == args.batch else 4
            print(f"[bench] pass {p + 1} of {PASSES}: decode at batch {b} ...", file=sys.stderr, flush=True)
            seconds[b].append(decode_run(engine, sampler, b, args.context, k, w, c.vocab_size, 2 + 100 * p + b))
        if not args.no_points:
            print(f"[bench] pass {p + 1} of {PASSES}: prefill of {T} tokens ...", file=sys.stderr, flush=True)
            prefills += prefill_run(engine, T, c.vocab_size, 2, 3 + p)
    dt = median(seconds[args.batch])
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    achieved = step_bytes(args.batch, args.steps) / (dt / args.steps) / 1e9
    line = {
        "metric": f"decode tok/s (LFM2-1.2B shape, batch {args.batch}, context {args.context})",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic token ids, random weights (seed 2)",
        "config": {
            "model": "LFM2-1.2B shape", "global_batch": args.batch, "seq_len": args.context, "parallelism": "single GPU",
            "layers": c.num_hidden_layers, "layers_full": full_layers,
            "attention_layers": nums["n_attn"], "conv_layers": nums["n_conv"],
            "hidden_size": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
            "head_dim": c.head_dim, "ff_dim": c.ff_dim, "vocab_size": c.vocab_size, "conv_L_cache": c.conv_L_cache,
            "tie_embedding": c.tie_embedding, "page_size": engine.page_size, "decode_tokens": args.steps + args.warmup,
        },
        "passes": PASSES, "ms_per_step_of_each_pass": [round(t / args.steps * 1e3, 4) for t in seconds[args.batch]],
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        pt = median(prefills)
        line["prefill"] = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                           "frac": round(prefill_flops(T) / pt / peak, 4), "runs": len(prefills),
                           "min_ms": round(min(prefills) * 1e3, 3), "max_ms": round(max(prefills) * 1e3, 3)}
        points = {}

        def decode_point(name, b, k, d, context=None):
            points[name] = round(b * k / d, 1)
            points[name + "_ms_per_step"] = round(d / k * 1e3, 4)
            points[name + "_frac"] = round(step_bytes(b, k, context) / (d / k) / 1e9 / HBM_PEAK_GBS, 4)

        for b in (1, 64):
            decode_point(f"decode_b{b}", b, args.steps if b == args.batch else points_steps, median(seconds[b]))
        # further sizes, one measurement each: larger batches, a long context, longer prompts
        for b in (128, 256):
            print(f"[bench] decode at batch {b} ...", file=sys.stderr, flush=True)
            decode_point(f"decode_b{b}", b, points_steps, decode_run(engine, sampler, b, args.context, points_steps, 4,
                                                                      c.vocab_size, 900 + b))
        print("[bench] decode at batch 8, context 32768 ...", file=sys.stderr, flush=True)
        decode_point("decode_b8_ctx32768", 8, points_steps,
                     decode_run(engine, sampler, 8, 32768, points_steps, 4, c.vocab_size, 33), context=32768)
        for tokens in (8192, 32768):
            print(f"[bench] prefill of {tokens} tokens ...", file=sys.stderr, flush=True)
            t = median(prefill_run(engine, tokens, c.vocab_size, 2, 40 + tokens))
            points[f"prefill_{tokens}"] = {"value": round(tokens / t, 1), "ms": round(t * 1e3, 3),
                                           "frac": round(prefill_flops(tokens) / t / peak, 4)}
        print("[bench] steps of a few dozen tokens ...", file=sys.stderr, flush=True)
        points.update(small_steps(engine, c.vocab_size, 5))
        del engine
        torch.cuda.empty_cache()
        points.update(smaller_shapes(args.dtype, points_steps))
        line["points"] = points
    print(json.dumps(line), flush=True)
    return 0


def smaller_shapes(dtype, steps):
    """The two smaller checkpoints' shapes, compact: a decode step at batch 8 and context 4096 with its
    share of the HBM peak, the continuous-batching workload (700M) and four 32,768-token requests (350M)."""
    import torch
    from imparo_amd.sampling import Sampler
    out = {}
    elem = 2 if dtype == "bfloat16" else 4
    for name, cfg, seed in (("lfm2_700m", LFM2_700M, 3), ("lfm2_350m", LFM2_350M, 4)):
        print(f"[bench] the {name} shape ...", file=sys.stderr, flush=True)
        nums = model_numbers(cfg)
        tokens = 32 * (3072 + 512 + 64) if name == "lfm2_700m" else 4 * (32768 + 128 + 64)
        engine = build_engine(cfg, seed, dtype, max_tokens=tokens, max_requests=32)
        d = decode_run(engine, Sampler(engine.device), 8, 4096, steps, 4, cfg["vocab_size"], 71)
        to_read = ((nums["layer_params"] + nums["head_params"]) * elem
                   + 8 * ((4096 - steps / 2) * nums["kv_bytes_per_token"] * elem / 2 + nums["conv_state_bytes"]))
        out[f"decode_b8_{name}_ms_per_step"] = round(d / steps * 1e3, 4)
        out[f"decode_b8_{name}_frac"] = round(to_read / (d / steps) / 1e9 / HBM_PEAK_GBS, 4)
        if name == "lfm2_700m":
            r = serving_workload(dtype, engine)
            times = r["step_times"]
            out["serving_lfm2_700m"] = {
                "generated_tok_s": r["value"], "all_tok_s": r["all_tokens_per_s"], "seconds": r["seconds"],
                "steps": r["steps"], "requests": 32,
                "decode_only": {k: times["decode_only"][k] for k in ("p50_ms", "max_ms", "mean_rows", "hbm_frac_p50")},
                "mixed": {k: times["mixed"][k] for k in ("p50_ms", "max_ms", "mean_prompt_tokens", "mfma_frac_p50")}}
        else:
            r = long_workload(dtype, 4, 32768, quiet=True, engine=engine)
            out["long_lfm2_350m"] = {"requests": 4, "prompt_len": 32768, "prefill_tok_s": r["prefill_tok_s"],
                                     "decode_tok_s": r["value"], "decode_ms_per_step": r["decode_ms_per_step"],
                                     "decode_hbm_frac": r["decode_hbm_frac"]}
        del engine
        torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    sys.exit(main())
