"""bin/trace_run as a user calls it: a subprocess, steps on standard input,
logits files out. The same requests whole, with the last 32 tokens one by one,
in portions of changing size, and mixed with others so that pages are used
again, in float32 and in bfloat16, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from conftest import prompt_tokens, ROOT
from tolerances import check_logits

pytestmark = pytest.mark.gpu
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def build_trace(vocab):
    """Steps and, per step, which (request key, positions) its rows are."""
    toks = {k: prompt_tokens(vocab, 100, 7) for k in "wsp"}        # the same request three ways
    for i, n in enumerate((70, 130, 40, 90, 64)):
        toks[f"m{i}"] = prompt_tokens(vocab, n, 21 + i)
    steps, rows = [], []

    def add(entries, end=()):
        steps.append({"step": len(steps), "end": list(end),
                      "entries": [{"id": k, "tokens": toks[k][lo:hi], "want": list(range(hi - lo))} for k, lo, hi in entries]})
        rows.append([(k, lo, hi) for k, lo, hi in entries])

    add([("w", 0, 100)], end=["w"])                                    # whole
    add([("s", 0, 68)])                                                # then the last 32 one by one
    for i in range(68, 100):
        add([("s", i, i + 1)], end=["s"] if i == 99 else [])
    at = 0                                                             # portions of changing size
    for n in [2, 5, 2, 31, 3, 17, 2, 38]:
        add([("p", at, at + n)], end=["p"] if at + n == 100 else [])
        at += n
    assert at == 100
    # mixed: up to four live, portions beside single tokens, a request left out of a step
    add([("m0", 0, 50), ("m1", 0, 9)])
    add([("m0", 50, 51), ("m1", 9, 80), ("m2", 0, 2)])
    add([("m0", 51, 52), ("m2", 2, 40), ("m3", 0, 33)], end=["m2"])
    add([("m0", 52, 70), ("m1", 80, 81), ("m3", 33, 35), ("m4", 0, 30)], end=["m0"])
    add([("m1", 81, 130), ("m3", 35, 36), ("m4", 30, 32)], end=["m1"])
    add([("m3", 36, 90), ("m4", 32, 64)], end=["m3", "m4"])
    return toks, steps, rows


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_trace_run(model_dirs, plain_models, tmp_path, name, dtype):
    vocab = plain_models[name].cfg["vocab_size"]
    toks, steps, rows = build_trace(vocab)
    out_dir = str(tmp_path / "logits")
    # the mixed part holds at most 128+192+128+64 = 512 rounded tokens; everything else less
    proc = subprocess.run([sys.executable, TRACE_RUN, "--model", model_dirs[name], "--dtype", dtype,
                           "--out", out_dir, "--max-tokens", "512"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                          timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    refs = {k: plain_models[name].logits(t) for k, t in toks.items()}
    for s, rws in zip(steps, rows):
        got = np.fromfile(os.path.join(out_dir, f"{s['step']}.f32"), dtype="<f4").reshape(-1, vocab)
        ref = torch.cat([refs[k][lo:hi] for k, lo, hi in rws])
        check_logits(torch.from_numpy(got), ref, dtype, f"{name} step {s['step']}")


def test_trace_run_writes_nothing_for_steps_that_want_nothing(model_dirs, tmp_path):
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [4], "want": [0]}], "end": ["a"]}]
    out_dir = str(tmp_path / "o")
    proc = subprocess.run([sys.executable, TRACE_RUN, "--model", model_dirs["A"], "--dtype", "float32",
                           "--out", out_dir, "--max-tokens", "64"],
                          input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert sorted(os.listdir(out_dir)) == ["1.f32"] and proc.stdout.split() == ["done", "0", "done", "1"]
