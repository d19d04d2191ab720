"""bin/trace_run as a user runs it: the same requests whole, with the last 32 tokens one by
one, and in batches of unequal lengths whose slots are used again, in float32 and in
bfloat16, against the plain implementation."""
import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as pl
from conftest import ROOT, TOL, rel_err

pytestmark = pytest.mark.gpu

TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")


def run_trace(folder, dtype, steps, out_dir, max_tokens):
    name = "float32" if dtype == torch.float32 else "bfloat16"
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run([sys.executable, TRACE_RUN, "--model", folder, "--dtype", name, "--out", out_dir,
                        "--max-tokens", str(max_tokens)], input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [l for l in p.stdout.splitlines() if l.startswith("done ")]
    assert done == [f"done {s['step']}" for s in steps]
    return p


def read_logits(out_dir, step, vocab):
    a = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
    return torch.from_numpy(a.reshape(-1, vocab).copy())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_three_ways(model_folders, tmp_path, name, dtype):
    folder = model_folders(name, dtype)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    vocab = c["vocab"]
    rnd = random.Random(31)
    lengths = [40, 97, 33, 130, 64, 71]
    reqs = {f"r{i}": [rnd.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}
    ref = {k: pl.forward(c, W, v, None if dtype == torch.float32 else torch.bfloat16) for k, v in reqs.items()}

    # (1) each request alone and whole
    steps = [{"step": i, "entries": [{"id": k, "tokens": v, "want": list(range(len(v)))}], "end": [k]}
             for i, (k, v) in enumerate(reqs.items())]
    out = str(tmp_path / "whole")
    run_trace(folder, dtype, steps, out, 192)                   # one request of up to 130 tokens at a time
    whole = {k: read_logits(out, i, vocab) for i, k in enumerate(reqs)}
    for k in reqs:
        assert rel_err(whole[k], ref[k]) < TOL[dtype], k

    # (2) the last 32 tokens one by one
    steps, n, where = [], 0, {}
    for k, v in reqs.items():
        n0 = len(v) - 32
        steps.append({"step": n, "entries": [{"id": k, "tokens": v[:n0], "want": list(range(n0))}], "end": []})
        where[k] = [n]
        n += 1
        for j in range(n0, len(v)):
            steps.append({"step": n, "entries": [{"id": k, "tokens": [v[j]], "want": [0]}],
                          "end": [k] if j == len(v) - 1 else []})
            where[k].append(n)
            n += 1
    out = str(tmp_path / "last32")
    run_trace(folder, dtype, steps, out, 192)
    for k in reqs:
        got = torch.cat([read_logits(out, s, vocab) for s in where[k]])
        assert rel_err(got, ref[k]) < TOL[dtype], k
        if dtype == torch.float32:               # one order of summation per query, however the tokens were cut
            assert torch.equal(got, whole[k]), k
        else:
            assert rel_err(got, whole[k]) < TOL[dtype], k

    # (3) batches of unequal lengths; the prompts are the first part of each request, the rest is
    #     decoded one by one; shorter requests end earlier; the second batch uses the first one's slots
    steps, n = [], 0
    got = {k: [] for k in reqs}
    order = {}
    for batch in (["r0", "r1", "r2"], ["r3", "r4", "r5"]):
        fed = {k: max(1, len(reqs[k]) // 3) for k in batch}
        steps.append({"step": n, "entries": [{"id": k, "tokens": reqs[k][:fed[k]], "want": list(range(fed[k]))}
                                             for k in batch], "end": []})
        order[n] = [(k, fed[k]) for k in batch]
        n += 1
        live = list(batch)
        while live:
            ent = [{"id": k, "tokens": [reqs[k][fed[k]]], "want": [0]} for k in live]
            order[n] = [(k, 1) for k in live]
            for k in live:
                fed[k] += 1
            ended = [k for k in live if fed[k] == len(reqs[k])]
            steps.append({"step": n, "entries": ent, "end": ended})
            live = [k for k in live if k not in ended]
            n += 1
    out = str(tmp_path / "batches")
    # the first batch holds 40 + 97 + 33 tokens = 64 + 128 + 64 rounded; the second 192 + 64 + 128
    run_trace(folder, dtype, steps, out, 384)
    for s, parts in order.items():
        lg = read_logits(out, s, vocab)
        o = 0
        for k, cnt in parts:
            got[k].append(lg[o:o + cnt])
            o += cnt
        assert o == lg.shape[0]
    for k in reqs:
        g = torch.cat(got[k])
        assert rel_err(g, ref[k]) < TOL[dtype], k
        if dtype == torch.float32:               # nor does the batch, or the place in the cache, change a bit
            assert torch.equal(g, whole[k]), k
        else:
            assert rel_err(g, whole[k]) < TOL[dtype], k


def test_steps_without_wanted_logits_write_no_file(model_folders, tmp_path):
    folder = model_folders("A", torch.float32)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": [1, 2, 3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": [4], "want": [0]}], "end": ["x"]},
             {"step": 2, "entries": [], "end": []}]
    out = str(tmp_path / "o")
    run_trace(folder, torch.float32, steps, out, 64)
    assert sorted(os.listdir(out)) == ["1.f32"]
    c, W = pl.read_config(folder), pl.read_weights(folder)
    assert rel_err(read_logits(out, 1, c["vocab"]), pl.forward(c, W, [1, 2, 3, 4])[3:4]) < TOL[torch.float32]
