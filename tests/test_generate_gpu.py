"""Generation through the Python entry point and the command line against the plain
implementation's generation loop (which runs every sequence whole again for each token)."""
import os
import random
import subprocess
import sys

import pytest
import torch

import plain_llama as pl
from conftest import ROOT, TOL, rel_err

pytestmark = pytest.mark.gpu


def _prompts(vocab, seed, lengths):
    rnd = random.Random(seed)
    return [[rnd.randrange(vocab) for _ in range(n)] for n in lengths]


@pytest.mark.parametrize("name,lengths,n_new", [("A", [5, 11, 17], 8), ("B", [1, 9, 23, 40], 12), ("C", [3, 70], 6)])
def test_greedy_generation_float32(model_folders, name, lengths, n_new):
    import bitnet_c_amd as bn
    folder = model_folders(name, torch.float32)
    llm = bn.load(folder, dtype="float32", max_tokens=1024)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompts = _prompts(c["vocab"], 1, lengths)
    got = llm.generate(prompts, max_new_tokens=n_new, temperature=0.0, stop_ids=())
    want = [pl.generate(c, W, p, n_new) for p in prompts]
    assert got == want
    # one batch after another gives the same tokens, and so does every request alone
    assert llm.generate(prompts, max_new_tokens=n_new, batch_size=2, stop_ids=()) == want
    assert [llm.generate([p], max_new_tokens=n_new, stop_ids=())[0] for p in prompts] == want
    llm.engine.cache.check()
    assert not llm.engine.cache.live_slots()
    # the step function through the entry object: the logits at a prompt's end pick the first generated token
    slot = llm.new_sequence()
    logits = llm.step([bn.StepEntry(slot, prompts[0], [len(prompts[0]) - 1])])
    assert logits.shape == (1, c["vocab"]) and int(logits[0].argmax()) == want[0][0]
    llm.release(slot)
    assert not llm.engine.cache.live_slots()


def test_stop_tokens_and_budgets(model_folders):
    import bitnet_c_amd as bn
    folder = model_folders("A", torch.float32)
    llm = bn.load(folder, dtype="float32", max_tokens=1024)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompts = _prompts(c["vocab"], 2, [6, 13])
    free = [pl.generate(c, W, p, 10) for p in prompts]
    stop = free[0][3]                                       # the first request's fourth token ends it
    want = [pl.generate(c, W, p, 10, stop_ids=(stop,)) for p in prompts]
    assert len(want[0]) <= 3
    res = llm.generate(prompts, max_new_tokens=10, stop_ids=(stop,), return_results=True)
    assert [r.tokens for r in res] == want
    assert res[0].finish == "stop" and stop not in res[0].tokens
    assert res[1].finish == ("stop" if len(want[1]) < 10 else "length")


@pytest.mark.parametrize("temperature,top_p,penalty", [(0.8, 1.0, 1.0), (0.7, 0.9, 1.0), (0.0, 0.9, 1.3), (1.1, 0.5, 1.2)])
def test_sampled_generation_follows_the_plain_sampler(model_folders, temperature, top_p, penalty):
    import bitnet_c_amd as bn
    folder = model_folders("B", torch.float32)
    llm = bn.load(folder, dtype="float32", max_tokens=1024)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompts = _prompts(c["vocab"], 3, [1, 9, 23, 40])
    got = llm.generate(prompts, max_new_tokens=12, temperature=temperature, top_p=top_p, seed=7,
                       repeat_penalty=penalty, stop_ids=())
    want = [pl.generate(c, W, p, 12, temperature, top_p, 7, (), penalty) for p in prompts]
    assert got == want
    # what a sequence samples does not depend on its batch
    alone = llm.generate(prompts[2:3], max_new_tokens=12, temperature=temperature, top_p=top_p, seed=7,
                         repeat_penalty=penalty, stop_ids=())
    assert alone[0] == want[2]


@pytest.mark.parametrize("with_penalty", [False, True])
def test_requests_of_one_batch_sample_each_in_their_own_way(model_folders, with_penalty):
    """Greedy, temperature and top-p requests in one batch (with a penalty among them the host must see every token
    before the next step; without, steps are queued on tokens that are still on the device), unequal budgets and a stop
    token: every request gets the plain sampler's tokens."""
    import bitnet_c_amd as bn
    from bitnet_c_amd.engine import Request, generate
    from bitnet_c_amd.sampling import SamplingParams, sample_batch
    folder = model_folders("B", torch.float32)
    llm = bn.load(folder, dtype="float32", max_tokens=2048)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompts = _prompts(c["vocab"], 5, [4, 17, 2, 33, 9])
    kinds = [(0.0, 0.9, 1.0), (0.8, 1.0, 1.0), (0.7, 0.9, 1.0), (0.0, 0.9, 1.0), (1.1, 0.5, 1.25 if with_penalty else 1.0)]
    budgets = [9, 4, 12, 1, 7]
    free = pl.generate(c, W, prompts[2], 12, 0.7, 0.9, 11, (), 1.0)
    stops = [(), (), (free[5],), (), ()]
    reqs = [Request(p, n, SamplingParams(temperature=t, top_p=tp, seed=11, repeat_penalty=pen), st)
            for p, n, (t, tp, pen), st in zip(prompts, budgets, kinds, stops)]
    steps_before = llm.engine.steps_run
    res = generate(llm.engine, reqs, sample_batch, batch_size=8)
    want = [pl.generate(c, W, p, n, t, tp, 11, st, pen) for p, n, (t, tp, pen), st in zip(prompts, budgets, kinds, stops)]
    assert [r.tokens for r in res] == want
    assert res[2].finish == "stop" and len(want[2]) < 12
    # the steps that ran: one for the prompts, then one a token of the longest request; queued ahead, the request that
    # its stop token ended had its row in one step more, which is no step more
    assert llm.engine.steps_run - steps_before == max(len(w) for w in want)
    assert not llm.engine.cache.live_slots()
    llm.engine.cache.check()


def test_bfloat16_generation_starts_like_the_plain_one(model_folders):
    import bitnet_c_amd as bn
    folder = model_folders("A", torch.bfloat16)
    llm = bn.load(folder, dtype="bfloat16", max_tokens=1024)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompts = _prompts(c["vocab"], 4, [5, 11, 17, 64, 65])
    got = llm.generate(prompts, max_new_tokens=8, stop_ids=())
    # Rounding may flip a near-tie, and two greedy sequences part for good from there, so counting equal tokens
    # says little.  Every token is checked where it was chosen instead: the plain implementation, fed the engine's
    # own sequence, must hold that token's logit within rounding of its largest one.
    for p, g in zip(prompts, got):
        assert len(g) == 8
        logits = pl.forward(c, W, p + g, torch.bfloat16)[len(p) - 1:-1]
        rms = float(logits.pow(2).mean().sqrt())
        for i, tok in enumerate(g):
            gap = float(logits[i].max() - logits[i, tok])
            assert gap <= TOL[torch.bfloat16] * rms, (p, g, i, gap / rms)
    # and where the plain implementation's choice is clear of every other token by more than that, it is the engine's
    for p, g in zip(prompts, got):
        first = pl.forward(c, W, p, torch.bfloat16)[-1]
        top2 = first.topk(2).values
        if float(top2[0] - top2[1]) > 2 * TOL[torch.bfloat16] * float(first.pow(2).mean().sqrt()):
            assert g[0] == int(first.argmax()), p


def test_command_line(model_folders):
    folder = model_folders("A", torch.float32)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    want = pl.generate(c, W, prompt, 6)
    base = [sys.executable, os.path.join(ROOT, "bin", "bitnet"), folder, "--prompt-token-ids",
            ",".join(map(str, prompt)), "-n", "6", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"]
    # the last one: switches of the reference's runtime that are always so here are taken and answered with a line
    for extra in ([], ["--no-prefill"], ["--maxseq", "64"], ["-t", "4", "--flash"]):
        p = subprocess.run(base + extra, capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-1500:]
        ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
        assert [int(x) for x in ids.split(",")] == want, extra
        assert "tok/s" in p.stderr
        assert ("--flash" in p.stderr) == ("--flash" in extra)
    p = subprocess.run(base + ["--kv16"], capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "--kv16" in p.stderr                 # a 16-bit cache and the float32 path exclude each other
    p = subprocess.run(base[:3] + ["--prompt-token-ids", "1,999"], capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "999" in p.stderr


def test_command_line_sizes_its_cache_by_the_model_s_context_length(tmp_path):
    """Without --maxseq the cache holds a sequence of the model's own context length (the reference:
    min(context length, --maxseq), src/model.c:256-257): a prompt of 5,000 tokens runs on a model of 8,192 positions,
    and is refused, with the reason, under --maxseq 4096."""
    import bitnet_c_amd as bn
    raw = dict(model_type="llama", vocab_size=97, hidden_size=32, intermediate_size=64, num_hidden_layers=1,
               num_attention_heads=2, num_key_value_heads=1, max_position_embeddings=8192, rope_theta=10000.0,
               rms_norm_eps=1e-5, tie_word_embeddings=True)
    folder = bn.write_model_folder(str(tmp_path / "long"), bn.LlamaConfig.from_dict(raw), 3, torch.float32)
    prompt = _prompts(97, 9, [5000])[0]
    base = [sys.executable, os.path.join(ROOT, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
            "-n", "2", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"]
    p = subprocess.run(base, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()]
    assert ids and len(ids[0].split(",")) == 2, p.stderr[-1500:]
    p = subprocess.run(base + ["--maxseq", "4096"], capture_output=True, text=True, timeout=300)
    assert "exceeds the sequence limit 4096" in p.stderr, p.stderr[-1500:]


def test_command_line_with_a_text_prompt(model_folders, tmp_path):
    """-p needs the folder's tokenizer.json: a word-level one is made here for a copy of the tiny
    model; the prompt is encoded with it and the generated ids are printed as its words."""
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers
    src = model_folders("A", torch.float32)
    folder = str(tmp_path / "with_tokenizer")
    shutil.copytree(src, folder)
    words = {f"w{i}": i for i in range(256)}
    tok = Tokenizer(models.WordLevel(vocab=words, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(os.path.join(folder, "tokenizer.json"))
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompt = [3, 1, 4, 1, 5]
    want = pl.generate(c, W, prompt, 5)
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "bitnet"), folder, "-p", " ".join(f"w{t}" for t in prompt),
                        "-n", "5", "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--no-bos"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
    assert [int(x) for x in ids.split(",")] == want
    assert p.stdout.split() == [f"w{t}" for t in want] or p.stdout.replace(" ", "").strip() == "".join(f"w{t}" for t in want)
    # without the tokenizer a text prompt is refused with a message that says what to do
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "bitnet"), src, "-p", "w1 w2", "-n", "2", "--fp32"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "tokenizer.json" in p.stderr + p.stdout


def test_command_line_benchmark_runs_top_logits_and_a_random_folder(tmp_path):
    """--random writes the folder from a configuration and --seed; --benchmark-runs repeats the
    request on the loaded model (every run from fresh request state: the same tokens); the
    --bench-warmup-tokens are generated but neither printed nor counted; --top-logits prints the
    largest logits before every sampling, the first of which is the token greedy decoding takes."""
    import json
    from conftest import TINY_B
    cfg_path = str(tmp_path / "cfg.json")
    with open(cfg_path, "w") as f:
        json.dump(TINY_B, f)
    folder = str(tmp_path / "made")
    prompt = [7, 2, 9, 4]
    exe = [sys.executable, os.path.join(ROOT, "bin", "bitnet")]
    common = ["--prompt-token-ids", ",".join(map(str, prompt)), "--repeat-penalty", "1.0", "--fp32", "--token-ids", "--quiet"]
    p = subprocess.run(exe + [folder, "--random", cfg_path, "--seed", "5", "-n", "7", "--top-logits", "3"] + common,
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    assert os.path.isfile(os.path.join(folder, "model.safetensors")) and os.path.isfile(os.path.join(folder, "config.json"))
    c, W = pl.read_config(folder), pl.read_weights(folder)
    want = pl.generate(c, W, prompt, 7)
    ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
    assert [int(x) for x in ids.split(",")] == want
    heads = [l for l in p.stderr.splitlines() if l.startswith("top_logits generate step=")]
    assert len(heads) == 7 and heads[0].endswith("k=3")
    firsts = [int(l.split("token=")[1].split()[0]) for l in p.stderr.splitlines() if l.startswith("top_logit ") and "rank=1 " in l]
    assert firsts == want
    lg = pl.forward(c, W, prompt)[-1]
    first_line = [l for l in p.stderr.splitlines() if l.startswith("top_logit step=0 rank=1 ")][0]
    assert abs(float(first_line.split("logit=")[1]) - float(lg.max())) <= 1e-4 * float(lg.pow(2).mean().sqrt())
    # the folder exists now: --random refuses to overwrite it
    p = subprocess.run(exe + [folder, "--random", cfg_path, "-n", "1"] + common, capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "already holds a model" in p.stderr + p.stdout
    # repeated runs: 1 unreported + 2 reported, 2 warm-up tokens each
    p = subprocess.run(exe + [folder, "-n", "5", "--benchmark-runs", "2", "--benchmark-warmup-runs", "1",
                              "--bench-warmup-tokens", "2"] + common, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    samples = [l for l in p.stderr.splitlines() if l.startswith("Benchmark sample run=")]
    assert [l.split()[2] for l in samples] == ["run=1", "run=2"]
    assert all("tokens=5" in l and "tok/s=" in l and "prompt_ms=" in l for l in samples)
    ids = [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
    assert [int(x) for x in ids.split(",")] == want[2:]
    p = subprocess.run(exe + [folder, "-n", "1", "--benchmark-warmup-runs", "1"] + common, capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "--benchmark-runs" in p.stderr + p.stdout


@pytest.mark.parametrize("fp32", [True, False])
def test_command_line_dumps_of_the_residual_stream(model_folders, tmp_path, fp32):
    """--dump-binary / --dump-tag / --dump-layer / --dump-pos and the statistics lines (the reference's
    diagnostics, src/main.c:144-147, src/transformer/cpu.c:213-251): the stream at a layer's input, before its
    feed-forward and at its output, against the plain implementation's layers; and the tokens are the same
    with the dumps as without."""
    import numpy as np
    dtype = torch.float32 if fp32 else torch.bfloat16
    folder = model_folders("B", dtype)
    c, W = pl.read_config(folder), pl.read_weights(folder)
    prompt = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3]
    rt = None if fp32 else torch.bfloat16
    toks = torch.tensor(prompt)
    inv_freq = pl.rope_inv_freq(c["head_dim"], c["theta"], c["rope_scaling"])
    xs = [W["model.embed_tokens.weight"][toks].float()]                 # the stream at every layer's input
    for l in range(c["layers"]):
        xs.append(pl.decoder_layer(xs[-1], torch.arange(len(prompt)), W, l, c, inv_freq, rt))
    base = [sys.executable, os.path.join(ROOT, "bin", "bitnet"), folder, "--prompt-token-ids", ",".join(map(str, prompt)),
            "-n", "4", "--repeat-penalty", "1.0", "--token-ids", "--quiet"] + (["--fp32"] if fp32 else [])
    plain_run = subprocess.run(base, capture_output=True, text=True, timeout=300)
    assert plain_run.returncode == 0, plain_run.stderr[-1500:]
    ids = lambda p: [l for l in p.stderr.splitlines() if l and l[0].isdigit()][0]
    tol = 1e-4 if fp32 else 3e-2
    stats = tmp_path / "stats.txt"
    for tag, layer, pos, want in (("bitnet_inp", 1, 7, xs[1][7]), ("bitnet_lout", 2, 9, xs[3][9]), ("bitnet_inp", 0, 0, xs[0][0])):
        out = tmp_path / f"{tag}_{layer}_{pos}.f32"
        p = subprocess.run(base + ["--dump-binary", str(out), "--dump-tag", tag, "--dump-layer", str(layer), "--dump-pos", str(pos),
                                   "--dump-stats", str(stats)], capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-1500:]
        assert ids(p) == ids(plain_run)
        got = torch.from_numpy(np.fromfile(out, dtype="<f4").copy())
        assert got.shape == want.shape and rel_err(got, want) < tol, (tag, layer, pos)
    # the lines of statistics: every tag of the selected layer and position, the numbers those of the vector
    lines = [l for l in stats.read_text().splitlines() if l.startswith("bitnet_lout pos=9 layer=2 ")]
    assert len(lines) == 1
    fields = dict(f.split("=", 1) for f in lines[0].split()[1:])
    assert int(fields["dim"]) == c["dim"]
    assert abs(float(fields["sum"]) - float(xs[3][9].sum())) < tol * float(xs[3][9].abs().sum())
    first = [float(v) for v in fields["first"].split(",")]
    assert len(first) == 16 and rel_err(torch.tensor(first), xs[3][9][:16]) < tol
    # the state before the feed-forward lies between the layer's input and its output: lout - ffn_inp is the feed-forward's output
    out = tmp_path / "ffn_inp.f32"
    p = subprocess.run(base + ["--dump-binary", str(out), "--dump-tag", "bitnet_ffn_inp", "--dump-layer", "1", "--dump-pos", "4"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-1500:]
    x_mid = torch.from_numpy(np.fromfile(out, dtype="<f4").copy())
    pfx = "model.layers.1."
    xb = pl.rmsnorm(x_mid[None, :], W[pfx + "post_attention_layernorm.weight"], c["eps"])
    if rt is not None:
        xb = xb.to(rt).float()
    ffn = pl.feed_forward(xb, W[pfx + "mlp.gate_proj.weight"].float(), W[pfx + "mlp.up_proj.weight"].float(),
                          W[pfx + "mlp.down_proj.weight"].float(), rt)[0]
    assert rel_err(x_mid + ffn, xs[2][4]) < tol
    bad = subprocess.run(base + ["--dump-binary", str(out)], capture_output=True, text=True, timeout=300)
    assert bad.returncode != 0 and "--dump-tag" in bad.stderr
