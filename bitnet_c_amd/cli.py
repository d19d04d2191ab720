"""Command line in the manner of the reference's `bitnet <model> [options]`
(src/main.c:110-168, 224-431): the same option names with the same meaning and the same
defaults where this library has the feature (-p, --prompt-token-ids, -n, --temp, --topp,
--seed, --maxseq, --repeat-penalty, --no-prefill, --quiet, --token-ids, --bos/--no-bos,
--top-logits, --benchmark-runs, --benchmark-warmup-runs, --bench-warmup-tokens).
The model is a folder (config.json + model.safetensors) instead of a GGUF file.  Text
prompts need the folder's tokenizer.json; token ids in, token ids out always works.
"""
from __future__ import annotations

import argparse
import os
import sys
import time


def _parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="bitnet", description="Generate with a model folder on one MI355X.")
    ap.add_argument("model", help="model folder (config.json, model.safetensors)")
    ap.add_argument("-p", dest="prompt", default="Hello", help='input prompt (default: "Hello")')
    ap.add_argument("--prompt-token-ids", default=None, help="comma-separated prompt token ids")
    ap.add_argument("-n", dest="n_tokens", type=int, default=256, help="number of tokens to generate (default 256; 0: prompt only)")
    ap.add_argument("--temp", type=float, default=0.0, help="temperature (default 0.0 = greedy)")
    ap.add_argument("--topp", type=float, default=0.9, help="top-p sampling (default 0.9)")
    ap.add_argument("--seed", type=int, default=42, help="random seed (default 42)")
    ap.add_argument("--maxseq", type=int, default=0, help="max sequence length (default: the model's)")
    ap.add_argument("--repeat-penalty", type=float, default=1.1, help="repetition penalty (default 1.1)")
    ap.add_argument("--no-prefill", action="store_true", help="feed the prompt one token at a time")
    ap.add_argument("--quiet", action="store_true", help="suppress generated text")
    ap.add_argument("--token-ids", action="store_true", help="print generated token ids to stderr")
    ap.add_argument("--bos", dest="bos", action="store_true", default=True, help="prepend BOS to a text prompt")
    ap.add_argument("--no-bos", dest="bos", action="store_false")
    ap.add_argument("--top-logits", type=int, default=0, help="print the K largest logits before every sampling (at most 32)")
    ap.add_argument("--benchmark-runs", type=int, default=0, help="measured runs of the same request on one loaded model")
    ap.add_argument("--benchmark-warmup-runs", type=int, default=0, help="unreported runs before the measured ones")
    ap.add_argument("--bench-warmup-tokens", type=int, default=0,
                    help="tokens generated after the prompt before the clock of tok/s starts")
    ap.add_argument("--fp32", action="store_true", help="run the whole model in float32")
    ap.add_argument("--random", default=None, metavar="CONFIG_JSON",
                    help="first write MODEL as a new folder: this configuration with random weights from --seed")
    # switches of the reference's runtime that select what is always so here, or what this library does not have: taken so
    # that a command line written for the reference runs, and answered with one line each (src/main.c:120-167, 268-275)
    ap.add_argument("-t", dest="threads", type=int, default=None, help="CPU threads of the reference: no effect (one GPU)")
    ap.add_argument("--flash", action="store_true", help="online-softmax attention: always on here")
    ap.add_argument("--kv16", action="store_true", help="16-bit cache: always so in bfloat16; refused with --fp32")
    # diagnostics of the reference (src/main.c:144-147, 333-340; the text dump is its BN_DUMP_LAYER_INP)
    ap.add_argument("--dump-binary", default=None, metavar="PATH", help="write a selected state of the residual stream as float32")
    ap.add_argument("--dump-tag", default=None, help="which state: bitnet_inp (a layer's input), bitnet_ffn_inp, bitnet_lout")
    ap.add_argument("--dump-layer", type=int, default=None, help="select the layer of the dumps")
    ap.add_argument("--dump-pos", type=int, default=None, help="select the token position of the dumps")
    ap.add_argument("--dump-stats", default=os.environ.get("BN_DUMP_LAYER_INP"), metavar="PATH",
                    help="append a line of statistics per dumped state (default: $BN_DUMP_LAYER_INP)")
    ap.add_argument("--batch-file", default=None, help="file with one comma-separated prompt (token ids) a line")
    ap.add_argument("--batch", type=int, default=8, help="sequences per batch with --batch-file (default 8)")
    return ap


def _ids(text: str, vocab: int):
    out = []
    for part in text.replace(" ", ",").split(","):
        if part == "":
            continue
        v = int(part)
        if not 0 <= v < vocab:                      # src/main.c:1566-1590 range-checks the ids
            raise SystemExit(f"prompt token id {v} is outside [0, {vocab})")
        out.append(v)
    if not out:
        raise SystemExit("no prompt token ids given")
    return out


MAX_TOP_LOGITS = 32      # src/generate.c:64


def _with_top_logits(sample_fn, k: int):
    """A sampler that first prints the k largest logits of every row, in the lines of
    src/generate.c:83-86 (one block per row; `step` counts the samplings)."""
    import torch
    k = min(k, MAX_TOP_LOGITS)
    step = [0]

    def fn(logits, samplers):
        kk = min(k, logits.shape[1])
        vals, idx = torch.topk(logits.float(), kk, dim=1)
        for row, (v, i) in enumerate(zip(vals.tolist(), idx.tolist())):
            label = "generate" if logits.shape[0] == 1 else f"generate[{row}]"
            print(f"top_logits {label} step={step[0]} k={kk}", file=sys.stderr)
            for r, (x, t) in enumerate(zip(v, i)):
                print(f"top_logit step={step[0]} rank={r + 1} token={t} logit={x:.9g}", file=sys.stderr)
        step[0] += 1
        return sample_fn(logits, samplers)
    return fn


DUMP_POINTS = {"layer_in": "bitnet_inp", "ffn_in": "bitnet_ffn_inp", "layer_out": "bitnet_lout"}   # src/transformer/cpu.c:401, :951, :981


def _dump_tap(args):
    """The engine's diagnostic tap for --dump-binary / --dump-stats: the residual stream of the selected layer
    and position at the reference's dump points, as the float32 vector (the file is rewritten at every
    match, as in src/transformer/cpu.c:221-229) and as the reference's line of statistics (:231-251)."""
    if not args.dump_binary and not args.dump_stats:
        return None
    if args.dump_binary and not args.dump_tag:
        raise SystemExit("--dump-binary needs --dump-tag (bitnet_inp, bitnet_ffn_inp or bitnet_lout)")
    if args.dump_tag and args.dump_tag not in DUMP_POINTS.values():
        raise SystemExit(f"--dump-tag: one of {', '.join(DUMP_POINTS.values())}")

    def tap(point, entry, stream, ctx):
        tag = DUMP_POINTS[point]
        if args.dump_layer is not None and entry != args.dump_layer:
            return
        if not args.dump_stats and tag != args.dump_tag:
            return
        x = stream.flush()                              # the sum itself: a part's output is held back until the next norm
        row = 0
        for p0, n in zip(ctx.pos0, ctx.n_new):
            for pos in range(p0, p0 + n):
                if args.dump_pos is None or pos == args.dump_pos:
                    v = x[row].float().cpu()
                    if args.dump_binary and tag == args.dump_tag:
                        with open(args.dump_binary, "wb") as f:
                            f.write(v.numpy().astype("<f4").tobytes())
                    if args.dump_stats:
                        first = ",".join(f"{t:.9g}" for t in v[:16].tolist())
                        with open(args.dump_stats, "a") as f:
                            f.write(f"{tag} pos={pos} layer={entry} dim={v.numel()} sum={float(v.sum()):.9g} "
                                    f"ss={float((v * v).sum()):.9g} min={float(v.min()):.9g} max={float(v.max()):.9g} "
                                    f"first={first}\n")
                row += 1
    return tap


def _check_benchmark_args(args) -> None:
    # src/main.c:921-931
    if args.benchmark_runs < 0 or args.benchmark_warmup_runs < 0 or args.bench_warmup_tokens < 0:
        raise SystemExit("--benchmark-runs, --benchmark-warmup-runs and --bench-warmup-tokens must not be negative")
    if args.benchmark_warmup_runs > 0 and args.benchmark_runs == 0:
        raise SystemExit("--benchmark-warmup-runs requires --benchmark-runs")
    if (args.benchmark_runs > 0 or args.bench_warmup_tokens > 0) and args.batch_file:
        raise SystemExit("--benchmark-runs and --bench-warmup-tokens take one prompt, not --batch-file")


def _note_reference_switches(args) -> None:
    if args.threads is not None:
        print("[bitnet] -t: no CPU threads to set, the model runs on one GPU", file=sys.stderr)
    if args.flash:
        print("[bitnet] --flash: attention is always computed with the online softmax here", file=sys.stderr)
    if args.kv16:
        if args.fp32:
            raise SystemExit("--kv16 with --fp32: the float32 path keeps a float32 cache (run without --fp32 for a 16-bit one)")
        print("[bitnet] --kv16: the bfloat16 path keeps its cache in 16 bits already", file=sys.stderr)


def main(argv=None) -> int:
    args = _parser().parse_args(argv)
    _check_benchmark_args(args)
    _note_reference_switches(args)
    import torch
    from . import api
    from .engine import Request, StepEntry, generate
    from .sampling import SamplingParams, sample_batch

    if args.random:
        import json
        from .config import architecture_for
        from .weights import write_model_folder
        if os.path.exists(os.path.join(args.model, "model.safetensors")):
            raise SystemExit(f"--random: {args.model} already holds a model")
        with open(args.random) as f:
            raw = json.load(f)
        write_model_folder(args.model, architecture_for(raw).config_cls.from_dict(raw), args.seed,
                           "float32" if args.fp32 else "bfloat16")
        print(f"[bitnet] wrote {args.model} (random weights, seed {args.seed})", file=sys.stderr)
    tok = None
    tok_path = os.path.join(args.model, "tokenizer.json")
    if os.path.isfile(tok_path):
        try:
            from tokenizers import Tokenizer
            tok = Tokenizer.from_file(tok_path)
        except Exception as e:                        # the tokenizer is a convenience, not the core
            print(f"[bitnet] tokenizer.json could not be loaded: {e}", file=sys.stderr)
    t0 = time.time()
    max_seq = args.maxseq
    # The cache holds min(the model's context length, --maxseq) positions for every sequence of a batch, as the
    # reference sizes its own (src/model.c:256-257), or what fits into the device's memory if that is less.
    llm = api.load(args.model, dtype="float32" if args.fp32 else "bfloat16", max_tokens=0, max_seq_len=max_seq,
                   n_seqs=args.batch if args.batch_file else 1)
    eng = llm.engine
    if eng.max_seq_len < (min(max_seq, eng.model.plan.max_positions or max_seq) if max_seq
                          else eng.model.plan.max_positions):
        print(f"[bitnet] the cache holds sequences of up to {eng.max_seq_len} tokens (what fits into the device's "
              f"memory beside the model); longer prompts are refused", file=sys.stderr)
    eng.tap = _dump_tap(args)
    vocab = eng.vocab_size
    cfg = llm.config
    if args.batch_file:
        with open(args.batch_file) as f:
            prompts = [_ids(l, vocab) for l in f if l.strip()]
    elif args.prompt_token_ids is not None:
        prompts = [_ids(args.prompt_token_ids, vocab)]
    else:
        if tok is None:
            raise SystemExit("a text prompt needs tokenizer.json in the model folder; "
                             "use --prompt-token-ids a,b,c")
        ids = tok.encode(args.prompt, add_special_tokens=False).ids
        if args.bos and getattr(cfg, "bos_token_id", None) is not None:
            ids = [int(cfg.bos_token_id)] + ids
        prompts = [ids]
    load_s = time.time() - t0
    params = SamplingParams(temperature=args.temp, top_p=args.topp, seed=args.seed,
                            repeat_penalty=args.repeat_penalty)
    stop = tuple(eng.model.plan.stop_ids)
    warm = args.bench_warmup_tokens
    reqs = [Request(p, args.n_tokens + warm, params, stop) for p in prompts]
    repeated = args.benchmark_runs > 0
    sampler = _with_top_logits(sample_batch, args.top_logits) if args.top_logits > 0 else sample_batch
    stamps = []                                       # when each token of the (single) request came

    def emit(i, t):
        stamps.append(time.time())
        if len(stamps) <= warm:
            return False
        if not args.quiet and not repeated and len(prompts) == 1:
            sys.stdout.write(tok.decode([t]) if tok is not None else f"{t} ")
            sys.stdout.flush()
        return False

    # the prompt one token at a time (src/generate.c:405-416), then the usual loop
    class OneByOne:
        def __init__(self, e):
            self.e = e
            self.cache, self.max_seq_len = e.cache, e.max_seq_len
        def new_sequence(self): return self.e.new_sequence()
        def release(self, s): self.e.release(s)
        def step(self, entries):
            ent = entries[0]
            if len(ent.tokens) == 1:
                return self.e.step(entries)
            for t in ent.tokens[:-1]:
                self.e.step([StepEntry(ent.slot, [t], [])])
            return self.e.step([StepEntry(ent.slot, [ent.tokens[-1]], [0])])

    # Repetitions start from fresh request state (a new slot, a new generator) and keep the loaded
    # model (src/main.c:1607-1616).
    total_runs = args.benchmark_warmup_runs + args.benchmark_runs if repeated else 1
    for run in range(total_runs):
        del stamps[:]
        torch.cuda.synchronize()
        t1 = time.time()
        if args.no_prefill and len(prompts) == 1:
            results = generate(OneByOne(eng), reqs, sampler, batch_size=1, on_token=emit)
        else:
            results = generate(eng, reqs, sampler, batch_size=args.batch, on_token=emit)
        torch.cuda.synchronize()
        t2 = time.time()
        if len(prompts) == 1:
            # the clock of tok/s starts after the prompt and the warm-up tokens (src/main.c:1651-1668)
            timed = max(0, len(stamps) - warm)
            # the first token is sampled from the prompt's logits: the prompt phase ends there
            prompt_end = stamps[0] if stamps else t2
            gen_start = stamps[warm] if warm and len(stamps) > warm else prompt_end
            for r in results:
                r.tokens = r.tokens[warm:]
            speed = timed / (t2 - gen_start) if timed and t2 > gen_start else 0.0
            if repeated and run >= args.benchmark_warmup_runs:
                print(f"Benchmark sample run={run - args.benchmark_warmup_runs + 1} tokens={timed} "
                      f"tok/s={speed:.2f} prompt_ms={(prompt_end - t1) * 1e3:.1f}", file=sys.stderr)
    dt = t2 - t1
    if not args.quiet and not repeated and len(prompts) == 1:
        sys.stdout.write("\n")
    n_gen = sum(len(r.tokens) for r in results)
    for i, r in enumerate(results):
        if r.finish.startswith("error"):
            print(f"[bitnet] request {i}: {r.finish}", file=sys.stderr)
        if args.token_ids or len(prompts) > 1:
            print(("" if len(prompts) == 1 else f"{i}: ") + ",".join(str(t) for t in r.tokens), file=sys.stderr)
    if len(prompts) == 1:
        print(f"tokens: {n_gen}  tok/s: {speed:.2f}  prompt_ms: {(prompt_end - t1) * 1e3:.1f}  "
              f"total_ms: {dt * 1e3:.1f}  load_ms: {load_s * 1e3:.0f}", file=sys.stderr)
    else:
        print(f"tokens: {n_gen}  tok/s: {n_gen / dt if dt > 0 else 0.0:.2f}  total_ms: {dt * 1e3:.1f}  "
              f"load_ms: {load_s * 1e3:.0f}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
