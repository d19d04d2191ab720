"""Command line in the manner of the reference's `bitnet <model> [options]`
(src/main.c:110-168, 224-431): the same option names with the same meaning and the same
defaults where this library has the feature (-p, --prompt-token-ids, -n, --temp, --topp,
--seed, --maxseq, --repeat-penalty, --no-prefill, --quiet, --token-ids, --bos/--no-bos).
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
    ap.add_argument("--fp32", action="store_true", help="run the whole model in float32")
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


def main(argv=None) -> int:
    args = _parser().parse_args(argv)
    import torch
    from . import api
    from .engine import Request, StepEntry, generate
    from .sampling import SamplingParams, sample_batch

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
    llm = api.load(args.model, dtype="float32" if args.fp32 else "bfloat16",
                   max_tokens=max(64, (max_seq or 4096) * (args.batch if args.batch_file else 1)),
                   max_seq_len=max_seq)
    eng = llm.engine
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
    reqs = [Request(p, args.n_tokens, params, stop) for p in prompts]

    def emit(i, t):
        if not args.quiet and len(prompts) == 1:
            sys.stdout.write(tok.decode([t]) if tok is not None else f"{t} ")
            sys.stdout.flush()
        return False

    torch.cuda.synchronize()
    t1 = time.time()
    if args.no_prefill and len(prompts) == 1:
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
        results = generate(OneByOne(eng), reqs, sample_batch, batch_size=1, on_token=emit)
    else:
        results = generate(eng, reqs, sample_batch, batch_size=args.batch, on_token=emit)
    torch.cuda.synchronize()
    dt = time.time() - t1
    if not args.quiet and len(prompts) == 1:
        sys.stdout.write("\n")
    n_gen = sum(len(r.tokens) for r in results)
    for i, r in enumerate(results):
        if r.finish.startswith("error"):
            print(f"[bitnet] request {i}: {r.finish}", file=sys.stderr)
        if args.token_ids or len(prompts) > 1:
            print(("" if len(prompts) == 1 else f"{i}: ") + ",".join(str(t) for t in r.tokens), file=sys.stderr)
    print(f"tokens: {n_gen}  tok/s: {n_gen / dt if dt > 0 else 0.0:.2f}  total_ms: {dt * 1e3:.1f}  "
          f"load_ms: {load_s * 1e3:.0f}", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
