#!/usr/bin/env python3
"""Decode and prefill throughput of the Llama-3.1-8B shape with random bf16 weights on one
MI355X.  One JSON line on stdout.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--shape 8b|13b|70b]
                    [--context C] [--prompt-lens LO,HI] [--prefill-tokens T]      (further lengths; not the default record)
    python bench.py --only kernel:skinny|attention_prompt|attention_decode|gemm     (single kernels at the benchmark's
                    layer sizes, for a profiler; nothing is timed or printed)

A step is one decode step of the whole batch: the step function, greedy sampling on the
device and the read-back of the tokens, as generation does it.  `value` is decoded
tokens a second at the default batch.  The same line carries the prefill of 2,048
tokens, the decode roofline (bytes the step has to read: every weight once plus the
cache of the live requests, over its time, against 8 TB/s) and decode at batch 1 and 64.
"""
import argparse
import json
import os
import random
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

# The benchmark configuration is the Llama-3.1-8B shape: context 4,096, prompts of 128..2048 tokens.
# The two other shapes are there for measurements at further sizes (--shape); they change nothing
# in the default record.
_LLAMA3_SCALING = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                       original_max_position_embeddings=8192)
SHAPES = {
    "8b": dict(name="llama-3.1-8b-shape", context=4096, prompt_lens=(128, 2048), config=dict(
        model_type="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
        num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
        max_position_embeddings=131072, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
        rope_scaling=_LLAMA3_SCALING)),
    "13b": dict(name="llama-2-13b-shape", context=4096, prompt_lens=(64, 2048), config=dict(
        model_type="llama", vocab_size=32000, hidden_size=5120, intermediate_size=13824,
        num_hidden_layers=40, num_attention_heads=40, num_key_value_heads=40, head_dim=128,
        max_position_embeddings=4096, rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)),
    "70b": dict(name="llama-3-70b-shape", context=8192, prompt_lens=(512, 4096), config=dict(
        model_type="llama", vocab_size=128256, hidden_size=8192, intermediate_size=28672,
        num_hidden_layers=80, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
        max_position_embeddings=8192, rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)),
}
PREFILL_TOKENS = 2048


# ---- single kernels at the benchmark's layer sizes (Llama-3.1-8B shape, bfloat16), for profilers -------------------
# Nothing is checked or timed here: the numerics of these kernels are in tests/test_kernels_gpu.py, their times in
# the profiler's output.

def _kernel_skinny(rows=8, copies=3):
    """The decode products at 8 rows, every weight matrix read cold (three copies in turn)."""
    import torch
    from bitnet_c_amd import ops
    shapes = [("qkv", 6144, 4096, False), ("o", 4096, 4096, False), ("gate_up", 14336, 4096, True),
              ("down", 4096, 14336, False), ("output", 128256, 4096, False)]
    for name, n, k, glu in shapes:
        ws = [torch.randn((2 * n if glu else n), k, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        x = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
        for w in ws:
            if glu:
                ops.linear_swiglu(x, w, True)
            else:
                ops.linear(x, w, torch.float32 if name == "output" else None)
        torch.cuda.synchronize()
        del ws


def _kernel_gemm(rows=2048, reps=3):
    """The prompt products at 2,048 rows through this library's own matrix-core kernel."""
    import torch
    from bitnet_c_amd import ops
    shapes = [("qkv", 6144, 4096, False), ("o", 4096, 4096, False), ("gate_up", 14336, 4096, True),
              ("down", 4096, 14336, False)]
    for name, n, k, glu in shapes:
        w = torch.randn((2 * n if glu else n), k, device="cuda:0", dtype=torch.bfloat16) * 0.02
        x = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
        for _ in range(reps):
            ops.gemm_mfma(x, w, None, glu)
        torch.cuda.synchronize()
        del w


def _kernel_cache(lengths, Hkv=8, hs=128):
    import torch
    pages = [(n + 63) // 64 for n in lengths]
    kp = torch.randn(sum(pages) + 1, Hkv, 64, hs, device="cuda:0", dtype=torch.bfloat16)
    vp = torch.randn(sum(pages) + 1, Hkv, hs, 64, device="cuda:0", dtype=torch.bfloat16)
    bt = torch.zeros(len(lengths), max(pages), dtype=torch.int32)
    p = 0
    for i, n in enumerate(pages):
        bt[i, :n] = torch.arange(p, p + n)
        p += n
    return kp, vp, bt.to("cuda:0")


def _kernel_attention_prompt(H=32, Hkv=8, hs=128):
    """Prompt attention over 2,048 and 8,192 tokens."""
    import torch
    from bitnet_c_amd import ops
    for t in (2048, 8192):
        kp, vp, bt = _kernel_cache([t], Hkv, hs)
        qkv = torch.randn(t, (H + 2 * Hkv) * hs, device="cuda:0", dtype=torch.bfloat16)
        out = torch.empty(t, H * hs, device="cuda:0", dtype=torch.bfloat16)
        _, _, qt = ops.attention_row_shape(H, Hkv, False, torch.bfloat16, hs)
        tiles = torch.tensor(ops.pair_tiles([(0, i, min(qt, t - i), i) for i in range(0, t, qt)]), dtype=torch.int32,
                             device="cuda:0")
        for _ in range(3):
            ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, hs ** -0.5, tiles=tiles, qt=qt)
        torch.cuda.synchronize()


def _kernel_attention_decode(H=32, Hkv=8, hs=128):
    """Decode attention (rotation and cache write inside), batch 1, 8 and 64, unequal lengths."""
    import torch
    from bitnet_c_amd import ops
    rnd = random.Random(0)
    for b in (1, 8, 64):
        lens = [rnd.randint(128, 2112) for _ in range(b)]
        kp, vp, bt = _kernel_cache(lens, Hkv, hs)
        qkv = torch.randn(b, (H + 2 * Hkv) * hs, device="cuda:0", dtype=torch.bfloat16)
        out = torch.empty(b, H * hs, device="cuda:0", dtype=torch.bfloat16)
        d_lens = torch.tensor(lens, dtype=torch.int32, device="cuda:0")
        order = torch.tensor(sorted(range(b), key=lambda i: -lens[i]), dtype=torch.int32, device="cuda:0")
        inv = torch.rand(hs // 2, device="cuda:0")
        n_splits, chunk = ops.decode_splits(b, H, Hkv, bt.shape[1] * 64)
        for _ in range(3):
            ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, hs ** -0.5, seq_lens=d_lens, n_splits=n_splits, chunk=chunk,
                          fused_rotate=inv, fused_write=True, by_length=order)
        torch.cuda.synchronize()


def _kernel_mid(rows=64, copies=3):
    """The products of a decode step of 64 rows, every weight matrix read cold: gate/up through this library's own kernel
    with the SwiGLU epilogue over the row-major matrix and over its streamed copy, and through the library; the
    feed-forward's last product and the output projection as partial sums, row-major and streamed."""
    import torch
    from bitnet_c_amd import ops
    x = torch.randn(rows, 4096, device="cuda:0", dtype=torch.bfloat16)
    ws = [torch.randn(28672, 4096, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
    streamed = [ops.stream_copy(w, ops.STREAM_TILE_ROWS) for w in ws]
    for w in ws:
        ops.linear_swiglu(x, w, True, allow_library=False)
    for w, sw in zip(ws, streamed):
        ops.linear_swiglu(x, w, True, streamed=sw)
    for w in ws:
        ops.swiglu(torch.matmul(x, w.t()), True)
    del ws, streamed
    for n, k in ((4096, 14336), (4096, 4096)):
        xs = torch.randn(rows, k, device="cuda:0", dtype=torch.bfloat16)
        ws = [torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        streamed = [ops.stream_copy(w) for w in ws]
        for w in ws:
            ops.linear_partial_sums(xs, w)
        for w, sw in zip(ws, streamed):
            ops.linear_partial_sums(xs, w, sw)
        del ws, streamed
    torch.cuda.synchronize()


KERNEL_WORKLOADS = {"skinny": _kernel_skinny, "gemm": _kernel_gemm, "attention_prompt": _kernel_attention_prompt,
                    "attention_decode": _kernel_attention_decode, "mid": _kernel_mid}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                    help="8b is the benchmark configuration; the others are further sizes")
    ap.add_argument("--layers", type=int, default=0,
                    help="fewer layers than the configuration has (named in the record)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points")
    ap.add_argument("--only", default=None, metavar="prefill|decode|kernel:NAME",
                    help="for profiling: run one phase alone (the record then lacks the other), or single kernels at "
                         "the benchmark's layer sizes (kernel:" + "|".join(sorted(KERNEL_WORKLOADS)) + ")")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--context", type=int, default=0, help="longest sequence (default: the shape's)")
    ap.add_argument("--prompt-lens", default=None, metavar="LO,HI", help="prompt lengths of the decode batches")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS, help="tokens of the measured prompt step")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2
    if args.only and args.only.startswith("kernel:"):
        name = args.only.split(":", 1)[1]
        if name not in KERNEL_WORKLOADS:
            ap.error(f"--only kernel:{name}: known kernels are {sorted(KERNEL_WORKLOADS)}")
        KERNEL_WORKLOADS[name]()
        return 0
    if args.only not in (None, "prefill", "decode"):
        ap.error("--only takes prefill, decode or kernel:NAME")

    import torch

    import bitnet_c_amd as bn
    from bitnet_c_amd import ops
    from bitnet_c_amd.sampling import SamplingParams, SequenceSampler, start_sampling
    from bitnet_c_amd.config import architecture_for
    from bitnet_c_amd.engine import DecoderModel
    from bitnet_c_amd.weights import random_tensors

    dev = "cuda:0"
    shape = SHAPES[args.shape]
    SHAPE, CONTEXT, (len_lo, len_hi) = shape["config"], shape["context"], shape["prompt_lens"]
    if args.prompt_lens:
        len_lo, len_hi = (int(v) for v in args.prompt_lens.split(","))
    CONTEXT = args.context or max(CONTEXT, len_hi + args.steps + args.warmup + 1, args.prefill_tokens)
    PREFILL = args.prefill_tokens
    args.layers = args.layers or SHAPE["num_hidden_layers"]
    raw = dict(SHAPE, num_hidden_layers=args.layers)
    cfg = bn.LlamaConfig.from_dict(raw)
    plan = architecture_for(raw).build_plan(cfg)
    t0 = time.time()
    model = DecoderModel(plan, torch.bfloat16, dev)
    tensors = random_tensors(plan.expected_tensors(), args.seed, torch.bfloat16, device=dev)
    model.load(tensors)
    del tensors
    torch.cuda.empty_cache()
    print(f"[bench] model built in {time.time() - t0:.1f} s, weights {model.weight_bytes() / 1e9:.2f} GB",
          file=sys.stderr, flush=True)

    max_batch = max(args.batch, 1 if args.no_points else 64)
    per_seq = ((len_hi + args.steps + args.warmup + 64 + 63) // 64) * 64
    engine = bn.Engine(model, max_tokens=max(max_batch * per_seq, 4096, PREFILL + 64), max_seq_len=CONTEXT)
    kept = sum(l.streamed.nbytes() for l in model.linears() if l.streamed is not None)
    print(f"[bench] streamed copies of the weight matrices: {kept / 1e9:.2f} of {model.streamed_bytes() / 1e9:.2f} GB",
          file=sys.stderr, flush=True)
    L, H, Hkv, hs = cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    kv_bytes_per_token = 2 * L * Hkv * hs * 2
    weight_bytes = model.weight_bytes()      # every weight a decode step reads once (no embedding table unless it is tied)
    rnd = random.Random(args.seed + 1)

    def sync():
        torch.cuda.synchronize()

    # ---- prefill of 2,048 tokens ------------------------------------------------------
    def prefill_once(n):
        toks = [rnd.randrange(cfg.vocab_size) for _ in range(n)]
        s = engine.new_sequence()
        sync()
        t = time.perf_counter()
        lg = engine.step([bn.StepEntry(s, toks, [n - 1])])
        ops.argmax(lg).cpu()
        sync()
        dt = time.perf_counter() - t
        engine.release(s)
        return dt

    if args.only == "decode":
        p_ms = float("nan")
    else:
        prefill_once(PREFILL)
        prefill_once(PREFILL)
        p_ms = sorted(prefill_once(PREFILL) for _ in range(5))[2] * 1e3
    T = PREFILL
    lin_params = L * (cfg.hidden_size * (cfg.q_dim + 2 * cfg.kv_dim) + cfg.q_dim * cfg.hidden_size
                      + 3 * cfg.hidden_size * cfg.intermediate_size)
    flops = 2.0 * T * lin_params + 4.0 * T * T * hs * H * L / 2 + 2.0 * cfg.vocab_size * cfg.hidden_size
    prefill = {"value": round(T / (p_ms / 1e3), 1), "tokens": T, "ms": round(p_ms, 3),
               "frac": round(flops / (p_ms / 1e3) / (PEAK_TFLOPS["bf16"] * 1e12), 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ---- decode -----------------------------------------------------------------------
    def decode(batch, steps, warmup):
        lens = [rnd.randint(len_lo, len_hi) for _ in range(batch)]
        slots = [engine.new_sequence() for _ in range(batch)]
        # the prompts, a few sequences a step to bound the activations: at most 8 and at most 2^18 tokens
        last = [0] * batch
        i = 0
        while i < batch:
            k = i + 1
            while k < batch and k - i < 8 and sum(lens[i:k + 1]) <= 1 << 18:
                k += 1
            ent = [bn.StepEntry(slots[j], [rnd.randrange(cfg.vocab_size) for _ in range(lens[j])], [lens[j] - 1])
                   for j in range(i, k)]
            toks = ops.argmax(engine.step(ent)).cpu().tolist()
            for j, t in zip(range(i, k), toks):
                last[j] = t
            i = k

        # as the generation loop runs greedy decoding: the tokens stay on the device, a step is queued on them, then the
        # host reads them (every token reaches the host, one step behind the device)
        greedy = [SequenceSampler(SamplingParams())] * batch
        entries = [bn.StepEntry(slots[j], [0], [0]) for j in range(batch)]
        engine.prepare_decode(batch)          # as generation does at a batch's start: no capture inside the clock
        lg = engine.step([bn.StepEntry(slots[j], [last[j]], [0]) for j in range(batch)])

        def one():
            nonlocal last, lg
            pending = start_sampling(lg, greedy)
            lg = engine.step(entries, device_tokens=pending.device_tokens)
            last = pending.tokens()

        for _ in range(warmup):
            one()
        sync()
        t = time.perf_counter()
        for _ in range(steps):
            one()
        sync()
        dt = time.perf_counter() - t
        ctx_mid = sum(lens) + batch * (1 + warmup + steps / 2.0)          # cached tokens read by a mid step
        for s in slots:
            engine.release(s)
        return dt / steps, ctx_mid

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill}), flush=True)
        return 0
    step_s, ctx_tokens = decode(args.batch, args.steps, args.warmup)
    value = args.batch / step_s
    bytes_step = weight_bytes + ctx_tokens * kv_bytes_per_token
    achieved = bytes_step / step_s / 1e9
    print(f"[bench] decode b{args.batch}: {step_s * 1e3:.3f} ms/step, {value:.1f} tok/s, {bytes_step / 1e9:.2f} GB a step, "
          f"{achieved:.0f} GB/s = {achieved / HBM_GBS:.3f} of {HBM_GBS:.0f}", file=sys.stderr, flush=True)
    points = {}
    if not args.no_points:
        for n in (128, 512):                  # short prompts: a step is the weights once and the host's work, not the matrix cores
            prefill_once(n)
            prefill_once(n)
            points[f"prefill_{n}_ms"] = round(sorted(prefill_once(n) for _ in range(5))[2] * 1e3, 3)
            print(f"[bench] prefill of {n} tokens: {points[f'prefill_{n}_ms']} ms", file=sys.stderr, flush=True)
        for b in (1, 64):
            s_b, ctx_b = decode(b, max(16, args.steps // 2), args.warmup)
            bytes_b = weight_bytes + ctx_b * kv_bytes_per_token
            gbs = bytes_b / s_b / 1e9
            points[f"decode_b{b}"] = round(b / s_b, 1)
            points[f"decode_b{b}_ms"] = round(s_b * 1e3, 4)
            points[f"decode_b{b}_gbs"] = round(gbs, 1)
            points[f"decode_b{b}_frac"] = round(gbs / HBM_GBS, 4)
            print(f"[bench] decode b{b}: {s_b * 1e3:.3f} ms/step, {b / s_b:.1f} tok/s, {bytes_b / 1e9:.2f} GB a step, "
                  f"{gbs:.0f} GB/s = {gbs / HBM_GBS:.3f} of {HBM_GBS:.0f}", file=sys.stderr, flush=True)

    rec = {
        "metric": f"decode tok/s @ batch {args.batch} ({shape['name']}, bf16)", "value": round(value, 1), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": f"synthetic: random N(0,0.02) weights, uniform random token ids, prompts of {len_lo}..{len_hi} tokens",
        "config": {"model": shape["name"], "layers": cfg.num_hidden_layers,
                   "layers_of_config": SHAPE["num_hidden_layers"], "hidden": cfg.hidden_size,
                   "heads": H, "kv_heads": Hkv, "head_dim": hs, "intermediate": cfg.intermediate_size,
                   "vocab": cfg.vocab_size, "rope_theta": cfg.rope_theta, "rope_scaling": "llama3 f8 l1 h4 o8192" if cfg.rope_scaling else "none",
                   "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings,
                   "global_batch": args.batch, "seq_len": CONTEXT, "prompt_lens": f"U[{len_lo},{len_hi}]",
                   "prefill_tokens": PREFILL, "streamed_weights": model.has_streamed, "parallelism": "none (1 GPU)"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBS, 4), "gb_per_step": round(bytes_step / 1e9, 3)},
        "points": points,
    }
    print(json.dumps(rec), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
