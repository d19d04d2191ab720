#!/usr/bin/env python3
"""Single kernels at the benchmark's layer sizes (Llama-3.1-8B shape, bfloat16), for profilers.

    python3 tests/workloads.py skinny            # the decode products at 8 rows, cold weights
    python3 tests/workloads.py attention_prompt  # prompt attention over 2,048 and 8,192 tokens
    python3 tests/workloads.py attention_decode  # decode attention, batch 8 and 64, unequal lengths
    python3 tests/workloads.py gemm              # the prompt products at 2,048 rows, this library's own kernel

No test: nothing is checked here; the numerics of these kernels are in test_kernels_gpu.py.
"""
import os
import random
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from bitnet_c_amd import ops  # noqa: E402

DEV = "cuda:0"
H, HKV, HS = 32, 8, 128


def skinny(rows=8, copies=3):
    shapes = [("qkv", 6144, 4096, False), ("o", 4096, 4096, False), ("gate_up", 14336, 4096, True),
              ("down", 4096, 14336, False), ("output", 128256, 4096, False)]
    for name, n, k, glu in shapes:
        ws = [torch.randn((2 * n if glu else n), k, device=DEV, dtype=torch.bfloat16) * 0.02 for _ in range(copies)]
        x = torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)
        for w in ws:
            if glu:
                ops.linear_swiglu(x, w, True)
            else:
                ops.linear(x, w, torch.float32 if name == "output" else None)
        torch.cuda.synchronize()
        del ws


def gemm(rows=2048, reps=3):
    shapes = [("qkv", 6144, 4096, False), ("o", 4096, 4096, False), ("gate_up", 14336, 4096, True),
              ("down", 4096, 14336, False)]
    for name, n, k, glu in shapes:
        w = torch.randn((2 * n if glu else n), k, device=DEV, dtype=torch.bfloat16) * 0.02
        x = torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)
        for _ in range(reps):
            ops.gemm_mfma(x, w, None, glu)
        torch.cuda.synchronize()
        del w


def _cache(lengths):
    pages = [(n + 63) // 64 for n in lengths]
    kp = torch.randn(sum(pages) + 1, HKV, 64, HS, device=DEV, dtype=torch.bfloat16)
    vp = torch.randn(sum(pages) + 1, HKV, HS, 64, device=DEV, dtype=torch.bfloat16)
    bt = torch.zeros(len(lengths), max(pages), dtype=torch.int32)
    p = 0
    for i, n in enumerate(pages):
        bt[i, :n] = torch.arange(p, p + n)
        p += n
    return kp, vp, bt.to(DEV)


def attention_prompt():
    for t in (2048, 8192):
        kp, vp, bt = _cache([t])
        qkv = torch.randn(t, (H + 2 * HKV) * HS, device=DEV, dtype=torch.bfloat16)
        out = torch.empty(t, H * HS, device=DEV, dtype=torch.bfloat16)
        _, _, qt = ops.attention_row_shape(H, HKV, False, torch.bfloat16, HS)
        tiles = torch.tensor([(0, i, min(qt, t - i), i) for i in range(0, t, qt)], dtype=torch.int32, device=DEV)
        for _ in range(3):
            ops.attention(qkv, out, kp, vp, bt, H, HKV, HS, HS ** -0.5, tiles=tiles, qt=qt)
        torch.cuda.synchronize()


def attention_decode():
    rnd = random.Random(0)
    for b in (8, 64):
        lens = [rnd.randint(128, 2112) for _ in range(b)]
        kp, vp, bt = _cache(lens)
        qkv = torch.randn(b, (H + 2 * HKV) * HS, device=DEV, dtype=torch.bfloat16)
        out = torch.empty(b, H * HS, device=DEV, dtype=torch.bfloat16)
        d_lens = torch.tensor(lens, dtype=torch.int32, device=DEV)
        order = torch.tensor(sorted(range(b), key=lambda i: -lens[i]), dtype=torch.int32, device=DEV)
        inv = torch.rand(HS // 2, device=DEV)
        n_splits, chunk = ops.decode_splits(b, H, HKV, bt.shape[1] * 64)
        for _ in range(3):
            ops.attention(qkv, out, kp, vp, bt, H, HKV, HS, HS ** -0.5, seq_lens=d_lens, n_splits=n_splits, chunk=chunk,
                          fused_rotate=inv, fused_write=True, by_length=order)
        torch.cuda.synchronize()


if __name__ == "__main__":
    which = sys.argv[1] if len(sys.argv) > 1 else ""
    if which not in ("skinny", "attention_prompt", "attention_decode", "gemm"):
        sys.exit(__doc__)
    {"skinny": skinny, "attention_prompt": attention_prompt, "attention_decode": attention_decode, "gemm": gemm}[which]()
