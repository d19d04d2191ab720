"""Attention mixer: grouped-query attention over the paged cache.

Order of the reference's layer (src/transformer/cpu.c:770-939): Q, K, V projections
(+ bias when the tensors exist) -> position encoding of Q and K -> K, V into the cache
-> for head h, kv head h / (H/Hkv): scores (q.k) * scale over the visible keys, softmax,
weighted sum of values -> output projection.  scale is a parameter (1/sqrt(head_dim)
for this architecture, src/model_arch.c:141-145); `window` > 0 limits the visible keys
to the last `window` positions.

The three projections are stored stacked ([Wq; Wk; Wv], as the reference's GPU upload
stacks them, include/backend_model.h:21-22) so that one product computes them.
A schedule entry that reads another entry's cache computes Q only.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, POSITION_ENCODINGS, CacheNeed, KVNeed, ParamSpec, Part, PartSpec
from .linear import Linear, upload


@MIXERS.register("attention")
class Attention(Part):
    @property
    def prompt_capturable(self) -> bool:      # a prompt step is read from the context's device tensors alone
        return getattr(self.position, "prompt_capturable", False)

    takes_deferred_norm = True      # forward accepts an ops.DeferredNorm for h
    gives_lazy_delta = True         # forward(..., lazy_ok=True) may return a LazyDelta

    def __init__(self, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 position: PartSpec, window: int = 0, bias: bool = False):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if head_dim % 2 or head_dim < 2 or head_dim > ops.MAX_HEAD_DIM:
            raise ValueError(f"attention: head_dim {head_dim} is not supported by the kernels "
                             f"(even, at most {ops.MAX_HEAD_DIM})")
        self.hidden, self.H, self.Hkv, self.hs = int(hidden), int(n_heads), int(n_kv_heads), int(head_dim)
        self.scale, self.window, self.has_bias = float(scale), int(window), bool(bias)
        self.position = POSITION_ENCODINGS.build(position)
        self.qkv, self.o = Linear(), Linear()

    @property
    def q_dim(self):
        return self.H * self.hs

    @property
    def kv_dim(self):
        return self.Hkv * self.hs

    def tensors(self):
        t = {"wq": ParamSpec((self.q_dim, self.hidden)), "wk": ParamSpec((self.kv_dim, self.hidden)),
             "wv": ParamSpec((self.kv_dim, self.hidden)), "wo": ParamSpec((self.hidden, self.q_dim))}
        if self.has_bias:
            t.update({"bq": ParamSpec((self.q_dim,), "normal"), "bk": ParamSpec((self.kv_dim,), "normal"),
                      "bv": ParamSpec((self.kv_dim,), "normal"), "bo": ParamSpec((self.hidden,), "normal")})
        return t

    def load(self, tensors, device, dtype):
        # stacked on the device: the host holds no copy beside the file's own bytes
        w = torch.cat([upload(tensors[n], device, dtype) for n in ("wq", "wk", "wv")], dim=0)
        b = None
        if self.has_bias:
            b = torch.cat([upload(tensors[n], device, torch.float32) for n in ("bq", "bk", "bv")])
        self.qkv.load(w, b, device, dtype)
        self.o.load(tensors["wo"], tensors.get("bo") if self.has_bias else None, device, dtype)
        self.position.prepare(device)

    def linears(self):
        return [self.qkv, self.o]

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(self.Hkv, self.hs, self.window))

    def wants_deferred_norm(self, ctx, rows: int) -> bool:
        """With more rows than the fused product takes, the norm's factor can only go into the decode kernel that
        rotates by itself (forward); a prompt step is better served by the plain norm."""
        if rows <= ops.FUSED_ROWS:
            return True
        fuse_ok, inv_freq = self.position.fusable(self.hs)
        return bool(ctx.is_decode and fuse_ok and inv_freq is not None and not self.has_bias and ops.LIBRARY_PRODUCTS
                    and ops.can_fuse_decode(self.qkv.weight.dtype, self.H, self.Hkv, self.hs))

    def forward(self, h, ctx, kv, lazy_ok: bool = False):
        H, Hkv, hs = self.H, self.Hkv, self.hs
        last = self.o.lazy if lazy_ok else self.o
        fuse_ok, inv_freq = self.position.fusable(hs)
        vt, blocked = kv.v_transposed, bool(kv.blocked)
        decode_fused = (ctx.is_decode and fuse_ok and ops.can_fuse_decode(self.qkv.weight.dtype, H, Hkv, hs)
                        and blocked)                            # the matrix-core kernels read blocked pages
        row_scale = None
        if isinstance(h, ops.DeferredNorm) and h.shape[0] > ops.FUSED_ROWS:
            # More rows than the fused product takes.  When the decode kernel rotates by itself it can apply the norm's
            # factor as well (it multiplies whole rows of q, k and v): the library's product of the copy, then that
            # kernel.  Else the norm is applied the plain way.
            if decode_fused and inv_freq is not None and not self.has_bias and kv.writes and ops.LIBRARY_PRODUCTS:
                row_scale, h = h, h.scaled
            else:
                h = h.materialize()
        if kv.writes:
            qkv = self.qkv(h)                                   # [T, (H + 2 Hkv) hs]
        else:
            qkv = self.qkv(h, rows=slice(0, self.q_dim))        # Q alone
            pad = torch.empty((h.shape[0], (H + 2 * Hkv) * hs), dtype=h.dtype, device=h.device)
            pad[:, :self.q_dim] = qkv
            qkv = pad
        out = torch.empty((h.shape[0], self.q_dim), dtype=h.dtype, device=h.device)
        if decode_fused:
            # one kernel: rotation of Q and the new K, the cache write, attention, merge of the splits
            if self.window:
                n_splits, chunk = 1, 0
            else:
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, kv.max_len, h.dtype)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, seq_lens=ctx.seq_lens, n_splits=n_splits, chunk=chunk,
                          fused_rotate=inv_freq, fused_write=kv.writes, by_length=ctx.by_length,
                          max_len_dev=ctx.max_len_dev if n_splits > 1 else None, v_transposed=vt, blocked=blocked,
                          row_scale=row_scale)
            return last(out)
        self.position.encode_and_store(qkv, ctx, H, Hkv, hs, kv)
        if ctx.is_decode:
            if self.window:                   # a window is short; its keys are not split
                n_splits, chunk = 1, 0
            else:
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, kv.max_len, h.dtype)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, seq_lens=ctx.seq_lens, n_splits=n_splits, chunk=chunk,
                          by_length=ctx.by_length, max_len_dev=ctx.max_len_dev if n_splits > 1 else None,
                          v_transposed=vt, blocked=blocked)
        else:
            # pages in another order than the matrix-core kernels' own: the vector kernel, with its tiles
            _, _, qt = ops.attention_row_shape(H, Hkv, False, h.dtype if blocked else None, hs)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, tiles=ctx.tiles(qt), qt=qt, v_transposed=vt, blocked=blocked)
        return last(out)
