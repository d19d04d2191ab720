"""Each HIP kernel alone against the plain implementation (or the formula written out in
float64), at other sizes than the engine tests use."""
import math
import random

import pytest
import torch

import plain_llama as pl
from conftest import rel_err

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
KTOL = {torch.float32: 2e-5}      # float32 kernels differ from the formula by summation order only


def close(got, ref, dtype) -> bool:
    """A kernel computes in float32 and rounds its result once to `dtype`.  float32: the largest
    difference is below 2e-5 of the reference's rms.  bfloat16: every element is within one
    rounding (2^-8 of its own size) of the reference, plus the float32 slack."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    rms = float(ref.pow(2).mean().sqrt()) if ref.numel() else 0.0
    slack = 2e-5 * max(rms, 1e-30)
    if dtype == torch.float32:
        return bool(((got - ref).abs() <= slack).all())
    return bool(((got - ref).abs() <= ref.abs() * 2.0 ** -8 + slack).all())


def _ops():
    from bitnet_c_amd import ops
    return ops


def _rand(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim,vocab", [(40, 19), (4096, 33), (1003, 7)])
def test_embed_gather(dtype, dim, vocab):
    ops = _ops()
    table = _rand((vocab, dim), dtype, 1)
    toks = torch.tensor([0, vocab - 1, 3, 3, 1], dtype=torch.int32)
    x = ops.embed_gather(table.cuda(), toks.cuda())
    assert x.dtype == torch.float32
    assert torch.equal(x.cpu(), table[toks.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [24, 100, 4096, 5123, 8192, 9000])
def test_add_rmsnorm(dtype, dim):
    ops = _ops()
    T, eps = 5, 1e-3
    x = _rand((T, dim), torch.float32, 2, 3.0)
    d = _rand((T, dim), dtype, 3)
    w = _rand((dim,), torch.float32, 4) + 1.0
    # without delta
    xg = x.cuda()
    h = ops.add_rmsnorm(xg, None, w.cuda(), eps, dtype)
    assert torch.equal(xg.cpu(), x)
    assert close(h.float(), pl.rmsnorm(x, w, eps), dtype)
    # with delta: x is updated in place in float32, the norm is of the sum
    xg = x.clone().cuda()
    h = ops.add_rmsnorm(xg, d.cuda(), w.cuda(), eps, dtype)
    s = x + d.float()
    assert torch.equal(xg.cpu(), s)
    assert close(h.float(), pl.rmsnorm(s, w, eps), dtype)
    # selected rows: x stays, the selected rows are normed with the delta added
    rows = torch.tensor([4, 0, 0], dtype=torch.int32)
    xg = x.clone().cuda()
    h = ops.add_rmsnorm(xg, d.cuda(), w.cuda(), eps, dtype, rows=rows.cuda())
    assert torch.equal(xg.cpu(), x)
    assert close(h.float(), pl.rmsnorm(s[rows.long()], w, eps), dtype)


def test_rmsnorm_eps_inside_root_on_device():
    ops = _ops()
    x = torch.full((1, 8), 1e-4)
    h = ops.add_rmsnorm(x.cuda(), None, torch.ones(8).cuda(), 1e-2, torch.float32)
    assert torch.allclose(h.cpu(), x / math.sqrt(1e-8 + 1e-2), rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_swiglu_bias_residual(dtype):
    ops = _ops()
    for T, F in ((7, 173), (5, 176), (300, 1024)):
        gu = _rand((T, 2 * F), dtype, 5, 2.0)
        out = ops.swiglu(gu.cuda())
        want = pl.swiglu(gu[:, :F].float(), gu[:, F:].float())
        assert close(out.float(), want, dtype), (T, F)
        if F % 8 == 0:
            gi = torch.stack([gu[:, :F].reshape(T, F // 8, 8), gu[:, F:].reshape(T, F // 8, 8)], dim=2).reshape(T, 2 * F)
            assert torch.equal(ops.swiglu(gi.contiguous().cuda(), True).cpu(), out.cpu()), (T, F)
    T = 7
    # the reference's own vector (test/test_transformer.c:645-677)
    g = torch.tensor([-2.0, -1.0, -0.25, 0.0, 0.25, 1.0, 2.0, 4.0])
    u = torch.tensor([1.0, 0.5, 2.0, 3.0, -1.0, 1.5, -0.5, 2.0])
    o = ops.swiglu(torch.cat([g, u]).view(1, 16).cuda())
    assert torch.allclose(o.cpu()[0], (g / (1 + torch.exp(-g))) * u, atol=1e-6)
    y = _rand((T, 50), dtype, 6)
    b = _rand((50,), torch.float32, 7)
    yg = y.clone().cuda()
    ops.bias_add(yg, b.cuda())
    assert close(yg.float(), y.float() + b, dtype)
    x = _rand((T, 50), torch.float32, 8)
    xg = x.clone().cuda()
    ops.residual_add(xg, y.cuda())
    assert torch.equal(xg.cpu(), x + y.float())


# ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 70, 172), (17, 130, 65), (70, 33, 300), (130, 257, 64)])
def test_gemm_tiled_float32(M, N, K):
    ops = _ops()
    x, w = _rand((M, K), torch.float32, 9), _rand((N, K), torch.float32, 10)
    y = ops.linear(x.cuda(), w.cuda())
    assert rel_err(y, (x.double() @ w.double().t()).float()) < 2e-6
    # a row's result does not depend on its batch: bit-equal alone and among others
    y1 = ops.linear(x[:1].contiguous().cuda(), w.cuda())
    assert torch.equal(y1.cpu()[0], y.cpu()[0])


@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(16, 8), (100, 64), (48, 1000), (4104, 4096), (31, 264)])
def test_skinny_gemm_bf16(M, N, K):
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 11), _rand((N, K), torch.bfloat16, 12, 0.05)
    ref = x.double() @ w.double().t()
    for lib in (True, False):                                     # above 16 rows: the library, or this kernel
        y32 = ops.linear(x.cuda(), w.cuda(), torch.float32, allow_library=lib)
        assert y32.dtype == torch.float32
        assert rel_err(y32, ref.float()) < 1e-5                   # bf16 products are exact in float32
        y16 = ops.linear(x.cuda(), w.cuda(), allow_library=lib)
        assert y16.dtype == torch.bfloat16 and close(y16.float(), ref.float(), torch.bfloat16)


@pytest.mark.parametrize("M", [1, 2, 5, 8, 9, 16])
@pytest.mark.parametrize("D,F", [(64, 40), (4096, 1024), (200, 328), (136, 16), (8192, 64)])
def test_products_with_the_norm_folded_in(M, D, F):
    """A part's last product adds itself to the stream and leaves the next norm deferred (the stream's
    bf16 copy times the norm's weights, sums of squares in parts); the next part's first product, plain
    or with the SwiGLU epilogue, applies it.  Against the plain formulas: the stream exactly (float32),
    the products within the rounding of their bf16 inputs and output."""
    ops = _ops()
    eps = 1e-5
    stream = _rand((M, D), torch.float32, 31, 2.0)
    act = _rand((M, F), torch.bfloat16, 32)
    w_out = _rand((D, F), torch.bfloat16, 33, 0.1)                   # the part's last product: F -> D
    norm_w = (_rand((D,), torch.float32, 34) * 0.2 + 1.0)
    w_in = _rand((2 * F, D), torch.bfloat16, 35, 0.05)               # the next part's first product: D -> F (gate, up)
    assert ops.can_defer_norm(M, D, F, torch.bfloat16)
    x = stream.clone().cuda()
    pre = ops.linear_into_stream(act.cuda(), w_out.cuda(), x, norm_w.cuda(), eps)
    want_x = stream.double() + act.double() @ w_out.double().t()
    assert rel_err(x, want_x.float()) < 1e-5                         # the stream itself: float32
    assert pre.scaled.dtype == torch.bfloat16 and close(pre.scaled.float(), (want_x * norm_w.double()).float(), torch.bfloat16)
    assert rel_err(pre.slots.sum(dim=1), want_x.pow(2).sum(dim=1).float()) < 1e-5
    # the plain path from the same stream: norm kernel, then the product
    h = ops.add_rmsnorm(x, None, norm_w.cuda(), eps, torch.bfloat16)
    assert torch.equal(pre.materialize(), h)
    exact_h = pl.rmsnorm(want_x.float(), norm_w, eps).double()
    exact = exact_h @ w_in[:F].double().t()
    got = ops.linear_prenorm(pre, w_in[:F].cuda().contiguous())
    classic = ops.linear(h, w_in[:F].cuda().contiguous())
    # both round the activations to bf16 once (at different places) and the result once: the fused product is
    # not further from the exact result than twice the plain one, plus one rounding of the result
    e_got, e_classic = rel_err(got.float(), exact.float()), rel_err(classic.float(), exact.float())
    assert e_got <= 2.0 * e_classic + 2.0 ** -7, (e_got, e_classic)
    if F % 8 == 0:
        wi = ops.interleave_gate_up(w_in[:F].cuda(), w_in[F:].cuda())
        g, u = exact_h @ w_in[:F].double().t(), exact_h @ w_in[F:].double().t()
        exact_glu = ((g / (1 + torch.exp(-g))) * u).float()
        got = ops.linear_swiglu_prenorm(pre, wi)
        classic = ops.linear_swiglu(h, wi, True)
        e_got, e_classic = rel_err(got.float(), exact_glu), rel_err(classic.float(), exact_glu)
        assert e_got <= 2.0 * e_classic + 2.0 ** -7, (e_got, e_classic)
    # a second product into the same stream (the next part's last one) keeps adding
    act2 = _rand((M, F), torch.bfloat16, 36)
    pre2 = ops.linear_into_stream(act2.cuda(), w_out.cuda(), x, norm_w.cuda(), eps)
    want_x2 = want_x + act2.double() @ w_out.double().t()
    assert rel_err(x, want_x2.float()) < 1e-5
    assert rel_err(pre2.slots.sum(dim=1), want_x2.pow(2).sum(dim=1).float()) < 1e-5


def test_products_with_the_norm_folded_in_refuse_what_they_cannot_take():
    ops = _ops()
    assert not ops.can_defer_norm(17, 64, 64, torch.bfloat16)              # more than one tile of rows
    assert not ops.can_defer_norm(8, 64, 64, torch.float32)
    assert not ops.can_defer_norm(8, 16 * 513, 64, torch.bfloat16)         # more column tiles than a consumer adds up
    x = torch.zeros(17, 64, device="cuda")
    with pytest.raises(ops.KernelError):
        ops.linear_into_stream(torch.zeros(17, 64, dtype=torch.bfloat16, device="cuda"),
                               torch.zeros(64, 64, dtype=torch.bfloat16, device="cuda"), x, torch.ones(64, device="cuda"), 1e-5)


@pytest.mark.parametrize("M", [1, 17, 33, 64, 100, 128])
@pytest.mark.parametrize("N,K", [(4096, 4096), (200, 328), (72, 1000), (136, 16), (264, 3592), (4096, 14336)])
def test_products_left_as_partial_sums(M, N, K):
    """A product left as float32 partial sums over ranges of K, which the kernel of the next norm (or the plain add)
    adds to the stream in slab order (the dispatcher does so for a part's last product from 17 to 128 rows when K is
    at least twice N, or at least N for widths up to 4,096; the kernel takes 1 to 128 rows of any shape), among them
    the last product of a feed-forward of the 8B shape (4,096 x 14,336).  The sums are exact up to their order; the
    norm is the plain formula on the sum."""
    ops = _ops()
    eps = 1e-6
    x, w = _rand((M, K), torch.bfloat16, 41), _rand((N, K), torch.bfloat16, 42, 0.05)
    stream = _rand((M, N), torch.float32, 43, 2.0)
    norm_w = _rand((N,), torch.float32, 44) * 0.2 + 1.0
    ref = x.double() @ w.double().t()
    assert ops.can_split_sums(M, N, K, torch.bfloat16) == (17 <= M <= 128 and K % 8 == 0 and (K >= 2 * N or (K >= N and N <= 4096)))
    parts = ops.linear_partial_sums(x.cuda(), w.cuda())
    assert parts.slabs.dtype == torch.float32 and tuple(parts.shape) == (M, N)
    assert rel_err(parts.slabs.sum(dim=0), ref.float()) < 1e-5
    # rows of a larger buffer (a row stride above K), as a part's activations may come
    xw = torch.zeros(M, K + 24, dtype=torch.bfloat16)
    xw[:, :K] = x
    assert torch.equal(ops.linear_partial_sums(xw.cuda()[:, :K], w.cuda()).slabs, parts.slabs)
    want_x = stream.double() + ref
    for out_dtype in (torch.bfloat16, torch.float32):
        xs = stream.clone().cuda()
        h = ops.add_rmsnorm(xs, parts, norm_w.cuda(), eps, out_dtype)
        assert rel_err(xs, want_x.float()) < 1e-5                                  # the stream took the sum
        assert h.dtype == out_dtype and close(h.float(), pl.rmsnorm(want_x.float(), norm_w, eps), out_dtype)
    # only some rows normed: the stream stays as it is
    rows = torch.tensor([M - 1, 0, M // 2], dtype=torch.int32)
    xs = stream.clone().cuda()
    h = ops.add_rmsnorm(xs, parts, norm_w.cuda(), eps, torch.float32, rows.cuda())
    assert torch.equal(xs.cpu(), stream)
    assert close(h, pl.rmsnorm(want_x.float(), norm_w, eps)[rows.long()], torch.float32)
    xs = stream.clone().cuda()
    ops.residual_add(xs, parts)
    assert rel_err(xs, want_x.float()) < 1e-5


@pytest.mark.parametrize("M", [17, 64, 128])
@pytest.mark.parametrize("D", [4096, 264, 5120])
@pytest.mark.parametrize("kind", ["none", "bf16", "f32", "slabs"])
def test_a_norm_left_to_its_consumer(M, D, kind):
    """sum_deferred: the stream takes what a part has produced (nothing, a tensor, or partial sums), and a consumer
    gets the bf16 copy of the new stream times the norm's weights with the rows' sums of squares in pieces.  What
    the consumers make of it is the plain norm: materialize(), and the gated unit whose kernel applies the factor
    to a product of the copy (act(s g) * (s u), s = 1/sqrt(mean + eps))."""
    ops = _ops()
    eps = 1e-5
    stream = _rand((M, D), torch.float32, 61, 2.0)
    norm_w = _rand((D,), torch.float32, 62) * 0.2 + 1.0
    delta, add = None, torch.zeros(M, D, dtype=torch.float64)
    if kind == "bf16":
        delta = _rand((M, D), torch.bfloat16, 63)
        add = delta.double()
        delta = delta.cuda()
    elif kind == "f32":
        delta = _rand((M, D), torch.float32, 63)
        add = delta.double()
        delta = delta.cuda()
    elif kind == "slabs":
        slabs = _rand((3, M, D), torch.float32, 63)
        add = slabs.double().sum(dim=0)
        delta = ops.PartialSums(slabs.cuda())
    want_x = (stream.double() + add).float()
    xs = stream.clone().cuda()
    pre = ops.sum_deferred(xs, delta, norm_w.cuda(), eps)
    assert rel_err(xs, want_x) < 1e-6
    assert tuple(pre.scaled.shape) == (M, D) and pre.scaled.dtype == torch.bfloat16
    assert tuple(pre.slots.shape) == (M, (D + 1023) // 1024)
    assert close(pre.scaled.float(), want_x * norm_w, torch.bfloat16)
    assert rel_err(pre.slots.sum(dim=1), want_x.double().pow(2).sum(dim=1).float()) < 1e-5
    normed = pl.rmsnorm(want_x, norm_w, eps)
    assert close(pre.materialize().float(), normed, torch.bfloat16)
    # the gated unit over a product of the copy: 2F columns, gate and up interleaved in blocks of 8
    F = 48
    gu = _rand((M, 2 * F), torch.bfloat16, 64, 3.0)
    got = ops.swiglu_scaled(gu.cuda(), pre, "silu")
    sc = 1.0 / torch.sqrt(want_x.double().pow(2).mean(dim=1) + eps)
    g8 = gu.double().view(M, F // 8, 2, 8) * sc[:, None, None, None]
    want = (g8[:, :, 0] / (1.0 + torch.exp(-g8[:, :, 0])) * g8[:, :, 1]).reshape(M, F)
    assert close(got.float(), want.float(), torch.bfloat16)
    assert ops.can_sum_deferred(M, D, torch.bfloat16) and not ops.can_sum_deferred(16, D, torch.bfloat16)
    assert not ops.can_sum_deferred(M, D, torch.float32)
    with pytest.raises(ops.KernelError):
        ops.sum_deferred(xs, _rand((M, D + 4), torch.bfloat16, 1).cuda(), norm_w.cuda(), eps)


@pytest.mark.parametrize("H,Hkv,hs,n_splits", [(8, 2, 128, 1), (8, 2, 128, 3), (6, 6, 64, 2)])
def test_decode_attention_applies_a_deferred_norm_s_factor(H, Hkv, hs, n_splits):
    """Rows of q, k, v that lack their norm's factor (a product of a deferred norm's copy): the decode kernel that
    rotates and stores by itself multiplies it in.  With factors that are powers of two nothing is rounded
    differently, so the output and the stored keys and values equal, bit for bit, those of the same rows with the
    factor applied beforehand."""
    ops = _ops()
    dtype = torch.bfloat16
    lens = [1, 64, 65, 300, 190]
    B = len(lens)
    seqs_k = [_rand((l, Hkv, hs), dtype, 70 + i) for i, l in enumerate(lens)]
    seqs_v = [_rand((l, Hkv, hs), dtype, 80 + i) for i, l in enumerate(lens)]
    kp, vp, bt = _paged(seqs_k, seqs_v, dtype, sum((l + 63) // 64 for l in lens) + 2, 90)
    qkv = _rand((B, (H + 2 * Hkv) * hs), dtype, 91)
    factor = torch.tensor([0.5, 2.0, 4.0, 0.25, 1.0])
    raw = (qkv.float() / factor[:, None]).to(dtype)
    assert torch.equal((raw.float() * factor[:, None]).to(dtype), qkv)
    slots = torch.zeros(B, 3)
    slots[:, 1] = 4.0 / factor ** 2                            # width 4, eps 0: 1 / sqrt(sum of the slots / 4) is the factor
    pre = ops.DeferredNorm(raw.cuda(), slots.cuda(), torch.zeros(B, 4).cuda(), None, 0.0)
    inv = pl.rope_inv_freq(hs, 10000.0).cuda()
    d_lens = torch.tensor(lens, dtype=torch.int32).cuda()
    chunk = ((bt.shape[1] + n_splits - 1) // n_splits) * 64
    outs = []
    for rows, rs in ((qkv, None), (raw, pre)):
        k_pages, v_pages = kp.clone().cuda(), vp.clone().cuda()
        out = torch.full((B, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(rows.cuda(), out, k_pages, v_pages, bt.cuda(), H, Hkv, hs, hs ** -0.5, seq_lens=d_lens,
                      n_splits=n_splits, chunk=chunk if n_splits > 1 else 0, fused_rotate=inv, fused_write=True, row_scale=rs)
        outs.append((out.cpu(), k_pages.cpu(), v_pages.cpu()))
    for a, b in zip(*outs):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))        # bits: the pages hold NaN where nothing was written
    assert not bool(outs[0][0].isnan().any())
    with pytest.raises(ops.KernelError):                                       # only where the kernel rotates by itself
        ops.attention(raw.cuda(), out, k_pages, v_pages, bt.cuda(), H, Hkv, hs, hs ** -0.5, seq_lens=d_lens, row_scale=pre)


def test_partial_sums_refuse_what_they_cannot_take():
    ops = _ops()
    assert ops.can_split_sums(64, 64, 128, torch.bfloat16) and ops.can_split_sums(128, 64, 512, torch.bfloat16)
    assert ops.can_split_sums(17, 64, 128, torch.bfloat16) and ops.can_split_sums(64, 64, 64, torch.bfloat16)
    assert not ops.can_split_sums(16, 64, 128, torch.bfloat16) and not ops.can_split_sums(129, 64, 128, torch.bfloat16)
    assert not ops.can_split_sums(64, 64, 56, torch.bfloat16)              # K below N
    assert not ops.can_split_sums(64, 5120, 5120, torch.bfloat16)          # a square product wider than the rule's bound
    assert ops.can_split_sums(64, 8192, 16384, torch.bfloat16)             # K twice N: any width
    assert not ops.can_split_sums(64, 64, 172, torch.bfloat16) and not ops.can_split_sums(64, 64, 128, torch.float32)
    z = lambda *shape: torch.zeros(*shape, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ops.KernelError):
        ops.linear_partial_sums(z(129, 64), z(64, 64))                 # more rows than the staged block holds
    with pytest.raises(ops.KernelError):
        ops.linear_partial_sums(z(32, 172), z(64, 172))                # K no multiple of 8
    with pytest.raises(ops.KernelError):
        ops.linear_partial_sums(z(32, 64), z(64, 72))                  # K of x and w differ
    parts = ops.linear_partial_sums(z(32, 64), z(48, 64))
    with pytest.raises(ops.KernelError):
        ops.add_rmsnorm(torch.zeros(32, 64, device="cuda"), parts, torch.ones(64, device="cuda"), 1e-5, torch.bfloat16)
    with pytest.raises(ops.KernelError):
        ops.residual_add(torch.zeros(31, 48, device="cuda"), parts)


@pytest.mark.parametrize("width", [0, 256, 192, 128])
@pytest.mark.parametrize("M,N,K", [(65, 16, 8), (100, 200, 328), (256, 256, 64), (300, 520, 192), (777, 1000, 136),
                                   (513, 4104, 1032), (1, 31, 264)])
def test_gemm_mfma(M, N, K, width):
    """The tiled matrix-core product, every tile width, at sizes that fill no tile: float32 results are
    the exact sums up to their order, bf16 results one rounding of them."""
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 21), _rand((N, K), torch.bfloat16, 22, 0.05)
    ref = (x.double() @ w.double().t()).float()
    y32 = ops.gemm_mfma(x.cuda(), w.cuda(), torch.float32, width=width)
    y16 = ops.gemm_mfma(x.cuda(), w.cuda(), width=width)
    # rows of a larger buffer (a row stride above K), as the stacked projections pass them
    xw = torch.zeros(M, K + 24, dtype=torch.bfloat16)
    xw[:, :K] = x
    y_strided = ops.gemm_mfma(xw.cuda()[:, :K], w.cuda(), torch.float32, width=width)
    assert y32.dtype == torch.float32 and rel_err(y32, ref) < 1e-5
    assert y16.dtype == torch.bfloat16 and close(y16.float(), ref, torch.bfloat16)
    assert torch.equal(y_strided, y32)
    # through the dispatcher: without the library, more than 64 rows take this kernel
    if M > 64:
        assert torch.equal(ops.linear(x.cuda(), w.cuda(), torch.float32, allow_library=False), y32)


@pytest.mark.parametrize("width", [0, 256, 192, 128])
@pytest.mark.parametrize("M,F,K", [(65, 8, 8), (100, 328, 120), (300, 1000, 512), (260, 2056, 264)])
def test_gemm_mfma_swiglu(M, F, K, width):
    """The same kernel with gate and up rows interleaved in blocks of 8 and the SwiGLU epilogue."""
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 23), _rand((2 * F, K), torch.bfloat16, 24, 0.1)
    g = x.double() @ w[:F].double().t()
    u = x.double() @ w[F:].double().t()
    want = ((g / (1 + torch.exp(-g))) * u).float()
    wi = ops.interleave_gate_up(w[:F].cuda(), w[F:].cuda())
    y32 = ops.gemm_mfma(x.cuda(), wi, torch.float32, glu8=True, width=width)
    y16 = ops.gemm_mfma(x.cuda(), wi, glu8=True, width=width)
    via = ops.linear_swiglu(x.cuda(), wi, True, allow_library=False)
    assert y32.shape == (M, F) and close(y32, want, torch.float32)
    assert close(y16.float(), want, torch.bfloat16)
    if M > 128:                                    # up to 128 rows the dispatcher has another kernel for this product
        assert torch.equal(via, y16)
    else:
        assert close(via.float(), want, torch.bfloat16)


@pytest.mark.parametrize("M", [1, 17, 24, 33, 48, 100, 128])
@pytest.mark.parametrize("F,K", [(8, 8), (328, 120), (1000, 512), (520, 4096), (136, 16)])
def test_swiglu_product_with_staged_activations(M, F, K):
    """The gate/up product of up to 128 rows with the SwiGLU epilogue (gate and up rows interleaved in blocks of 8,
    activations staged once per workgroup): against the exact result, and that the dispatcher uses it when it may
    not call the library."""
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 51), _rand((2 * F, K), torch.bfloat16, 52, 0.1)
    g = x.double() @ w[:F].double().t()
    u = x.double() @ w[F:].double().t()
    want = ((g / (1 + torch.exp(-g))) * u).float()
    wi = ops.interleave_gate_up(w[:F].cuda(), w[F:].cuda())
    xd = x.cuda()
    y = torch.full((M, F), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = ops._fn("splitk_gemm", "bn_splitk_gemm_swiglu")(xd.data_ptr(), wi.data_ptr(), y.data_ptr(), M, F, K, K, K, F,
                                                         ops.ACTIVATIONS["silu"], None, 0, 0, 0.0, 0,
                                                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert close(y.float(), want, torch.bfloat16)
    lo, hi = ops.SWIGLU_STAGED_ROWS
    if lo <= M <= hi:                              # without the library this is the kernel of these row counts
        assert torch.equal(ops.linear_swiglu(xd, wi, True, allow_library=False), y)
    # over the streamed copy of the weights (other workgroup sizes, the same sums): the same bits
    ws = ops.stream_copy(wi, 16)
    y2 = torch.full((M, F), float("nan"), dtype=torch.bfloat16, device="cuda")
    rc = ops._fn("splitk_gemm", "bn_splitk_gemm_swiglu")(xd.data_ptr(), ws.tiles.data_ptr(), y2.data_ptr(), M, F, K, K, ws.k_tiles,
                                                         F, ops.ACTIVATIONS["silu"], None, 0, 0, 0.0, 1,
                                                         torch.cuda.current_stream().cuda_stream)
    assert rc == 0 and torch.equal(y2, y)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 50, 64, 128])
@pytest.mark.parametrize("D,F", [(264, 328), (4096, 520), (1000, 136), (5120, 64)])
def test_staged_swiglu_product_applies_a_deferred_norm(M, D, F):
    """The staged gate/up product takes a deferred norm: its activations are the stream's bf16 copy times the norm's
    weights, and the rows' 1/sqrt(mean + eps), from sums of squares that arrive in parts (many parts of few columns as
    the fused product of up to 16 rows leaves them, few parts of 1,024 columns as sum_deferred does), multiplies gate
    and up in the epilogue.  Against the plain formulas on the same stream, over the row-major weights and over their
    streamed copy (the same bits); and the dispatcher's own choice gives a result of the same accuracy."""
    ops = _ops()
    eps = 1e-5
    stream = _rand((M, D), torch.float32, 91, 2.0)
    norm_w = _rand((D,), torch.float32, 92) * 0.2 + 1.0
    w = _rand((2 * F, D), torch.bfloat16, 93, 0.05)
    x = stream.clone().cuda()
    if M <= 16:
        act, w_out = _rand((M, 64), torch.bfloat16, 94), _rand((D, 64), torch.bfloat16, 95, 0.1)
        pre = ops.linear_into_stream(act.cuda(), w_out.cuda(), x, norm_w.cuda(), eps)
        want_x = stream.double() + act.double() @ w_out.double().t()
    else:
        delta = _rand((M, D), torch.bfloat16, 94)
        pre = ops.sum_deferred(x, delta.cuda(), norm_w.cuda(), eps)
        want_x = stream.double() + delta.double()
    h = pl.rmsnorm(want_x.float(), norm_w, eps).double()
    g, u = h @ w[:F].double().t(), h @ w[F:].double().t()
    exact = ((g / (1 + torch.exp(-g))) * u).float()
    wi = ops.interleave_gate_up(w[:F].cuda(), w[F:].cuda())
    got = ops._staged_swiglu(pre.scaled, wi, pre, "silu")
    assert got is not None and got.dtype == torch.bfloat16
    classic = ops.linear_swiglu(pre.materialize(), wi, True)
    e_got, e_classic = rel_err(got.float(), exact), rel_err(classic.float(), exact)
    assert e_got <= 2.0 * e_classic + 2.0 ** -7, (e_got, e_classic)
    assert torch.equal(ops._staged_swiglu(pre.scaled, wi, pre, "silu", ops.stream_copy(wi, 16)), got)
    routed = ops.linear_swiglu_prenorm(pre, wi) if (M <= 16 or ops.LIBRARY_PRODUCTS) else got
    assert rel_err(routed.float(), exact) <= 2.0 * e_classic + 2.0 ** -7


def test_the_streamed_copy_is_the_lanes_order():
    """The streamed copy of a weight matrix by its definition: tile (a, b) holds rows R a .. R a + R - 1 and columns
    32 b .. 32 b + 31 (R rows a tile, at most 16), lane l = r + 16 g of a wave (r < R) gets elements 8 (R g + r) .. + 7 of the
    tile, which are columns 8 g .. 8 g + 7 of row r; rows past N and columns past K are zero; unstream gives the matrix
    back.  The height that a matrix gets unasked is the one that spreads its tiles evenly over the CUs."""
    ops = _ops()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert ops.stream_tile_rows(16 * cus) == 16 and ops.stream_tile_rows(16 * cus * 7) == 16
    assert ops.stream_tile_rows(24 * cus) == 12 and ops.stream_tile_rows(20 * cus) == 10      # 6,144 and 5,120 on 256 CUs
    for N, K, R in ((31, 264, 16), (48, 64, 12), (100, 1000, 10), (16, 8, 16), (50, 96, 7), (6144, 64, None)):
        w = _rand((N, K), torch.bfloat16, 71, 0.5).cuda()
        sw = ops.stream_copy(w, R)
        R = R or ops.stream_tile_rows(N)
        nt, kt = (N + R - 1) // R, (K + 31) // 32
        assert tuple(sw.tiles.shape) == (nt, kt, 32 * R) and (sw.N, sw.K, sw.k_tiles, sw.tile_rows) == (N, K, kt, R)
        assert sw.nbytes() == nt * kt * 64 * R
        assert torch.equal(ops.unstream(sw), w)
        t, wc = sw.tiles.cpu(), w.cpu()
        for a, b, r, g in ((0, 0, 0, 0), (nt - 1, kt - 1, R - 1, 3), (nt - 1, 0, 1, 1), (0, kt - 1, R // 2, 2), (nt // 2, kt // 2, 5, 0)):
            row, col = R * a + r, 32 * b + 8 * g
            want = torch.zeros(8, dtype=torch.bfloat16)
            if row < N and col < K:
                n = min(8, K - col)
                want[:n] = wc[row, col:col + n]
            at = 8 * (R * g + r)
            assert torch.equal(t[a, b, at:at + 8], want), (N, K, R, a, b, r, g)
    with pytest.raises(ops.KernelError):                   # a copy of another matrix
        ops.linear(torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda"), torch.zeros(32, 64, dtype=torch.bfloat16, device="cuda"),
                   streamed=ops.stream_copy(torch.zeros(48, 64, dtype=torch.bfloat16, device="cuda")))
    with pytest.raises(ops.KernelError):
        ops.stream_copy(torch.zeros(48, 64, dtype=torch.bfloat16, device="cuda"), 17)


@pytest.mark.parametrize("M", [1, 8, 16, 17, 64, 128])
@pytest.mark.parametrize("N,K,R", [(100, 64, 16), (48, 1000, 12), (264, 3592, 10), (4104, 4096, 16), (31, 264, 7), (4096, 14336, None),
                                   (6144, 512, None)])
def test_products_over_the_streamed_copy_are_the_same_bits(M, N, K, R):
    """Every product that takes a streamed copy of its weights forms the same sums in the same order as over the
    row-major matrix: the plain product of up to 16 rows (bf16 and float32 results), the products with a norm folded
    in (before, after, with the gated unit), and the partial sums of up to 128 rows.  N and K that are no multiples
    of the tile's rows and 32 columns among them, tiles of 7 to 16 rows, and the height a matrix gets unasked."""
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 81).cuda(), _rand((N, K), torch.bfloat16, 82, 0.05).cuda()
    sw = ops.stream_copy(w, R)
    a, b = ops.linear_partial_sums(x, w), ops.linear_partial_sums(x, w, sw)
    if a.slabs.shape == b.slabs.shape:
        assert torch.equal(a.slabs, b.slabs)
    else:                           # narrower tiles, more workgroups along the columns, other ranges of K: the same sum
        assert rel_err(b.slabs.sum(dim=0), a.slabs.sum(dim=0)) < 1e-6
    if M > 16:
        return
    for out in (torch.bfloat16, torch.float32):
        assert torch.equal(ops.linear(x, w, out), ops.linear(x, w, out, streamed=sw))
    if N > 16 * 512:
        return
    eps = 1e-5
    norm_w = (_rand((N,), torch.float32, 83) * 0.2 + 1.0).cuda()
    s1, s2 = _rand((M, N), torch.float32, 84, 2.0).cuda(), _rand((M, N), torch.float32, 84, 2.0).cuda()
    p1 = ops.linear_into_stream(x, w, s1, norm_w, eps)
    p2 = ops.linear_into_stream(x, w, s2, norm_w, eps, sw)
    assert torch.equal(s1, s2) and torch.equal(p1.scaled, p2.scaled)
    assert p2.slots.shape[1] == (N + sw.tile_rows - 1) // sw.tile_rows           # one part per row of tiles
    assert rel_err(p2.slots.sum(dim=1), p1.slots.sum(dim=1)) < 1e-6
    if R is None:                                                  # the copy's own height is the row-major kernel's tile
        assert torch.equal(p1.slots, p2.slots)
    # the next product reads either norm; its own weights streamed or not
    if N % 8 == 0:
        F = 40
        w_in = _rand((2 * F, N), torch.bfloat16, 85, 0.05).cuda()
        si, si16 = ops.stream_copy(w_in, 10), ops.stream_copy(w_in, 16)
        for pre in (p1, p2):
            assert torch.equal(ops.linear_prenorm(pre, w_in), ops.linear_prenorm(pre, w_in, si))
            # gate and up interleaved: tiles of 16 rows are read, a copy of another height is passed over
            want = ops.linear_swiglu_prenorm(pre, w_in)
            assert torch.equal(want, ops.linear_swiglu_prenorm(pre, w_in, streamed=si16))
            assert torch.equal(want, ops.linear_swiglu_prenorm(pre, w_in, streamed=si))


@pytest.mark.parametrize("activation", ["gelu_tanh", "relu2", "silu"])
def test_every_gated_epilogue_takes_the_activation(activation):
    """The gate's activation is an argument of every kernel that ends in a gated unit: the gated-unit kernel
    itself, the streaming product (both weight layouts), its form with the norm folded in, the product with
    staged activations and the tiled matrix-core product.  Against the plain formula of that activation; and
    the three activations differ from each other by far more than the tolerance."""
    ops = _ops()
    F, K = 328, 264
    w = _rand((2 * F, K), torch.bfloat16, 62, 0.1)
    wi = ops.interleave_gate_up(w[:F].cuda(), w[F:].cuda())

    def want_for(x):
        g, u = x.double() @ w[:F].double().t(), x.double() @ w[F:].double().t()
        return pl.swiglu(g, u, activation).float()

    others = [a for a in ops.ACTIVATIONS if a != activation]
    x8 = _rand((8, K), torch.bfloat16, 61)
    for o in others:
        g, u = x8.double() @ w[:F].double().t(), x8.double() @ w[F:].double().t()
        assert rel_err(pl.swiglu(g, u, o).float(), want_for(x8)) > 0.05
    for dtype in DTYPES:                                                    # the gated-unit kernel, both layouts
        gu = _rand((7, 2 * F), dtype, 63, 2.0)
        want = pl.swiglu(gu[:, :F].float(), gu[:, F:].float(), activation)
        assert close(ops.swiglu(gu.cuda(), False, activation).float(), want, dtype)
        gi = torch.stack([gu[:, :F].reshape(7, F // 8, 8), gu[:, F:].reshape(7, F // 8, 8)], dim=2).reshape(7, 2 * F)
        assert close(ops.swiglu(gi.contiguous().cuda(), True, activation).float(), want, dtype)
    for M in (1, 8, 16, 40):                                                # the streaming product
        x = _rand((M, K), torch.bfloat16, 64 + M)
        assert close(ops.linear_swiglu(x.cuda(), w.cuda(), allow_library=False, activation=activation).float(),
                     want_for(x), torch.bfloat16), M
        assert close(ops.linear_swiglu(x.cuda(), wi, True, allow_library=False, activation=activation).float(),
                     want_for(x), torch.bfloat16), M
    for M in (24, 100):                                                     # staged activations (17 to 128 rows)
        x = _rand((M, K), torch.bfloat16, 70 + M)
        assert close(ops.linear_swiglu(x.cuda(), wi, True, allow_library=False, activation=activation).float(),
                     want_for(x), torch.bfloat16), M
    x = _rand((200, K), torch.bfloat16, 80)                                 # the tiled matrix-core product
    assert close(ops.gemm_mfma(x.cuda(), wi, glu8=True, activation=activation).float(), want_for(x), torch.bfloat16)
    # with the library the product is stored in bf16 first and the gated-unit kernel reads that: against the plain
    # formula on the stored gate and up values
    yl = ops.linear(x.cuda(), wi).float().cpu().reshape(200, F // 8, 2, 8)
    gl, ul = yl[:, :, 0].reshape(200, F), yl[:, :, 1].reshape(200, F)
    assert close(ops.linear_swiglu(x.cuda(), wi, True, activation=activation).float(), pl.swiglu(gl, ul, activation), torch.bfloat16)
    # the norm folded in: a stream, its deferred norm, the gated product that applies it
    M, D = 5, K
    stream = _rand((M, D), torch.float32, 81, 2.0)
    norm_w = _rand((D,), torch.float32, 82) * 0.2 + 1.0
    act_in = _rand((M, 64), torch.bfloat16, 83)
    w_out = _rand((D, 64), torch.bfloat16, 84, 0.1)
    xs = stream.clone().cuda()
    pre = ops.linear_into_stream(act_in.cuda(), w_out.cuda(), xs, norm_w.cuda(), 1e-5)
    h = pl.rmsnorm((stream.double() + act_in.double() @ w_out.double().t()).float(), norm_w, 1e-5)
    exact = want_for(h)
    got = ops.linear_swiglu_prenorm(pre, wi, activation)
    classic = ops.linear_swiglu(pre.materialize(), wi, True, activation=activation)
    e_got, e_classic = rel_err(got.float(), exact), rel_err(classic.float(), exact)
    assert e_got <= 2.0 * e_classic + 2.0 ** -7, (e_got, e_classic)
    with pytest.raises(ops.KernelError):
        ops.swiglu(_rand((2, 16), torch.float32, 1).cuda(), False, "gelu")


def test_embedding_multiplier_and_logit_softcap_kernels():
    ops = _ops()
    table = _rand((50, 72), torch.bfloat16, 90)
    toks = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    assert torch.equal(ops.embed_gather(table.cuda(), toks.cuda()).cpu(), table[toks.long()].float())
    got = ops.embed_gather(table.cuda(), toks.cuda(), math.sqrt(72.0))
    assert torch.equal(got.cpu(), table[toks.long()].float() * torch.tensor(math.sqrt(72.0), dtype=torch.float32))
    lg = _rand((5, 389), torch.float32, 91, 40.0)
    g = lg.clone().cuda()
    ops.softcap_(g, 30.0)
    assert torch.allclose(g.cpu(), torch.tanh(lg / 30.0) * 30.0, atol=1e-5) and float(g.abs().max()) <= 30.0
    with pytest.raises(ops.KernelError):
        ops.softcap_(g, 0.0)


def test_gemm_mfma_refuses_what_it_cannot_take():
    ops = _ops()
    x, w = _rand((70, 36), torch.bfloat16, 25).cuda(), _rand((16, 36), torch.bfloat16, 26).cuda()
    with pytest.raises(ops.KernelError):
        ops.gemm_mfma(x, w)                               # K is not a multiple of 8
    with pytest.raises(ops.KernelError):
        ops.gemm_mfma(x.float(), w.float())               # bf16 only
    # the check that the dispatcher makes without loading the kernel is the kernel's own
    from bitnet_c_amd.csrc import build
    supports = build.load("gemm_mfma").bn_gemm_mfma_supports
    for M, N, K, ldx, ldw in [(70, 16, 36, 36, 36), (70, 16, 40, 40, 40), (1, 1, 8, 8, 8), (5, 5, 4, 8, 8), (5, 5, 16, 12, 16),
                              (5, 5, 16, 8, 16), (0, 5, 16, 16, 16), (5, 0, 16, 16, 16), (3000, 4104, 4096, 4104, 4096)]:
        assert ops.gemm_mfma_supported(M, N, K, ldx, ldw) == bool(supports(M, N, K, ldx, ldw)), (M, N, K, ldx, ldw)
    # the dispatcher sends such a shape to the plain tiled kernel instead
    y = ops.linear(x, w, allow_library=False)
    assert close(y.float(), (x.double().cpu() @ w.double().cpu().t()).float(), torch.bfloat16)


@pytest.mark.parametrize("M,F,K", [(1, 24, 64), (8, 172, 64), (20, 100, 264), (64, 1000, 512), (40, 14336, 256), (33, 8, 8), (17, 328, 120)])
def test_skinny_gemm_dual_swiglu(M, F, K):
    ops = _ops()
    x, w = _rand((M, K), torch.bfloat16, 13), _rand((2 * F, K), torch.bfloat16, 14, 0.1)
    y = ops.linear_swiglu(x.cuda(), w.cuda(), allow_library=False)
    g = x.double() @ w[:F].double().t()
    u = x.double() @ w[F:].double().t()
    want = ((g / (1 + torch.exp(-g))) * u).float()
    assert close(y.float(), want, torch.bfloat16)
    if F % 8 == 0:          # gate and up rows interleaved in blocks of 8
        wi = ops.interleave_gate_up(w[:F].cuda(), w[F:].cuda())
        assert torch.equal(wi[:8].cpu(), w[:8]) and torch.equal(wi[8:16].cpu(), w[F:F + 8])
        assert close(ops.linear_swiglu(x.cuda(), wi, True, allow_library=False).float(), want, torch.bfloat16)
        xl = _rand((100, K), torch.bfloat16, 15)                    # more than 64 rows: product, then the kernel
        yl = ops.linear(xl.cuda(), wi).float().cpu().reshape(100, F // 8, 2, 8)
        gl, ul = yl[:, :, 0].reshape(100, F), yl[:, :, 1].reshape(100, F)
        assert close(ops.linear_swiglu(xl.cuda(), wi, True).float(), pl.swiglu(gl, ul), torch.bfloat16)
        assert close(gl, (xl.double() @ w[:F].double().t()).float(), torch.bfloat16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_linear_odd_shapes_and_many_rows(dtype):
    ops = _ops()
    for M, N, K in [(3, 50, 172), (100, 70, 172), (200, 96, 64), (130, 40, 100)]:
        x, w = _rand((M, K), dtype, 15), _rand((N, K), dtype, 16, 0.05)
        y = ops.linear(x.cuda(), w.cuda())
        assert close(y.float(), (x.double() @ w.double().t()).float(), dtype), (M, N, K)
        y32 = ops.linear(x.cuda(), w.cuda(), torch.float32)
        assert y32.dtype == torch.float32
        assert rel_err(y32, (x.double() @ w.double().t()).float()) < 1e-5, (M, N, K)
        # float32 logits of a bf16 model at many rows agree with the same rows taken alone
        if dtype == torch.bfloat16 and K % 8 == 0:
            y1 = ops.linear(x[:1].contiguous().cuda(), w.cuda(), torch.float32)
            assert rel_err(y1, y32[:1]) < 1e-6


# ---------------------------------------------------------------------------------------
def _paged(seqs_k, seqs_v, dtype, n_pages, seed, blocked=None):
    """Random distinct pages for every sequence; returns k_pages, v_pages, block_table.  The pages lie as the kernels
    read them unasked at this type and head size (ops.kernel_v_layout); blocked=False: bf16 values transposed, whatever
    the head size (what the vector kernel reads)."""
    Hkv, hs = seqs_k[0].shape[1], seqs_k[0].shape[2]
    if blocked is None:
        blocked = _ops().kernel_v_layout(dtype, hs) == "blocked"
    rnd = random.Random(seed)
    free = list(range(n_pages))
    rnd.shuffle(free)
    # unused pages hold NaN: a kernel that reads a key it must not see shows it
    k_pages = torch.full((n_pages, Hkv, 64, hs), float("nan"), dtype=dtype)
    v_pages = torch.full((n_pages, Hkv, 64, hs), float("nan"), dtype=dtype)
    vt = dtype == torch.bfloat16                      # bf16 caches keep V transposed inside a page
    width = max((k.shape[0] + 63) // 64 for k in seqs_k)
    bt = torch.zeros((len(seqs_k), width), dtype=torch.int32)
    for s, (k, v) in enumerate(zip(seqs_k, seqs_v)):
        for i in range((k.shape[0] + 63) // 64):
            p = free.pop()
            bt[s, i] = p
            n = min(64, k.shape[0] - 64 * i)
            k_pages[p, :, :n] = k[64 * i:64 * i + n].transpose(0, 1).to(dtype)
            v_pages[p, :, :n] = v[64 * i:64 * i + n].transpose(0, 1).to(dtype)
    if vt:
        v_pages = v_pages.transpose(2, 3).contiguous()
    if blocked:
        k_pages, v_pages = _ops().to_blocked_pages(k_pages, v_pages)
    return k_pages, v_pages, bt


def _as_rows(ops, dtype, hs, kp, vp):
    """Pages as the kernels wrote them unasked -> keys as rows, values as rows too (float32 on the host)."""
    layout = ops.kernel_v_layout(dtype, hs)
    if layout == "blocked":
        kp, vp = ops.from_blocked_pages(kp, vp)
    kp, vp = kp.cpu().float(), vp.cpu().float()
    return kp, (vp.transpose(2, 3) if layout != "rows" else vp)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,hs,rope_dims", [(4, 2, 16, 16), (6, 3, 40, 24), (5, 5, 24, 24), (8, 1, 128, 128),
                                                 (2, 2, 256, 64), (8, 2, 64, 32)])
def test_rope_kv_write(dtype, H, Hkv, hs, rope_dims):
    """Rotation and the write into the pages, in the layout that the kernels use unasked at each type and head size
    (rows for float32, transposed values for bf16, blocked pages at the head sizes of the matrix-core kernels)."""
    ops = _ops()
    lens_before, n_new = [0, 70, 130], [5, 1, 66]
    T = sum(n_new)
    qkv = _rand((T, (H + 2 * Hkv) * hs), dtype, 17)
    inv_freq = pl.rope_inv_freq(hs, 10000.0, None, rope_dims)
    positions, seq_index = [], []
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        positions += list(range(p0, p0 + n))
        seq_index += [s] * n
    pos = torch.tensor(positions, dtype=torch.int32)
    n_pages = 12
    bt = torch.tensor([[3, 0, 0, 0], [7, 1, 0, 0], [2, 9, 5, 11]], dtype=torch.int32)
    vt = dtype == torch.bfloat16
    kp = torch.zeros((n_pages, Hkv, 64, hs), dtype=dtype).cuda()
    vp = torch.zeros((n_pages, Hkv, hs, 64) if vt else (n_pages, Hkv, 64, hs), dtype=dtype).cuda()
    q_in = qkv.clone()
    g = qkv.cuda()
    ops.rope_kv_write(g, pos.cuda(), H, Hkv, hs, inv_freq=inv_freq.cuda(), rope_dims=rope_dims,
                      seq_index=torch.tensor(seq_index, dtype=torch.int32).cuda(), block_table=bt.cuda(),
                      k_pages=kp, v_pages=vp)
    q_ref = pl.apply_rope(q_in[:, :H * hs].float().view(T, H, hs), pos, inv_freq)
    k_ref = pl.apply_rope(q_in[:, H * hs:(H + Hkv) * hs].float().view(T, Hkv, hs), pos, inv_freq)
    v_ref = q_in[:, (H + Hkv) * hs:].float().view(T, Hkv, hs)
    assert close(g[:, :H * hs].float().view(T, H, hs), q_ref, dtype)
    assert torch.equal(g[:, H * hs:].cpu(), q_in[:, H * hs:])            # K, V of the input stay as they are
    kp_raw, vp_raw = kp.cpu(), vp.cpu()
    kp, vp = _as_rows(ops, dtype, hs, kp, vp)
    written = torch.zeros((n_pages, 64), dtype=torch.bool)
    for t in range(T):
        page, off = int(bt[seq_index[t], positions[t] // 64]), positions[t] % 64
        written[page, off] = True
        assert close(kp[page, :, off], k_ref[t], dtype), t
        assert torch.equal(vp[page, :, off], v_ref[t].to(dtype).float())
    assert float(kp.transpose(1, 2)[~written].abs().sum()) == 0.0
    assert float(vp.transpose(1, 2)[~written].abs().sum()) == 0.0
    # position -1 is a padding row: nothing is rotated or written; Q-only form leaves the cache alone
    g2 = q_in.clone().cuda()
    kp2 = torch.zeros((n_pages, Hkv, 64, hs), dtype=dtype).cuda()
    ops.rope_kv_write(g2, torch.full((T,), -1, dtype=torch.int32).cuda(), H, Hkv, hs, inv_freq=inv_freq.cuda(),
                      rope_dims=rope_dims, seq_index=torch.zeros(T, dtype=torch.int32).cuda(), block_table=bt.cuda(),
                      k_pages=kp2,
                      v_pages=torch.zeros((n_pages, Hkv, hs, 64) if vt else (n_pages, Hkv, 64, hs), dtype=dtype).cuda())
    assert torch.equal(g2.cpu(), q_in) and float(kp2.abs().sum()) == 0.0
    g3 = q_in.clone().cuda()
    ops.rope_kv_write(g3, pos.cuda(), H, Hkv, hs, inv_freq=inv_freq.cuda(), rope_dims=rope_dims)
    assert torch.equal(g3.cpu(), g.cpu())
    # with the tokens cut at page boundaries, transposed V pages are written in runs of positions: the
    # same bytes (the sequences start at 0, 70, 130: unaligned runs, whole pages and a page's tail)
    from bitnet_c_amd.engine.step import _page_tiles
    tiles = _page_tiles(n_new, lens_before)
    assert sum(t[2] for t in tiles) == T and all(t[3] // 64 == (t[3] + t[2] - 1) // 64 for t in tiles)
    g4 = q_in.clone().cuda()
    kp4 = torch.zeros((n_pages, Hkv, 64, hs), dtype=dtype).cuda()
    vp4 = torch.zeros((n_pages, Hkv, hs, 64) if vt else (n_pages, Hkv, 64, hs), dtype=dtype).cuda()
    ops.rope_kv_write(g4, pos.cuda(), H, Hkv, hs, inv_freq=inv_freq.cuda(), rope_dims=rope_dims,
                      seq_index=torch.tensor(seq_index, dtype=torch.int32).cuda(), block_table=bt.cuda(),
                      k_pages=kp4, v_pages=vp4, page_tiles=torch.tensor(tiles, dtype=torch.int32).cuda())
    assert torch.equal(g4.cpu(), g.cpu()) and torch.equal(kp4.cpu(), kp_raw) and torch.equal(vp4.cpu(), vp_raw)


FAR_POSITIONS = [8191, 8192, 65535, 131071]
LLAMA3_8B_SCALING = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                         original_max_position_embeddings=8192)


def test_blocked_pages_by_their_definition():
    """The order of a blocked page, written out from its definition: a (page, kv head) is two blocks of 32 positions; a
    block's keys are, for each chunk c of 32 dimensions, two tiles of 16 key rows (tile row i: the block's position
    8 (i / 4) + i % 4, and 4 further for the second tile) in which lane i + 16 g holds dimensions 32 c + 8 g .. + 7, 8
    elements a lane and 64 lanes a tile; its values are, for each tile t of 16 dimensions, the lanes i + 16 g holding
    positions 8 g .. 8 g + 7 of dimension 16 t + i.  Conversion there and back; and the kernels agree: what the cache
    write stores into blocked pages reads back as the same keys and values that it stores into plain pages."""
    ops = _ops()
    for hs in (64, 128, 32):
        ki, vi = ops.blocked_page_index(hs)
        assert tuple(ki.shape) == (64, hs) and tuple(vi.shape) == (hs, 64)
        assert sorted(ki.reshape(-1).tolist()) == list(range(64 * hs)) == sorted(vi.reshape(-1).tolist())
        for p, d in ((0, 0), (63, hs - 1), (5, 9), (36, 17), (31, 31), (44, hs - 8), (12, 40 % hs)):
            b, r = divmod(p, 32)
            tile, i = (r // 4) % 2, 4 * (r // 8) + r % 4
            assert 8 * (r // 8) + r % 4 + 4 * tile == r
            c, g, e = d // 32, (d % 32) // 8, d % 8
            assert int(ki[p, d]) == b * 32 * hs + ((2 * c + tile) * 64 + (i + 16 * g)) * 8 + e
            t, i2 = d // 16, d % 16
            g2, e2 = (p % 32) // 8, p % 8
            assert int(vi[d, p]) == b * 32 * hs + (t * 64 + (i2 + 16 * g2)) * 8 + e2
        k = _rand((3, 2, 64, hs), torch.bfloat16, 5)
        v = _rand((3, 2, hs, 64), torch.bfloat16, 6)
        kb, vb = ops.to_blocked_pages(k, v)
        assert kb.shape == k.shape and vb.shape == v.shape and not torch.equal(kb, k)
        k2, v2 = ops.from_blocked_pages(kb, vb)
        assert torch.equal(k2, k) and torch.equal(v2, v)
        assert float(kb[1, 1].reshape(-1)[int(ki[37, 11])]) == float(k[1, 1, 37, 11])
        assert float(vb[2, 0].reshape(-1)[int(vi[13, 50])]) == float(v[2, 0, 13, 50])
    assert ops.kernel_v_layout(torch.bfloat16, 128) == "blocked" and ops.kernel_v_layout(torch.bfloat16, 64) == "blocked"
    assert ops.kernel_v_layout(torch.bfloat16, 96) == "transposed" and ops.kernel_v_layout(torch.bfloat16) == "transposed"
    assert ops.kernel_v_layout(torch.float32, 128) == "rows"
    # the writers: blocked pages hold what transposed pages hold (single tokens, and a prompt's tokens by page tiles)
    from bitnet_c_amd.engine.step import _page_tiles
    H, Hkv, hs, T = 4, 2, 64, 100
    qkv = _rand((T, (H + 2 * Hkv) * hs), torch.bfloat16, 7).cuda()
    pos = torch.arange(30, 30 + T, dtype=torch.int32).cuda()
    seq = torch.zeros(T, dtype=torch.int32).cuda()
    bt = torch.tensor([[2, 0, 3]], dtype=torch.int32).cuda()
    inv = pl.rope_inv_freq(hs, 10000.0).cuda()
    tiles = torch.tensor(_page_tiles([T], [30]), dtype=torch.int32).cuda()
    got = {}
    for blocked in (False, True):
        for by_tiles in (False, True):
            kp = torch.zeros((4, Hkv, 64, hs), dtype=torch.bfloat16).cuda()
            vp = torch.zeros((4, Hkv, hs, 64), dtype=torch.bfloat16).cuda()
            ops.rope_kv_write(qkv.clone(), pos, H, Hkv, hs, inv_freq=inv, rope_dims=hs, seq_index=seq, block_table=bt,
                              k_pages=kp, v_pages=vp, page_tiles=tiles if by_tiles else None, v_transposed=True, blocked=blocked)
            got[blocked, by_tiles] = ops.from_blocked_pages(kp, vp) if blocked else (kp, vp)
    for key in ((False, True), (True, False), (True, True)):
        assert torch.equal(got[key][0], got[False, False][0]) and torch.equal(got[key][1], got[False, False][1]), key
    assert float(got[False, False][0].float().abs().sum()) > 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_rope_kv_write_at_far_positions(dtype):
    """Positions around and far beyond the frequency table's original_max_position_embeddings, with the rescaled
    table of the 8B configuration: angles of up to 131,071 radians, where float32 holds the angle to 2^-7 and the
    range reduction of sine and cosine does the rest.  Against the plain rotation; and the plain rotation at a
    neighbouring position or with the unscaled table is far away, so neither mistake could pass."""
    ops = _ops()
    H, Hkv, hs = 4, 2, 128
    inv = pl.rope_inv_freq(hs, 500000.0, LLAMA3_8B_SCALING)
    T = len(FAR_POSITIONS)
    qkv = _rand((T, (H + 2 * Hkv) * hs), dtype, 480)
    pos = torch.tensor(FAR_POSITIONS, dtype=torch.int32)
    bt = torch.zeros((T, 2048), dtype=torch.int32)
    for t, p in enumerate(FAR_POSITIONS):
        bt[t, p // 64] = t + 1                                   # page 0 stays untouched
    vt = dtype == torch.bfloat16
    kp = torch.zeros((T + 1, Hkv, 64, hs), dtype=dtype).cuda()
    vp = torch.zeros((T + 1, Hkv, hs, 64) if vt else (T + 1, Hkv, 64, hs), dtype=dtype).cuda()
    g = qkv.clone().cuda()
    ops.rope_kv_write(g, pos.cuda(), H, Hkv, hs, inv_freq=inv.cuda(), rope_dims=hs,
                      seq_index=torch.arange(T, dtype=torch.int32).cuda(), block_table=bt.cuda(), k_pages=kp, v_pages=vp)
    q_in = qkv[:, :H * hs].float().view(T, H, hs)
    k_in = qkv[:, H * hs:(H + Hkv) * hs].float().view(T, Hkv, hs)
    q_ref, k_ref = pl.apply_rope(q_in, pos, inv), pl.apply_rope(k_in, pos, inv)
    got_q = g[:, :H * hs].float().view(T, H, hs).cpu()
    assert close(got_q, q_ref, dtype)
    kp, _ = _as_rows(ops, dtype, hs, kp, vp)
    for t, p in enumerate(FAR_POSITIONS):
        assert close(kp[t + 1, :, p % 64], k_ref[t], dtype), p
    assert float(kp[0].abs().sum()) == 0.0
    assert rel_err(pl.apply_rope(q_in, pos - 1, inv), q_ref) > 0.5                               # a position off by one
    assert rel_err(pl.apply_rope(q_in, pos, pl.rope_inv_freq(hs, 500000.0)), q_ref) > 0.5        # the table not rescaled


def test_decode_attention_rotates_and_stores_at_far_positions():
    """The decode kernel's own rotation, angle = (length - 1) * f_i, at lengths 8,192 to 131,072 with the rescaled
    table of the 8B configuration.  Each sequence's cache holds one marked key 1,000 positions back, rotated for
    its position by the plain implementation; query and new key carry the same raw vector, so the marked key's
    score is sum |q_i|^2 cos(1000 f_i) and shares the weight with the new key only when the query was turned by
    the right angle.  The stored key is the plain rotation, and the output the plain attention over all keys."""
    ops = _ops()
    dtype, H, Hkv, hs = torch.bfloat16, 4, 1, 128
    inv = pl.rope_inv_freq(hs, 500000.0, LLAMA3_8B_SCALING)
    scale = hs ** -0.5
    B = len(FAR_POSITIONS)
    g = torch.Generator().manual_seed(490)
    raw = torch.zeros(hs)
    for i in (3, 17, 30, 41, 52, 63):                             # pairs of fast and of slow (rescaled) frequencies
        raw[i], raw[i + hs // 2] = 4.5, -3.0
    raw[0], raw[hs // 2] = 6.0, -3.0                              # the fastest pair turns by one radian a position
    new_key = 0.762 * raw          # so that the new key's score equals the marked key's (sum |q_i|^2 cos(1000 f_i))
    qkv = torch.zeros((B, (H + 2 * Hkv) * hs))
    for h in range(H):
        qkv[:, h * hs:(h + 1) * hs] = raw * (1.0 - 0.05 * h)
    qkv[:, H * hs:(H + 1) * hs] = new_key
    qkv[:, (H + 1) * hs:] = torch.randn(B, hs, generator=g)
    qkv = qkv.to(dtype)
    seqs_k, seqs_v, refs, new_keys = [], [], [], []
    for b, p in enumerate(FAR_POSITIONS):
        L = p + 1
        far = p - 1000
        k = torch.zeros((L, Hkv, hs))
        k[far, 0] = pl.apply_rope(raw.view(1, 1, hs), torch.tensor([far]), inv)[0, 0]
        k_new = pl.apply_rope(qkv[b, H * hs:(H + 1) * hs].float().view(1, 1, hs), torch.tensor([p]), inv)[0, 0]
        k[p, 0] = k_new
        k = k.to(dtype)
        v = torch.randn((L, Hkv, hs), generator=g).to(dtype)
        v[p, 0] = qkv[b, (H + 1) * hs:]
        q = pl.apply_rope(qkv[b, :H * hs].float().view(1, H, hs), torch.tensor([p]), inv)[0].to(dtype).double()
        sc = (q @ k[:, 0].double().t()) * scale                    # [H, L]
        w = torch.softmax(sc, dim=1)
        # the marked key and the new one hold nearly all the weight (scores near 15 against 131,072 keys at 0),
        # and share it
        assert float((w[:, far] + w[:, p]).min()) > 0.8 and float(w[:, far].min()) > 0.25 and float(w[:, p].min()) > 0.25
        refs.append((w @ v[:, 0].double()).reshape(H * hs).float())
        new_keys.append(k[p, 0].float())
        kk, vv = k.clone(), v.clone()
        kk[p], vv[p] = float("nan"), float("nan")                  # the kernel must write this place itself
        seqs_k.append(kk)
        seqs_v.append(vv)
    kp, vp, bt = _paged(seqs_k, seqs_v, dtype, sum((p + 64) // 64 for p in FAR_POSITIONS) + 2, 491)
    kp, vp, bt = kp.cuda(), vp.cuda(), bt.cuda()
    lens = torch.tensor([p + 1 for p in FAR_POSITIONS], dtype=torch.int32).cuda()
    n_splits, chunk = ops.decode_splits(B, H, Hkv, bt.shape[1] * 64)
    out = torch.full((B, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv.cuda(), out, kp, vp, bt, H, Hkv, hs, scale, seq_lens=lens, n_splits=n_splits, chunk=chunk,
                  fused_rotate=inv.cuda(), fused_write=True)
    assert mfma_close(out.float(), torch.stack(refs))
    kp_rows, vp_rows = _as_rows(ops, dtype, hs, kp, vp)
    for b, p in enumerate(FAR_POSITIONS):
        page = int(bt[b, p // 64])
        assert close(kp_rows[page, 0, p % 64], new_keys[b], dtype), p
        assert torch.equal(vp_rows[page, 0, p % 64], qkv[b, (H + 1) * hs:].float()), p
    # the same query turned for the position before would have weighted the two keys otherwise
    q_off = pl.apply_rope(qkv[0, :hs].float().view(1, 1, hs), torch.tensor([FAR_POSITIONS[0] - 1]), inv)[0, 0]
    k_far = seqs_k[0][FAR_POSITIONS[0] - 1000, 0].float()
    q_on = pl.apply_rope(qkv[0, :hs].float().view(1, 1, hs), torch.tensor([FAR_POSITIONS[0]]), inv)[0, 0]
    assert abs(float(q_off @ k_far) - float(q_on @ k_far)) * scale > 1.0


def test_rope_reference_vector_on_device():
    # test/test_transformer.c:636-643 through the kernel: angles pi/2 and 0
    ops = _ops()
    H, hs = 2, 8                                        # rope_dims 4 of head size 8: the rest passes through
    qkv = torch.tensor([1.0, 2, 3, 4, 9, 9, 9, 9, -1, -2, -3, -4, 7, 7, 7, 7]).view(1, 16)
    g = qkv.clone().cuda()
    ops.rope_kv_write(g, torch.tensor([1], dtype=torch.int32).cuda(), H, 0, hs,
                      inv_freq=torch.tensor([math.pi / 2, 0.0]).cuda(), rope_dims=4)
    want = torch.tensor([-3.0, 2, 1, 4, 9, 9, 9, 9, 3, -2, -1, -4, 7, 7, 7, 7])
    assert torch.allclose(g.cpu()[0], want, atol=1e-6)


def mfma_close(got, ref) -> bool:
    """The matrix-core attention rounds the softmax weights to bf16 before the second product
    (8 bits: each weight is off by at most 2^-9 of itself, so a weighted mean of values is off by
    at most 2^-9 of the largest |value| it mixes, here below 2^-9 * 5 for unit normal values),
    and its result once more."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return bool(((got - ref).abs() <= ref.abs() * 2.0 ** -8 + 5 * 2.0 ** -9).all())


def _attn_case(dtype, H, Hkv, hs, lens_before, n_new, window, seed, blocked=None):
    """Random sequences; returns the kernel's output and the plain implementation's, rows in
    batch order.  blocked as _paged's."""
    ops = _ops()
    seqs_q, seqs_k, seqs_v = [], [], []
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        L = p0 + n
        seqs_q.append(_rand((L, H, hs), dtype, seed + 3 * s))
        seqs_k.append(_rand((L, Hkv, hs), dtype, seed + 3 * s + 1))
        seqs_v.append(_rand((L, Hkv, hs), dtype, seed + 3 * s + 2))
    n_pages = sum((p0 + n + 63) // 64 for p0, n in zip(lens_before, n_new)) + 3
    kp, vp, bt = _paged(seqs_k, seqs_v, dtype, n_pages, seed, blocked)
    scale = 1.0 / math.sqrt(hs)
    qrows, ref = [], []
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        full = pl.attention(seqs_q[s].float(), seqs_k[s].float(), seqs_v[s].float(), scale, window or None)
        ref.append(full[p0:].reshape(n, H * hs))
        qrows.append(seqs_q[s][p0:].reshape(n, H * hs))
    q = torch.cat(qrows).contiguous()
    # the kernel takes the Q heads out of a qkv buffer: give it a wider row to test the stride
    qkv = torch.cat([q, torch.full((q.shape[0], 2 * Hkv * hs), float("nan"), dtype=dtype)], dim=1).contiguous()
    return ops, qkv.cuda(), kp.cuda(), vp.cuda(), bt.cuda(), torch.cat(ref), scale


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,hs,window", [(4, 2, 16, 0), (5, 5, 24, 0), (6, 2, 32, 0), (8, 2, 128, 0), (32, 1, 64, 0),
                                             (2, 1, 256, 0), (4, 2, 16, 7), (4, 4, 64, 100), (20, 1, 40, 0),
                                             (32, 8, 128, 0), (8, 8, 128, 33), (6, 2, 64, 0), (40, 2, 64, 0),
                                             (3, 3, 20, 0), (4, 2, 36, 9), (2, 1, 6, 0), (6, 2, 250, 0)])
@pytest.mark.parametrize("force_vector", [False, True])
def test_attention_prompt_form(dtype, H, Hkv, hs, window, force_vector):
    lens_before, n_new = [0, 0, 64, 130, 5, 0], [1, 37, 64, 3, 70, 300]
    ops = _ops()
    if force_vector and not ops.mfma_attention(dtype, hs):
        pytest.skip("the vector kernel is what runs anyway")
    # force_vector: pages with transposed values instead of blocked ones, which the vector kernel reads
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, n_new, window, 100,
                                                  blocked=False if force_vector else None)
    _, _, qt = ops.attention_row_shape(H, Hkv, False, None if force_vector else dtype, hs)
    tiles, r = [], 0
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        for i in range(0, n, qt):
            tiles.append((s, r + i, min(qt, n - i), p0 + i))
        r += n
    out = torch.full((qkv.shape[0], H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, window=window,
                  tiles=torch.tensor(tiles, dtype=torch.int32).cuda(), qt=qt, force_vector=force_vector,
                  blocked=False if force_vector else None)
    assert mfma_close(out.float(), ref) if ops.mfma_attention(dtype, hs) and not force_vector else close(out.float(), ref, dtype)


@pytest.mark.parametrize("H,Hkv,hs,T", [(32, 8, 128, 1200), (32, 8, 64, 2200)])
def test_attention_prompt_form_with_more_workgroups_than_cus(H, Hkv, hs, T):
    """One long prompt: the launch has more tiles than the chip has CUs, which is where a workgroup of the
    matrix-core kernel takes two tiles (the second case has an odd number of them; here they come in
    ascending order, which the kernel must take as well as any other)."""
    dtype = torch.bfloat16
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, [0], [T], 0, 500)
    _, _, qt = ops.attention_row_shape(H, Hkv, False, dtype, hs)
    tiles = [(0, i, min(qt, T - i), i) for i in range(0, T, qt)]
    assert len(tiles) * Hkv > 256
    out = torch.full((T, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, tiles=torch.tensor(tiles, dtype=torch.int32).cuda(), qt=qt)
    assert mfma_close(out.float(), ref)


@pytest.mark.parametrize("hs,window", [(128, 100), (64, 0)])
def test_attention_prompt_form_launch_of_many_rounds(hs, window):
    """Dozens of sequences of unequal lengths, some continuing a cached prefix: several rounds of workgroups over
    the chip, which is where the matrix-core kernel runs one group of waves a workgroup (two workgroups a CU)."""
    import random
    dtype, H, Hkv = torch.bfloat16, 32, 8
    rnd = random.Random(5)
    n_seqs = 24 if hs == 128 else 40                   # a tile holds 32 tokens at head size 128, 64 at 64
    n_new = [rnd.randint(300, 520) for _ in range(n_seqs)]
    lens_before = [rnd.choice([0, 0, 64, 100]) for _ in range(n_seqs)]
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, n_new, window, 700)
    _, _, qt = ops.attention_row_shape(H, Hkv, False, dtype, hs)
    tiles, r = [], 0
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        tiles += [(s, r + i, min(qt, n - i), p0 + i) for i in range(0, n, qt)]
        r += n
    assert (len(tiles) + 1) // 2 * Hkv >= 4 * 256
    out = torch.full((qkv.shape[0], H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, window=window,
                  tiles=torch.tensor(ops.pair_tiles(tiles), dtype=torch.int32).cuda(), qt=qt)
    assert mfma_close(out.float(), ref)


@pytest.mark.parametrize("window", [0, 200])
def test_attention_prompt_form_paired_tiles_of_several_sequences(window):
    """Three sequences of unequal lengths, one of them continuing a cached prefix, in the order the engine hands
    the tiles over (long with short inside a sequence), with more tiles than CUs and an odd number of them in
    each of the sequences; with and without a window."""
    dtype, H, Hkv, hs = torch.bfloat16, 32, 8, 128
    lens_before, n_new = [0, 64, 0], [650, 333, 900]
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, n_new, window, 300)
    _, _, qt = ops.attention_row_shape(H, Hkv, False, dtype, hs)
    tiles, r = [], 0
    for s, (p0, n) in enumerate(zip(lens_before, n_new)):
        tiles += [(s, r + i, min(qt, n - i), p0 + i) for i in range(0, n, qt)]
        r += n
    assert len(tiles) * Hkv > 256 and len(tiles) % 2 == 1
    out = torch.full((qkv.shape[0], H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, window=window,
                  tiles=torch.tensor(ops.pair_tiles(tiles), dtype=torch.int32).cuda(), qt=qt)
    assert mfma_close(out.float(), ref)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,hs,window", [(4, 2, 16, 0), (5, 5, 24, 0), (8, 2, 128, 0), (12, 4, 64, 0),
                                             (16, 1, 32, 0), (4, 2, 16, 50), (8, 8, 64, 129), (32, 8, 128, 0),
                                             (40, 2, 128, 0), (6, 6, 128, 70), (3, 3, 20, 0), (4, 2, 36, 50),
                                             (2, 1, 6, 0)])
@pytest.mark.parametrize("force_splits", [1, 0, 5])
@pytest.mark.parametrize("force_vector", [False, True])
def test_attention_decode_form(dtype, H, Hkv, hs, window, force_splits, force_vector):
    lens_before, n_new = [0, 63, 64, 700, 129, 300], [1] * 6
    ops = _ops()
    if force_vector and not ops.mfma_attention(dtype, hs):
        pytest.skip("the vector kernel is what runs anyway")
    # force_vector: pages with transposed values instead of blocked ones, which the vector kernel reads
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, n_new, window, 200,
                                                  blocked=False if force_vector else None)
    B = len(n_new)
    # two padding rows at the end: length 0, their output is zero and nothing else changes
    qkv = torch.cat([qkv, torch.zeros((2, qkv.shape[1]), dtype=dtype).cuda()])
    bt = torch.cat([bt, torch.zeros((2, bt.shape[1]), dtype=torch.int32).cuda()])
    lens = torch.tensor([p + 1 for p in lens_before] + [0, 0], dtype=torch.int32).cuda()
    max_len = bt.shape[1] * 64
    if force_splits == 0:
        n_splits, chunk = ops.decode_splits(B + 2, H, Hkv, max_len, dtype)
    elif force_splits == 1:
        n_splits, chunk = 1, 0
    elif dtype == torch.float32:
        pytest.skip("a float32 cache's keys are cut in the kernel's own runs and no others")
    else:
        chunk = ((max_len + force_splits - 1) // force_splits + 63) // 64 * 64
        n_splits = (max_len + chunk - 1) // chunk
    if window:
        n_splits, chunk = 1, 0
    out = torch.full((B + 2, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, window=window, seq_lens=lens,
                  n_splits=n_splits, chunk=chunk, force_vector=force_vector, blocked=False if force_vector else None)
    if ops.mfma_attention(dtype, hs) and not force_vector:
        assert mfma_close(out[:B].float(), ref)
    else:
        assert close(out[:B].float(), ref, dtype)
    assert float(out[B:].float().abs().sum()) == 0.0


def test_decode_attention_handed_out_by_length():
    """70 sequences of unequal lengths, 8 kv heads: more workgroups than CUs, so the matrix-core
    kernel hands them out by length when it is given the order.  The result is the plain one,
    and bit for bit the one without the hint."""
    dtype, H, Hkv, hs = torch.bfloat16, 8, 8, 128
    rnd = random.Random(7)
    lens_before = [rnd.randrange(0, 200) for _ in range(70)]
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, [1] * 70, 0, 600)
    lens = [p + 1 for p in lens_before]
    d_lens = torch.tensor(lens, dtype=torch.int32).cuda()
    order = sorted(range(70), key=lambda i: (-lens[i], i))
    outs = []
    for hint in (None, torch.tensor(order, dtype=torch.int32).cuda()):
        out = torch.full((70, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, seq_lens=d_lens, by_length=hint)
        outs.append(out.cpu())
    assert mfma_close(outs[1].float(), ref)
    assert torch.equal(outs[0], outs[1])
    with pytest.raises(ops.KernelError):
        ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, seq_lens=d_lens, by_length=d_lens[:5].contiguous())


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_a_far_key(dtype):
    """One key among 900 has a large score with the query: the output must be its value row,
    wherever it lies (first page, a page's edge, the last position)."""
    ops = _ops()
    for H, Hkv, hs, L in ((4, 2, 32, 900), (8, 2, 128, 900)):
      for far in (0, 63, 64, 449, 898, 899):
        k = _rand((L, Hkv, hs), dtype, 300, 0.1)
        v = _rand((L, Hkv, hs), dtype, 301)
        q = _rand((1, H, hs), dtype, 302, 0.1)
        k[far] = 0
        k[far, :, 0] = 16.0
        q[0, :, 0] = 16.0                                   # score 256 * scale at `far`, about 0 elsewhere
        kp, vp, bt = _paged([k], [v], dtype, 20, far)
        qkv = q.reshape(1, H * hs).contiguous().cuda()
        # (a float32 cache's keys are cut in the kernel's own runs of 2,048 and no others)
        for n_splits, chunk in ((1, 0), (4, 256), (15, 64)) if dtype == torch.bfloat16 else ((1, 0), (1, ops.F32_FOLD_KEYS)):
            out = torch.empty((1, H * hs), dtype=dtype).cuda()
            ops.attention(qkv, out, kp.cuda(), vp.cuda(), bt.cuda(), H, Hkv, hs, 1 / math.sqrt(hs),
                          seq_lens=torch.tensor([L], dtype=torch.int32).cuda(), n_splits=n_splits, chunk=chunk)
            want = v[far].float().repeat_interleave(H // Hkv, dim=0).reshape(1, H * hs)
            assert rel_err(out.float(), want) < 1e-3, (far, n_splits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,hs,window", [(4, 2, 32, 70), (8, 2, 128, 64), (6, 6, 64, 129)])
def test_attention_at_the_window_s_edge(dtype, H, Hkv, hs, window):
    """A key with a large score just inside the window is the whole answer, and the same key one
    position further back (just outside) must not be seen at all: the decode form for the last
    position, the prompt form for a chunk of rows whose windows begin at different keys."""
    ops = _ops()
    L, n_new = 300, 40
    scale = 1 / math.sqrt(hs)
    for back in (window - 1, window):                       # the last key inside, the first one outside
        k = _rand((L, Hkv, hs), dtype, 310, 0.1)
        v = _rand((L, Hkv, hs), dtype, 311)
        q = _rand((L, H, hs), dtype, 312, 0.1)
        t = L - 1
        far = t - back
        k[far] = 0
        k[far, :, 0] = 16.0
        q[:, :, 0] = 16.0
        kp, vp, bt = _paged([k], [v], dtype, 8, far)
        ref = pl.attention(q.float(), k.float(), v.float(), scale, window).reshape(L, H * hs)
        if back == window - 1:                              # inside: the answer is that key's value row
            assert rel_err(ref[t:t + 1], v[far].float().repeat_interleave(H // Hkv, dim=0).reshape(1, H * hs)) < 1e-3
        else:                                               # outside: the plain answer without it is something else
            assert rel_err(ref[t:t + 1], v[far].float().repeat_interleave(H // Hkv, dim=0).reshape(1, H * hs)) > 0.5
        check = (lambda o, r: mfma_close(o, r)) if ops.mfma_attention(dtype, hs) else (lambda o, r: close(o, r, dtype))
        # decode form: the row at position t
        out = torch.empty((1, H * hs), dtype=dtype).cuda()
        ops.attention(q[t:t + 1].reshape(1, H * hs).contiguous().cuda(), out, kp.cuda(), vp.cuda(), bt.cuda(), H, Hkv, hs,
                      scale, window=window, seq_lens=torch.tensor([L], dtype=torch.int32).cuda())
        assert check(out.float(), ref[t:t + 1]), ("decode", back)
        # prompt form: the last n_new rows; the key leaves the window of each row at a different place
        _, _, qt = ops.attention_row_shape(H, Hkv, False, dtype, hs)
        tiles = torch.tensor([(0, i, min(qt, n_new - i), L - n_new + i) for i in range(0, n_new, qt)], dtype=torch.int32).cuda()
        outp = torch.empty((n_new, H * hs), dtype=dtype).cuda()
        ops.attention(q[L - n_new:].reshape(n_new, H * hs).contiguous().cuda(), outp, kp.cuda(), vp.cuda(), bt.cuda(), H, Hkv,
                      hs, scale, window=window, tiles=tiles, qt=qt)
        assert check(outp.float(), ref[L - n_new:]), ("prompt", back)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,hs", [(8, 2, 128), (6, 3, 48)])
def test_attention_over_a_long_context(dtype, H, Hkv, hs):
    """20,000 cached positions: a decode row with the split plan the engine would pick, and a
    prompt chunk of 70 tokens that continues at position 19,930.  The reference is the plain
    formula for the wanted rows only (scores, softmax, weighted values in float64)."""
    ops = _ops()
    L, n_new = 20000, 70
    k = _rand((L, Hkv, hs), dtype, 400)
    v = _rand((L, Hkv, hs), dtype, 401)
    q = _rand((n_new, H, hs), dtype, 402)
    scale = 1.0 / math.sqrt(hs)
    kp, vp, bt = _paged([k], [v], dtype, (L + 63) // 64 + 5, 403)
    kp, vp, bt = kp.cuda(), vp.cuda(), bt.cuda()

    def plain_rows(first_pos):
        rows = []
        for t in range(q.shape[0]):
            n_kv = first_pos + t + 1
            for h in range(H):
                kh = h // (H // Hkv)
                sc = (k[:n_kv, kh].double() @ q[t, h].double()) * scale
                rows.append(pl.softmax(sc[None, :].float())[0].double() @ v[:n_kv, kh].double())
        return torch.stack(rows).reshape(q.shape[0], H * hs).float()

    def check(out, ref):
        if ops.mfma_attention(dtype, hs):
            assert mfma_close(out.float(), ref)
        else:
            assert close(out.float(), ref, dtype)

    qkv = q.reshape(n_new, H * hs).contiguous().cuda()
    # the chunk of a prompt: rows at positions L - n_new .. L - 1
    _, _, qt = ops.attention_row_shape(H, Hkv, False, dtype, hs)
    tiles = torch.tensor([(0, i, min(qt, n_new - i), L - n_new + i) for i in range(0, n_new, qt)], dtype=torch.int32).cuda()
    out = torch.full((n_new, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, out, kp, vp, bt, H, Hkv, hs, scale, tiles=tiles, qt=qt)
    ref = plain_rows(L - n_new)
    check(out, ref)
    # one decoded token at the last position, split as the engine splits it
    n_splits, chunk = ops.decode_splits(1, H, Hkv, bt.shape[1] * 64, dtype)
    assert n_splits > 1
    out1 = torch.full((1, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv[-1:].contiguous(), out1, kp, vp, bt, H, Hkv, hs, scale,
                  seq_lens=torch.tensor([L], dtype=torch.int32).cuda(), n_splits=n_splits, chunk=chunk)
    check(out1, ref[-1:])
    if dtype == torch.float32:
        # float32 keys are summed in runs of 2,048 that are folded in order, by one workgroup that walks them all (the
        # prompt form, a decode row that is not split) or by a workgroup a run and the fold kernel: the same bits
        assert (n_splits, chunk) == ((bt.shape[1] * 64 + ops.F32_FOLD_KEYS - 1) // ops.F32_FOLD_KEYS, ops.F32_FOLD_KEYS)
        assert torch.equal(out1, out[-1:])
        out2 = torch.full((1, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(qkv[-1:].contiguous(), out2, kp, vp, bt, H, Hkv, hs, scale,
                      seq_lens=torch.tensor([L], dtype=torch.int32).cuda(), n_splits=1, chunk=0)
        assert torch.equal(out2, out1)
        wide = torch.zeros((1, 2048), dtype=torch.int32).cuda()            # a table for 131,072 keys: 64 runs, most of them empty
        wide[:, :bt.shape[1]] = bt
        out3 = torch.full((1, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(qkv[-1:].contiguous(), out3, kp, vp, wide, H, Hkv, hs, scale,
                      seq_lens=torch.tensor([L], dtype=torch.int32).cuda(), n_splits=64, chunk=ops.F32_FOLD_KEYS)
        assert torch.equal(out3, out1)
        with pytest.raises(ops.KernelError):                               # runs of another length are refused
            ops.attention(qkv[-1:].contiguous(), out3, kp, vp, bt, H, Hkv, hs, scale,
                          seq_lens=torch.tensor([L], dtype=torch.int32).cuda(), n_splits=5, chunk=4096)


# ---------------------------------------------------------------------------------------
def test_argmax_ties_and_odd_vocab():
    ops = _ops()
    x = _rand((5, 1009), torch.float32, 400)
    x[1, 17] = x[1, 900] = 50.0                    # a tie: the lower index wins
    x[2, 1008] = 60.0
    x[3, 0] = 70.0
    got = ops.argmax(x.cuda()).cpu().tolist()
    assert got == torch.argmax(x, dim=1).tolist() and got[1] == 17 and got[2] == 1008 and got[3] == 0
    assert ops.argmax(torch.tensor([[1.0, 3.0, 2.0, 0.5]]).cuda()).item() == 1        # test/test_safety.c:208-211
    big = _rand((3, 128256), torch.float32, 401)                 # the two-stage form
    big[0, 5] = big[0, 100000] = 9.0                             # a tie across parts: the lower index
    big[1, 128255] = 9.0
    big[2, 2004] = big[2, 2003] = 9.0                            # a tie at a part's edge (2004 per part)
    assert ops.argmax(big.cuda()).cpu().tolist() == [5, 128255, 2003]
    assert ops.argmax(torch.full((2, 20000), -float("inf")).cuda()).cpu().tolist() == [0, 0]


@pytest.mark.parametrize("vocab", [4, 389, 128256])
@pytest.mark.parametrize("temperature,top_p", [(0.8, 1.0), (1.0, 0.0), (0.7, 0.9), (1.3, 0.5)])
def test_sample_matches_the_plain_sampler(vocab, temperature, top_p):
    ops = _ops()
    B = 6
    logits = _rand((B, vocab), torch.float32, 500, 3.0)
    rng = pl.XorShift64Star(99)
    rs = [rng.next_float() for _ in range(B)]
    got = ops.sample(logits.cuda(), temperature, top_p, torch.tensor(rs, dtype=torch.float32).cuda()).cpu().tolist()

    class Fixed:
        def __init__(self, r): self.r = r
        def next_float(self): return self.r
    want = [pl.sample(logits[i], temperature, top_p, Fixed(rs[i])) for i in range(B)]
    # the two may differ when r falls within rounding of a boundary of the cdf; with 6 draws from a
    # continuous r that has probability ~1e-6, so equality is demanded
    assert got == want


@pytest.mark.parametrize("vocab", [16384, 70001, 128256])
def test_sample_with_a_row_spread_over_many_workgroups(vocab):
    """From 16,384 logits a row on, every pass of the sampler is a launch of 32 workgroups a row.  It has to
    draw what the one-workgroup form and the plain sampler draw: peaked and flat rows, plain cdf walk and
    top-p, a batch of rows with different uniform numbers."""
    ops = _ops()
    B = 12
    g = torch.Generator().manual_seed(vocab)
    rows = [torch.randn(vocab, generator=g) * s for s in (0.5, 3.0, 8.0)] * 4                 # flat ... peaked
    logits = torch.stack(rows)
    rng = pl.XorShift64Star(5)
    rs = [rng.next_float() for _ in range(B)]
    r = torch.tensor(rs, dtype=torch.float32).cuda()

    class Fixed:
        def __init__(self, r): self.r = r
        def next_float(self): return self.r
    for temperature, top_p in ((1.0, 0.9), (0.7, 0.5), (1.3, 1.0), (1.0, 0.999), (0.05, 0.9)):
        wide = ops.sample(logits.cuda(), temperature, top_p, r).cpu().tolist()
        one = ops.sample(logits.cuda(), temperature, top_p, r, force_one_workgroup=True).cpu().tolist()
        want = [pl.sample(logits[i], temperature, top_p, Fixed(rs[i])) for i in range(B)]
        # the three add the probabilities in different orders; a draw changes only where r falls within
        # rounding of a boundary, which 12 draws do not hit
        assert wide == want, (temperature, top_p, wide, want)
        assert one == want, (temperature, top_p, one, want)
    # a dominant logit far from the start of the row, top-p below its probability: always that token
    lg = torch.zeros(3, vocab)
    lg[:, vocab - 7] = 30.0
    assert ops.sample(lg.cuda(), 1.0, 0.5, r[:3].contiguous()).cpu().tolist() == [vocab - 7] * 3


def test_sample_among_equal_probabilities():
    """All logits equal, or in a few equal groups: top-p orders equal probabilities by index, and the
    walk has to find the k-th member of a group across the ranges that the waves own."""
    ops = _ops()

    class Fixed:
        def __init__(self, r): self.r = r
        def next_float(self): return self.r
    rng = pl.XorShift64Star(7)
    for vocab in (1000, 70000):
        for kind in ("flat", "steps"):
            lg = torch.zeros(8, vocab) if kind == "flat" else (torch.arange(vocab) % 5).float().repeat(8, 1) * 0.5
            rs = [rng.next_float() for _ in range(8)]
            for top_p in (0.9, 0.3, 1.0):
                got = ops.sample(lg.cuda(), 1.0, top_p, torch.tensor(rs, dtype=torch.float32).cuda()).cpu().tolist()
                want = [pl.sample(lg[i], 1.0, top_p, Fixed(rs[i])) for i in range(8)]
                # The plain sampler adds float32 probabilities one by one, the kernel adds them exactly (in
                # fixed point): among thousands of equal probabilities the two walks may stop one member of
                # the group apart (the next index with that probability), never further.
                step = 1 if kind == "flat" else 5
                assert all(abs(g - w) in (0, step) for g, w in zip(got, want)), (vocab, kind, top_p, got, want)
                assert all(float(lg[i, g]) == float(lg[i, w]) for i, (g, w) in enumerate(zip(got, want)))


def test_sample_reference_cases_on_device():
    ops = _ops()
    # top-p 0.5 with a dominant logit: always token 0 (test/test_safety.c:256-272)
    lg = torch.tensor([[10.0, 0.0, 0.0, 0.0]] * 64).cuda()
    rng = pl.XorShift64Star(42)
    r = torch.tensor([rng.next_float() for _ in range(64)], dtype=torch.float32).cuda()
    assert sum(t == 0 for t in ops.sample(lg, 1.0, 0.5, r).cpu().tolist()) > 51
    assert ops.sample(torch.tensor([[5.0]]).cuda(), 0.5, 0.9, torch.tensor([0.3]).cuda()).item() == 0   # vocab 1
    # temperature 0 ignores the uniforms
    assert ops.sample(torch.tensor([[1.0, 3.0, 2.0, 0.5]]).cuda(), 0.0, 0.9).item() == 1


def test_repeat_penalty_on_device():
    ops = _ops()
    lg = torch.tensor([[2.0, 2.1, 2.0, 2.0], [1.0, -1.0, 0.5, 3.0]]).cuda()
    recent = torch.tensor([[1, 1, 1, -1], [1, 3, 3, 1]], dtype=torch.int32).cuda()
    ops.repeat_penalty_(lg, recent, 1.5)
    want = torch.tensor([[2.0, 2.1 / 1.5, 2.0, 2.0], [1.0, -1.5, 0.5, 2.0]])
    assert torch.allclose(lg.cpu(), want, atol=1e-6)
    assert ops.argmax(lg).cpu().tolist()[0] != 1           # test/test_safety.c:229-238


@pytest.mark.parametrize("H,Hkv,hs,window", [(32, 8, 128, 0), (8, 2, 64, 0), (16, 1, 128, 0), (6, 6, 64, 90), (4, 4, 128, 0)])
@pytest.mark.parametrize("force_splits", [1, 0, 7])
def test_decode_attention_that_rotates_and_stores_itself(H, Hkv, hs, window, force_splits):
    """The decode kernel doing rope_kv_write's work: unrotated qkv in, the new key and value stored,
    against rope_kv_write followed by the same attention; run twice in a row.  Every wave of a workgroup asks for its
    first block of 32 keys before it knows the length: the lengths put the new token's place into the first block of
    each of the four waves (which must then be read again behind the store), into a later block, and behind a
    sequence's end (a block that is dropped)."""
    ops = _ops()
    dtype = torch.bfloat16
    lens_before = [0, 63, 64, 700, 129, 300, 31, 100, 127, 32]
    B = len(lens_before)
    seqs_k = [_rand((p + 1, Hkv, hs), dtype, 700 + i) for i, p in enumerate(lens_before)]
    seqs_v = [_rand((p + 1, Hkv, hs), dtype, 800 + i) for i, p in enumerate(lens_before)]
    kp, vp, bt = _paged(seqs_k, seqs_v, dtype, sum((p + 64) // 64 for p in lens_before) + 2, 7)
    inv_freq = pl.rope_inv_freq(hs, 10000.0)
    qkv = _rand((B + 1, (H + 2 * Hkv) * hs), dtype, 900)
    lens = torch.tensor([p + 1 for p in lens_before] + [0], dtype=torch.int32)
    pos = lens - 1
    bt = torch.cat([bt, torch.zeros((1, bt.shape[1]), dtype=torch.int32)])
    max_len = bt.shape[1] * 64
    if window or force_splits == 1:
        n_splits, chunk = 1, 0
    elif force_splits == 0:
        n_splits, chunk = ops.decode_splits(B + 1, H, Hkv, max_len)
    else:
        chunk = ((max_len + force_splits - 1) // force_splits + 63) // 64 * 64
        n_splits = (max_len + chunk - 1) // chunk
    scale = hs ** -0.5
    # reference: the two kernels one after the other
    q1, k1, v1 = qkv.clone().cuda(), kp.clone().cuda(), vp.clone().cuda()
    ops.rope_kv_write(q1, pos.cuda(), H, Hkv, hs, inv_freq=inv_freq.cuda(), rope_dims=hs,
                      seq_index=torch.arange(B + 1, dtype=torch.int32).cuda(), block_table=bt.cuda(), k_pages=k1, v_pages=v1)
    want = torch.empty((B + 1, H * hs), dtype=dtype).cuda()
    ops.attention(q1, want, k1, v1, bt.cuda(), H, Hkv, hs, scale, window=window, seq_lens=lens.cuda(),
                  n_splits=n_splits, chunk=chunk)
    for _ in range(2):
        q2, k2, v2 = qkv.clone().cuda(), kp.clone().cuda(), vp.clone().cuda()
        got = torch.full((B + 1, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(q2, got, k2, v2, bt.cuda(), H, Hkv, hs, scale, window=window, seq_lens=lens.cuda(),
                      n_splits=n_splits, chunk=chunk, fused_rotate=inv_freq.cuda(), fused_write=True)
        torch.cuda.synchronize()
        assert torch.equal(q2.cpu(), qkv)                            # the input stays unrotated
        # the stored key and value are the ones rope_kv_write stores (NaN marks untouched places in both)
        assert torch.equal(torch.nan_to_num(k2.float(), nan=-7.0).cpu(), torch.nan_to_num(k1.float(), nan=-7.0).cpu())
        assert torch.equal(torch.nan_to_num(v2.float(), nan=-7.0).cpu(), torch.nan_to_num(v1.float(), nan=-7.0).cpu())
        assert mfma_close(got[:B].float(), want[:B].float())
        assert float(got[B:].float().abs().sum()) == 0.0


@pytest.mark.parametrize("dtype,H,Hkv,hs", [(torch.bfloat16, 8, 2, 128), (torch.bfloat16, 6, 3, 48), (torch.bfloat16, 4, 4, 64)])
def test_decode_attention_with_the_longest_length_in_device_memory(dtype, H, Hkv, hs):
    """The form a captured step uses: a fixed number of splits and a block table as wide as the longest sequence
    the engine allows, the keys per split derived inside the kernel from a device-side integer.  Whatever the
    longest sequence of a launch is, the result is the plain one; and with the integer equal to what the
    table's width gives, it is bit for bit the result of the host-side plan."""
    lens_before = [0, 63, 64, 700, 129, 300]
    B = len(lens_before)
    ops, qkv, kp, vp, bt, ref, scale = _attn_case(dtype, H, Hkv, hs, lens_before, [1] * B, 0, 230)
    wide = torch.zeros((B, 40), dtype=torch.int32).cuda()                  # room for 2,560 keys a sequence
    wide[:, :bt.shape[1]] = bt
    lens = torch.tensor([p + 1 for p in lens_before], dtype=torch.int32).cuda()
    check = (lambda o: mfma_close(o, ref)) if ops.mfma_attention(dtype, hs) else (lambda o: close(o, ref, dtype))
    n_splits, _ = ops.decode_splits(B, H, Hkv, 40 * 64)
    assert n_splits > 1
    outs = {}
    for max_len in (701, 1000, 2560):
        out = torch.full((B, H * hs), float("nan"), dtype=dtype).cuda()
        ops.attention(qkv, out, kp, vp, wide, H, Hkv, hs, scale, seq_lens=lens, n_splits=n_splits,
                      max_len_dev=torch.tensor([max_len], dtype=torch.int32).cuda())
        assert check(out.float()), max_len
        outs[max_len] = out
    host = torch.full((B, H * hs), float("nan"), dtype=dtype).cuda()
    ops.attention(qkv, host, kp, vp, wide, H, Hkv, hs, scale, seq_lens=lens, n_splits=n_splits,
                  chunk=ops.split_chunk(2560, n_splits))
    assert torch.equal(host, outs[2560])
    with pytest.raises(ops.KernelError):                                   # the prompt form has no such integer
        ops.attention(qkv, host, kp, vp, wide, H, Hkv, hs, scale, tiles=torch.zeros((1, 4), dtype=torch.int32).cuda(),
                      qt=ops.attention_row_shape(H, Hkv, False, dtype, hs)[2],
                      max_len_dev=torch.tensor([5], dtype=torch.int32).cuda())
