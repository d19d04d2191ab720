"""Pins the plain implementation by what fixes it beside the reference's text: vectors
that the reference's own tests hold, special cases that reduce to a library routine, and
invariants.  Each is chosen so that a plausible mistake fails it."""
import math

import pytest
import torch

import plain_llama as pl


def test_rmsnorm_reference_vector():
    # test/test_transformer.c:427-449
    x = torch.tensor([1.0, 2.0, 3.0, 4.0])
    out = pl.rmsnorm(x, torch.ones(4), 1e-5)
    want = x / math.sqrt(7.5 + 1e-5)
    assert torch.allclose(out, want, atol=1e-5)


def test_rmsnorm_is_library_rms_norm_and_eps_is_inside_the_root():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 40, generator=g)
    w = torch.randn(40, generator=g)
    assert torch.allclose(pl.rmsnorm(x, w, 1e-6), torch.nn.functional.rms_norm(x, (40,), w, 1e-6), atol=1e-6)
    tiny = torch.full((8,), 1e-4)                      # mean(x^2) = 1e-8 << eps
    out = pl.rmsnorm(tiny, torch.ones(8), 1e-2)
    assert torch.allclose(out, tiny / math.sqrt(1e-8 + 1e-2), rtol=1e-5)       # not x/(rms + eps)
    assert not torch.allclose(out, tiny / (1e-4 + 1e-2), rtol=1e-2)


def test_softmax_reference_vectors():
    # test/test_transformer.c:482-505 and :507-546
    p = pl.softmax(torch.tensor([[1.0, 2.0, 3.0]]))[0]
    e = torch.exp(torch.tensor([1.0, 2.0, 3.0]))
    assert torch.allclose(p, e / e.sum(), atol=1e-6) and abs(float(p.sum()) - 1) < 1e-6
    v = torch.tensor([[3.25, -1.0, 0.5, 8.0, -4.0, 2.0, 1.25]])
    assert torch.allclose(pl.softmax(v), torch.softmax(v, -1), atol=2e-6)
    assert torch.allclose(pl.softmax(v + 100.0), pl.softmax(v), atol=1e-6)     # shift invariance


def test_rope_reference_vector_fixes_pairing_and_sign():
    # test/test_transformer.c:636-643: cos = {0, 1}, sin = {1, 0} on two heads of size 4
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0], [-1.0, -2.0, -3.0, -4.0]]).view(1, 2, 4)
    # angles pi/2 and 0 at position 1: inv_freq = [pi/2, 0]
    out = pl.apply_rope(x, torch.tensor([1]), torch.tensor([math.pi / 2, 0.0]))
    want = torch.tensor([[-3.0, 2.0, 1.0, 4.0], [3.0, -2.0, -1.0, -4.0]]).view(1, 2, 4)
    assert torch.allclose(out, want, atol=1e-6)


def test_rope_identity_norm_and_relative_positions():
    # test/test_transformer.c:548-574: position 0 is the identity, the norm is kept
    f = pl.rope_inv_freq(4, 10000.0)
    v = torch.tensor([1.0, 0.0, 0.0, 1.0]).view(1, 1, 4)
    assert torch.allclose(pl.apply_rope(v, torch.tensor([0]), f), v, atol=1e-6)
    w = torch.ones(1, 1, 4)
    assert abs(float(pl.apply_rope(w, torch.tensor([5]), f).pow(2).sum()) - 4.0) < 1e-4
    # a two-dimensional head is a plane rotation by pos radians
    r = pl.apply_rope(torch.tensor([1.0, 0.0]).view(1, 1, 2), torch.tensor([3]), pl.rope_inv_freq(2, 123.0))
    assert torch.allclose(r.view(2), torch.tensor([math.cos(3.0), math.sin(3.0)]), atol=1e-6)
    # <R_p q, R_s k> depends on p - s only
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 16, generator=g), torch.randn(1, 1, 16, generator=g)
    f = pl.rope_inv_freq(16, 10000.0)
    def dot(p, s):
        return float((pl.apply_rope(q, torch.tensor([p]), f) * pl.apply_rope(k, torch.tensor([s]), f)).sum())
    assert abs(dot(9, 4) - dot(25, 20)) < 1e-4 and abs(dot(9, 4) - dot(4, 9)) > 1e-3
    # frequencies: f_i = theta^(-2i/d) (test/test_transformer.c:412)
    assert torch.allclose(pl.rope_inv_freq(8, 10000.0),
                          torch.tensor([1.0 / 10000.0 ** (2 * i / 8) for i in range(4)]), rtol=1e-6)


def test_llama3_scaling_limits():
    base = pl.rope_inv_freq(64, 500000.0)
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
              original_max_position_embeddings=64)
    assert torch.equal(pl.rope_inv_freq(64, 500000.0, dict(sc, factor=1.0)), base)         # factor 1: unscaled
    huge = dict(sc, original_max_position_embeddings=10 ** 12)
    assert torch.equal(pl.rope_inv_freq(64, 500000.0, huge), base)                          # all wavelengths short
    small = dict(sc, original_max_position_embeddings=1, low_freq_factor=1.0, high_freq_factor=2.0)
    assert torch.allclose(pl.rope_inv_freq(64, 500000.0, small)[1:], base[1:] / 8.0, rtol=1e-6)  # all long
    f = pl.rope_inv_freq(64, 500000.0, sc)
    assert torch.all(f[1:] < f[:-1])                                                        # still decreasing
    assert torch.all(f <= base * (1 + 1e-6)) and torch.all(f >= base / 8.0 * (1 - 1e-6))


def test_llama3_scaling_is_continuous_at_both_thresholds():
    """A wavelength a hair inside the interpolated band gets (almost) the value of the region next to it:
    at orig/high_freq_factor the unscaled frequency, at orig/low_freq_factor the frequency divided by
    `factor`.  The interpolation weights the other way round (or a band taken in wavelength instead of
    orig/wavelength) jumps by the factor at an edge; the middle of the band lies strictly between."""
    hd, theta, i = 64, 500000.0, 9
    base = float(theta ** (-2.0 * i / hd))
    wavelen = 2 * math.pi / base
    sc = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0)
    eps = 1e-7

    def scaled(orig):
        return float(pl.rope_inv_freq(hd, theta, dict(sc, original_max_position_embeddings=orig)).double()[i])

    # wavelength == orig/high: orig = 4 * wavelength.  A little more orig: the wavelength is short (unscaled);
    # a little less: it is just inside the band
    short, inside = scaled(4.0 * wavelen * (1 + eps)), scaled(4.0 * wavelen * (1 - eps))
    assert abs(short - base) < 1e-6 * base
    assert abs(inside - base) < 1e-5 * base                       # not base / 8
    # wavelength == orig/low: orig = wavelength.  A little less orig: the wavelength is long (divided by the
    # factor); a little more: just inside the band
    long_, inside = scaled(wavelen * (1 - eps)), scaled(wavelen * (1 + eps))
    assert abs(long_ - base / 8.0) < 1e-6 * base
    assert abs(inside - base / 8.0) < 1e-5 * base                 # not base
    # the middle of the band in orig/wavelength (2.5 between 1 and 4): smooth = 0.5
    mid = scaled(2.5 * wavelen)
    assert abs(mid - 0.5 * (base / 8.0 + base)) < 1e-5 * base


def test_attention_reference_vector():
    # test/test_transformer.c:8372-8456: one head, one-hot keys
    keys = torch.eye(4).view(4, 1, 4)
    vals = torch.tensor([[1.0, 2, 3, 4], [5, 6, 7, 8], [0, 0, 0, 0], [0, 0, 0, 0]]).view(4, 1, 4)
    q = torch.tensor([[1.0, 0, 0, 0], [0, 1.0, 0, 0]]).view(2, 1, 4)
    out = pl.attention(q, keys[:2], vals[:2], 1.0 / math.sqrt(4))
    assert torch.allclose(out[0, 0], vals[0, 0], atol=1e-5)
    w0, w1 = math.exp(0.0), math.exp(0.5)
    assert torch.allclose(out[1, 0], (w0 * vals[0, 0] + w1 * vals[1, 0]) / (w0 + w1), atol=1e-5)


@pytest.mark.parametrize("H,Hkv", [(4, 4), (6, 2), (4, 1)])
def test_attention_is_library_sdpa(H, Hkv):
    g = torch.Generator().manual_seed(2)
    T, hs = 9, 8
    q, k, v = (torch.randn(T, n, hs, generator=g) for n in (H, Hkv, Hkv))
    out = pl.attention(q, k, v, 1.0 / math.sqrt(hs))
    kk = k.repeat_interleave(H // Hkv, dim=1)          # head h uses kv head h // (H/Hkv)
    vv = v.repeat_interleave(H // Hkv, dim=1)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(out, ref, atol=1e-5)
    # a future token does not change the past
    out2 = pl.attention(q[:5], k[:5], v[:5], 1.0 / math.sqrt(hs))
    assert torch.allclose(out2, out[:5], atol=1e-6)


def test_attention_window():
    g = torch.Generator().manual_seed(3)
    T, hs = 12, 8
    q, k, v = (torch.randn(T, 2, hs, generator=g) for _ in range(3))
    full = pl.attention(q, k, v, 0.3)
    win = pl.attention(q, k, v, 0.3, window=4)
    assert torch.allclose(win[:4], full[:4], atol=1e-6)            # the window is not full yet
    # query 8 sees keys 5..8 (no rope here): the last row of the four-token sequence 5..8
    four = pl.attention(q[5:9], k[5:9], v[5:9], 0.3)
    assert torch.allclose(win[8], four[3], atol=1e-6) and not torch.allclose(win[8], full[8], atol=1e-4)
    # a window of one position: every query sees itself alone, the output is its own value row
    one = pl.attention(q, k, v, 0.3, window=1)
    assert torch.allclose(one, v.repeat_interleave(1, dim=1), atol=1e-6)


def test_swiglu_reference_vector():
    # test/test_transformer.c:645-677, the exact-activation mode
    g = torch.tensor([-2.0, -1.0, -0.25, 0.0, 0.25, 1.0, 2.0, 4.0])
    u = torch.tensor([1.0, 0.5, 2.0, 3.0, -1.0, 1.5, -0.5, 2.0])
    assert torch.allclose(pl.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-6)
    assert torch.allclose(pl.swiglu(g, u), (g / (1 + torch.exp(-g))) * u, atol=0)


def test_other_gate_activations_and_the_bounds_around_the_blocks():
    g = torch.tensor([-3.0, -1.0, -0.25, 0.0, 0.25, 1.0, 2.0, 4.0])
    u = torch.tensor([1.0, 0.5, 2.0, 3.0, -1.0, 1.5, -0.5, 2.0])
    assert torch.allclose(pl.swiglu(g, u, "gelu_tanh"), torch.nn.functional.gelu(g, approximate="tanh") * u, atol=1e-6)
    assert torch.equal(pl.swiglu(g, u, "relu2"), torch.tensor([0.0, 0, 0, 0, 0.0625, 1, 4, 16]) * u)
    assert torch.equal(pl.swiglu(g, u), pl.swiglu(g, u, "silu"))
    from conftest import TINY_A
    c, W = _tiny(TINY_A, 9)
    toks = [5, 6, 7]
    base = pl.forward(c, W, toks)
    # a soft-cap far above the logits changes almost nothing; a small one bounds them and keeps their order
    assert torch.allclose(pl.forward(c, W, toks, softcap=1e4), base, atol=1e-5)
    cap = float(base.abs().max())
    capped = pl.forward(c, W, toks, softcap=cap)
    assert abs(float(capped.abs().max()) - math.tanh(1.0) * cap) < 1e-5 * cap
    assert torch.equal(capped.argsort(dim=1), base.argsort(dim=1))
    # the embedding multiplier: the first norm takes a common factor out again (up to eps), so the logits move little
    # with it, while a model whose first block were not normed would scale: the multiplier acts before the first block
    W1 = dict(W)
    W1["model.embed_tokens.weight"] = W["model.embed_tokens.weight"] * 8.0
    W1["lm_head.weight"] = W["lm_head.weight"]
    assert torch.allclose(pl.forward(c, W, toks, emb_scale=8.0), pl.forward(c, W1, toks), atol=1e-5)


def _tiny(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    c = dict(dim=cfg["hidden_size"], ffn=cfg["intermediate_size"], layers=cfg["num_hidden_layers"],
             heads=cfg["num_attention_heads"], kv_heads=cfg["num_key_value_heads"],
             head_dim=cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"],
             vocab=cfg["vocab_size"], theta=cfg["rope_theta"], eps=cfg["rms_norm_eps"],
             tied=cfg["tie_word_embeddings"], rope_scaling=cfg.get("rope_scaling"), max_pos=0)
    W = {"model.embed_tokens.weight": torch.randn(c["vocab"], c["dim"], generator=g) * 0.02,
         "model.norm.weight": torch.rand(c["dim"], generator=g) + 0.5}
    if not c["tied"]:
        W["lm_head.weight"] = torch.randn(c["vocab"], c["dim"], generator=g) * 0.02
    for l in range(c["layers"]):
        p = f"model.layers.{l}."
        qd, kd = c["heads"] * c["head_dim"], c["kv_heads"] * c["head_dim"]
        for n, s in (("self_attn.q_proj", (qd, c["dim"])), ("self_attn.k_proj", (kd, c["dim"])),
                     ("self_attn.v_proj", (kd, c["dim"])), ("self_attn.o_proj", (c["dim"], qd)),
                     ("mlp.gate_proj", (c["ffn"], c["dim"])), ("mlp.up_proj", (c["ffn"], c["dim"])),
                     ("mlp.down_proj", (c["dim"], c["ffn"]))):
            W[p + n + ".weight"] = torch.randn(*s, generator=g) * 0.05
        W[p + "input_layernorm.weight"] = torch.rand(c["dim"], generator=g) + 0.5
        W[p + "post_attention_layernorm.weight"] = torch.rand(c["dim"], generator=g) + 0.5
    return c, W


def test_layer_order_and_residual_with_zero_output_matrices():
    # Wo = 0 and Wdown = 0: logits = lm_head(norm(E[token])) at any depth
    from conftest import TINY_A
    c, W = _tiny(TINY_A, 4)
    for k in list(W):
        if k.endswith("o_proj.weight") or k.endswith("down_proj.weight"):
            W[k] = torch.zeros_like(W[k])
    toks = [3, 200, 17, 5]
    x = W["model.embed_tokens.weight"][toks]
    want = pl.rmsnorm(x, W["model.norm.weight"], c["eps"]) @ W["lm_head.weight"].t()
    assert torch.allclose(pl.forward(c, W, toks), want, atol=1e-6)


def test_the_feed_forward_reads_the_stream_after_the_attention_add():
    """x += attention(norm(x)) comes first and the feed-forward reads the sum (src/transformer/cpu.c:939, then
    :1247).  Here the embeddings are zero in dimension 0, only the attention's output matrix writes it, and
    gate and up read nothing else: with parallel residuals (both parts reading the layer's input) the
    feed-forward would see zero there and add nothing, so its output matrix could not matter."""
    from conftest import TINY_A
    c, W = _tiny(dict(TINY_A, num_hidden_layers=1), 8)
    W["model.embed_tokens.weight"][:, 0] = 0.0
    p = "model.layers.0."
    wo = torch.zeros_like(W[p + "self_attn.o_proj.weight"])
    wo[0] = W[p + "self_attn.o_proj.weight"][0] * 40.0            # the attention writes dimension 0 only
    W[p + "self_attn.o_proj.weight"] = wo
    for n in ("mlp.gate_proj.weight", "mlp.up_proj.weight"):
        w = torch.zeros_like(W[p + n])
        w[:, 0] = 1.0 + W[p + n][:, 0].abs() * 10.0                # gate and up read dimension 0 only
        W[p + n] = w
    toks = [3, 200, 17, 5, 9]
    with_ffn = pl.forward(c, W, toks)
    W0 = dict(W)
    W0[p + "mlp.down_proj.weight"] = torch.zeros_like(W[p + "mlp.down_proj.weight"])
    without = pl.forward(c, W0, toks)
    assert float((with_ffn - without).abs().max()) > 1e-2 * float(without.abs().max())
    # by hand for the last token: the stream after the add, normed, through the gated unit
    x = W["model.embed_tokens.weight"][toks]
    H, Hkv, hs = c["heads"], c["kv_heads"], c["head_dim"]
    xb = pl.rmsnorm(x, W[p + "input_layernorm.weight"], c["eps"])
    pos = torch.arange(len(toks))
    f = pl.rope_inv_freq(hs, c["theta"])
    q = pl.apply_rope((xb @ W[p + "self_attn.q_proj.weight"].t()).view(-1, H, hs), pos, f)
    k = pl.apply_rope((xb @ W[p + "self_attn.k_proj.weight"].t()).view(-1, Hkv, hs), pos, f)
    v = (xb @ W[p + "self_attn.v_proj.weight"].t()).view(-1, Hkv, hs)
    x1 = x + pl.attention(q, k, v, 1 / math.sqrt(hs)).reshape(len(toks), H * hs) @ wo.t()
    assert float(x1[:, 0].abs().min()) > 0 and torch.equal(x1[:, 1:], x[:, 1:])
    h = pl.rmsnorm(x1, W[p + "post_attention_layernorm.weight"], c["eps"])
    x2 = x1 + (torch.nn.functional.silu(h @ W[p + "mlp.gate_proj.weight"].t()) * (h @ W[p + "mlp.up_proj.weight"].t())) \
        @ W[p + "mlp.down_proj.weight"].t()
    want = pl.rmsnorm(x2, W["model.norm.weight"], c["eps"]) @ W["lm_head.weight"].t()
    assert torch.allclose(with_ffn, want, atol=1e-5, rtol=1e-4)


def test_tied_output_is_the_embedding_matrix():
    from conftest import TINY_B
    c, W = _tiny(TINY_B, 5)
    toks = [1, 2, 3, 380, 7]
    tied = pl.forward(c, W, toks)
    c2 = dict(c, tied=False)
    W2 = dict(W)
    W2["lm_head.weight"] = W["model.embed_tokens.weight"].clone()
    assert torch.equal(pl.forward(c2, W2, toks), tied)


def test_positions_shift_when_only_distances_count():
    # without the final layers' dependence on absolute position, a shift of all positions changes nothing
    from conftest import TINY_A
    c, W = _tiny(TINY_A, 6)
    toks = [9, 8, 7, 6, 5, 4]
    a = pl.forward(c, W, toks, pos0=0)
    b = pl.forward(c, W, toks, pos0=37)
    assert torch.allclose(a, b, atol=2e-5)


def test_the_shift_of_positions_shows_a_rotation_that_is_not_relative(monkeypatch):
    """What the invariance above catches: a key rotated by another angle than a query at the same position
    (here: keys not rotated at all, and keys rotated the other way round) makes the logits depend on where the
    sequence starts.  The same shift on the faulty forms changes the logits by far more than the bound above."""
    from conftest import TINY_A
    c, W = _tiny(TINY_A, 6)
    toks = [9, 8, 7, 6, 5, 4]
    real = pl.apply_rope
    H, Hkv = c["heads"], c["kv_heads"]
    assert H != Hkv                                               # queries and keys are told apart by their head count

    def keys_unrotated(x, positions, inv_freq):
        return x.clone().to(torch.float32) if x.shape[1] == Hkv else real(x, positions, inv_freq)

    def keys_backwards(x, positions, inv_freq):
        return real(x, -positions if x.shape[1] == Hkv else positions, inv_freq)

    for bad in (keys_unrotated, keys_backwards):
        monkeypatch.setattr(pl, "apply_rope", bad)
        a, b = pl.forward(c, W, toks, pos0=0), pl.forward(c, W, toks, pos0=37)
        assert float((a - b).abs().max()) > 1e-3, bad.__name__
    monkeypatch.setattr(pl, "apply_rope", real)


def test_prefix_logits_do_not_depend_on_the_future():
    from conftest import TINY_B
    c, W = _tiny(TINY_B, 7)
    toks = list(range(20, 33))
    full = pl.forward(c, W, toks)
    assert torch.allclose(pl.forward(c, W, toks[:6]), full[:6], atol=1e-6)


def test_sampler_reference_cases():
    # test/test_safety.c:201-276
    rng = pl.XorShift64Star(42)
    assert pl.sample(torch.tensor([1.0, 3.0, 2.0, 0.5]), 0.0, 0.9, rng) == 1
    assert pl.sample(torch.tensor([5.0]), 0.5, 0.9, rng) == 0
    assert pl.sample(torch.tensor([2.0, 2.1, 2.0, 2.0]), 0.0, 0.9, rng, recent=[1, 1, 1], penalty=1.5) != 1
    assert pl.sample(torch.tensor([1.0, 5.0, 1.0, 1.0]), 0.0, 0.9, rng, recent=[], penalty=1.5) == 1
    rng = pl.XorShift64Star(42)
    hits = sum(pl.sample(torch.tensor([10.0, 0.0, 0.0, 0.0]), 1.0, 0.5, rng) == 0 for _ in range(100))
    assert hits > 80
    assert pl.sample(torch.tensor([1.0, 1.0, 1.0]), 0.0, 0.9, rng) == 0          # first of equal maxima


class _Fixed:
    """Stands in for the generator: hands out the given numbers."""

    def __init__(self, *values):
        self.values = list(values)

    def next_float(self):
        return self.values.pop(0)


def test_top_p_nucleus_vectors():
    """src/sampler.c:77-135 on probabilities 0.15, 0.5, 0.05, 0.3 with top-p 0.9: candidates sorted by falling
    probability (tokens 1, 3, 0, 2), cut at the first whose running sum exceeds 0.9 (token 0 at 0.95, included),
    and the walk compares r * 0.95, the kept sum and neither 1 nor top-p, with the running sums."""
    logits = torch.log(torch.tensor([0.15, 0.5, 0.05, 0.3]))
    def pick(r):
        return pl.sample(logits, 1.0, 0.9, _Fixed(r))
    assert pick(0.0) == 1 and pick(0.52) == 1          # 0.52 * 0.95 = 0.494 < 0.5; unscaled it would be past 0.5
    assert pick(0.53) == 3                             # 0.5035
    assert pick(0.55) == 3                             # 0.5225; scaled by top-p (0.495) it would still be token 1
    assert pick(0.84) == 3 and pick(0.85) == 0         # 0.798 < 0.8 <= 0.8075
    assert pick(0.9999) == 0                           # token 2 lies beyond the cut and is never drawn
    # top-p outside (0, 1): the plain walk over all tokens in index order
    assert pl.sample(logits, 1.0, 1.0, _Fixed(0.66)) == 2 and pl.sample(logits, 1.0, 0.0, _Fixed(0.14)) == 0
    # temperature divides the logits first: at 0.5 the probabilities are squared and renormalised
    sq = torch.tensor([0.15, 0.5, 0.05, 0.3]) ** 2
    sq = sq / sq.sum()
    r = float(sq[1]) / float(sq[1] + sq[3]) * 0.999    # top-p 0.9 keeps tokens 1 and 3 (0.686 + 0.247 > 0.9)
    assert pl.sample(logits, 0.5, 0.9, _Fixed(r)) == 1 and pl.sample(logits, 0.5, 0.9, _Fixed(r * 1.002)) == 3


def test_top_p_cutoff_only_shortens_the_sort():
    """Tokens below (1 - p) / (n - 1) are dropped before the sort (src/sampler.c:88-98).  They could not have
    been kept anyway: were the first token whose running sum exceeds p (not the very first of all) below the
    cutoff, everything from it on, at most n - 1 tokens none larger than it, would weigh less than 1 - p,
    while the sum before it is at most p.  So the draw is the same as from the nucleus built over all tokens,
    which is what pins the rule here: random distributions, with many tokens under the cutoff, against a
    nucleus written without any cutoff."""
    g = torch.Generator().manual_seed(5)
    for trial in range(200):
        n = int(torch.randint(2, 40, (1,), generator=g))
        logits = torch.randn(n, generator=g) * float(torch.rand(1, generator=g) * 6 + 0.5)
        top_p = float(torch.rand(1, generator=g) * 0.9 + 0.05)
        r = float(torch.rand(1, generator=g))
        p = torch.softmax(logits, 0)
        if float(p.max()) < (1.0 - top_p) / (n - 1):
            continue                                   # every token under the cutoff: the reference reads out of bounds
        order = sorted(range(n), key=lambda i: (-float(p[i]), i))
        cum, kept = 0.0, []
        for i in order:
            kept.append(i)
            cum += float(p[i])
            if cum > top_p:
                break
        acc, want = 0.0, kept[-1]
        for i in kept:
            acc += float(p[i])
            if r * cum < acc:
                want = i
                break
        below = int((p < (1.0 - top_p) / (n - 1)).sum())
        assert pl.sample(logits, 1.0, top_p, _Fixed(r)) == want, (trial, n, top_p, below)


def test_rng_is_xorshift64star():
    r = pl.XorShift64Star(0)                     # seed 0 means 42 (src/sampler.c:22)
    s = pl.XorShift64Star(42)
    a = [r.next_u32() for _ in range(4)]
    assert a == [s.next_u32() for _ in range(4)]
    # one step by hand
    st = 42
    st ^= st >> 12
    st ^= (st << 25) & ((1 << 64) - 1)
    st ^= st >> 27
    assert a[0] == ((st * 0x2545F4914F6CDD1D) & ((1 << 64) - 1)) >> 32
    f = pl.XorShift64Star(7).next_float()
    assert 0.0 <= f < 1.0


def test_multinomial_follows_the_distribution():
    rng = pl.XorShift64Star(123)
    logits = torch.log(torch.tensor([0.1, 0.6, 0.3]))
    counts = [0, 0, 0]
    for _ in range(3000):
        counts[pl.sample(logits, 1.0, 1.0, rng)] += 1
    assert abs(counts[1] / 3000 - 0.6) < 0.04 and abs(counts[0] / 3000 - 0.1) < 0.03
