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
    # continuity at both thresholds: a wavelength just inside the band is close to the band's end value
    w = 2 * math.pi / base.double()
    lo_edge, hi_edge = 64 / 1.0, 64 / 4.0
    assert any(hi_edge < x < lo_edge for x in w.tolist()), "the test configuration has no band member"


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
    only = pl.attention(q[8:9], k[5:9], v[5:9], 0.3)               # query 8 sees keys 5..8 (no rope here)
    # the one query must be the last of its four keys: run it as a 4-token sequence's last row
    four = pl.attention(torch.cat([q[5:8], q[8:9]]), k[5:9], v[5:9], 0.3)
    assert torch.allclose(win[8], four[3], atol=1e-6) and not torch.allclose(win[8], full[8], atol=1e-4)
    del only


def test_swiglu_reference_vector():
    # test/test_transformer.c:645-677, the exact-activation mode
    g = torch.tensor([-2.0, -1.0, -0.25, 0.0, 0.25, 1.0, 2.0, 4.0])
    u = torch.tensor([1.0, 0.5, 2.0, 3.0, -1.0, 1.5, -0.5, 2.0])
    assert torch.allclose(pl.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-6)
    assert torch.allclose(pl.swiglu(g, u), (g / (1 + torch.exp(-g))) * u, atol=0)


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
    # and a wrong pairing would break exactly this: rotate interleaved pairs instead
    assert not torch.allclose(a, pl.forward(c, W, toks[::-1]), atol=1e-3)


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
