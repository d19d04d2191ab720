"""Plain, slow implementation of the dense Llama-style decoder, for tests only.

Whole sequences, no cache, one function per part, CPU tensors.  It shares no code
with the package under test: it has its own config reading, its own safetensors
reading (through the `safetensors` library) and its own sampler.  Each function
cites the lines of the reference (artalis-io/bitnet.c, paths from its root) whose formula it
writes out.

Everything is computed in float32 with float64 sums where the reference has them.
`round_to` (a torch dtype or None) rounds activations where an engine that keeps
activations in a narrower type would store them; None keeps float32 throughout.
"""
from __future__ import annotations

import json
import math
import os

import torch

F32 = torch.float32
F64 = torch.float64


def _rt(x: torch.Tensor, round_to) -> torch.Tensor:
    if round_to is None:
        return x
    return x.to(round_to).to(F32)


# ----------------------------------------------------------------------------------
# configuration (own reader; defaults from src/model.c:252-266 and include/model_config.h:6-7)
# ----------------------------------------------------------------------------------

def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        raw = json.load(f)
    c = {}
    c["dim"] = int(raw["hidden_size"])
    c["ffn"] = int(raw["intermediate_size"])
    c["layers"] = int(raw["num_hidden_layers"])
    c["heads"] = int(raw["num_attention_heads"])
    # head_count_kv == 0 / absent -> equals head_count (src/model.c:252-254)
    c["kv_heads"] = int(raw.get("num_key_value_heads") or c["heads"])
    # attention.key_length given -> head size, else dim / heads (src/model.c:285-287)
    c["head_dim"] = int(raw.get("head_dim") or c["dim"] // c["heads"])
    c["vocab"] = int(raw["vocab_size"])
    c["theta"] = float(raw.get("rope_theta") or 10000.0)      # src/model.c:259-260
    c["eps"] = float(raw.get("rms_norm_eps") or 1e-5)         # src/model.c:264-266
    c["tied"] = bool(raw.get("tie_word_embeddings", False))   # src/model.c:453,486-493
    c["rope_scaling"] = raw.get("rope_scaling")
    c["act"] = raw.get("hidden_act", "silu")                  # SiLU for this architecture (src/model_arch.c:807-810)
    c["max_pos"] = int(raw.get("max_position_embeddings", 0))
    return c


def read_weights(folder: str) -> dict:
    from safetensors.torch import load_file
    return {k: v.to(F32) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


# ----------------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------------

def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """out_i = x_i * (1/sqrt(mean(x^2) + eps)) * w_i, eps inside the root, the sum of
    float32 squares accumulated in double (src/transformer/rmsnorm_scalar.c:4-13)."""
    x = x.to(F32)
    sq = (x * x).to(F64)                       # the products are float32, the sum is double
    mean = (sq.sum(dim=-1, keepdim=True) / x.shape[-1]).to(F32)
    scale = 1.0 / torch.sqrt(mean + torch.tensor(eps, dtype=F32))
    return x * scale * w.to(F32)               # that multiplication order


def rope_inv_freq(head_dim: int, theta: float, rope_scaling: dict | None = None,
                  rope_dims: int | None = None) -> torch.Tensor:
    """f_i = theta^(-2i/rope_dims), i < rope_dims/2 (src/model_arch.c:322-338 builds the
    same geometric sequence by repeated multiplication; test/test_transformer.c:408-412
    writes it as 1/powf(theta, 2i/head_size)).  Computed in double, rounded once.

    llama3 scaling has no counterpart in the reference; it is written from its
    definition: wavelengths shorter than orig/high stay, longer than orig/low are
    divided by `factor`, and those between are interpolated linearly in orig/wavelength."""
    rd = rope_dims or head_dim
    i = torch.arange(rd // 2, dtype=F64)
    f = theta ** (-2.0 * i / rd)
    if rope_scaling:
        kind = rope_scaling.get("rope_type", rope_scaling.get("type"))
        if kind == "llama3":
            factor = float(rope_scaling["factor"])
            low = float(rope_scaling["low_freq_factor"])
            high = float(rope_scaling["high_freq_factor"])
            orig = float(rope_scaling["original_max_position_embeddings"])
            wavelen = 2.0 * math.pi / f
            smooth = (orig / wavelen - low) / (high - low)
            mid = (1.0 - smooth) * f / factor + smooth * f
            f = torch.where(wavelen < orig / high, f, torch.where(wavelen > orig / low, f / factor, mid))
        elif kind not in (None, "default"):
            raise ValueError(f"rope scaling {kind!r}")
    return f.to(F32)


def apply_rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """x: [T, n_heads, head_dim].  Split-half pairs (i, i + rope_dims/2):
    out[i] = v0*cos - v1*sin, out[i+half] = v0*sin + v1*cos
    (src/transformer/cpu_backend.c:283-296); angle = pos * f_i in float32, cosf/sinf
    (src/transformer.c:143-162).  Dimensions beyond rope_dims pass through."""
    half = inv_freq.numel()
    ang = positions.to(F32)[:, None] * inv_freq[None, :]        # [T, half] float32
    cos = torch.cos(ang)[:, None, :]
    sin = torch.sin(ang)[:, None, :]
    out = x.clone().to(F32)
    v0 = x[..., :half].to(F32)
    v1 = x[..., half:2 * half].to(F32)
    out[..., :half] = v0 * cos - v1 * sin
    out[..., half:2 * half] = v0 * sin + v1 * cos
    return out


def softmax(scores: torch.Tensor) -> torch.Tensor:
    """max-subtract, exp, sum in double, scale (src/transformer/math_scalar.c:38-68; the
    exact expf of the online variant, not the polynomial)."""
    m = scores.max(dim=-1, keepdim=True).values
    e = torch.exp(scores - m)
    s = e.to(F64).sum(dim=-1, keepdim=True)
    return (e.to(F64) / s).to(F32)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
              window: int | None = None) -> torch.Tensor:
    """q: [T, H, hs] (rotated), k, v: [T, Hkv, hs] (k rotated).  For head h the kv head
    is h // (H/Hkv) (src/transformer/gqa_scalar.c:77); score = (q.k)*scale, product
    first (gqa_scalar.c:92-93); only positions <= the query's are visited, there is
    no mask tensor (gqa_scalar.c:69,80; batched_attn_scalar.c:127-141); softmax; then
    the weighted sum of value rows in position order (gqa_scalar.c:104-119).
    `window`: only the last `window` positions are visited (the ring buffer of
    src/transformer.c:139 seen as a sliding window)."""
    T, H, hs = q.shape
    Hkv = k.shape[1]
    kv_mul = H // Hkv
    out = torch.zeros(T, H, hs, dtype=F32)
    for h in range(H):
        kh = h // kv_mul
        for t in range(T):
            lo = 0 if window is None else max(0, t - window + 1)
            kk = k[lo:t + 1, kh].to(F32)                  # [n_kv, hs]
            s = (kk @ q[t, h].to(F32)) * scale
            p = softmax(s[None, :])[0]
            out[t, h] = (p[:, None] * v[lo:t + 1, kh].to(F32)).sum(dim=0)
    return out


def silu(g: torch.Tensor) -> torch.Tensor:
    """g / (1 + exp(-g)), the exact form (src/transformer/cpu_backend.c:356, :387)."""
    return g / (1.0 + torch.exp(-g))


def gelu_tanh(g: torch.Tensor) -> torch.Tensor:
    """0.5 g (1 + tanh(0.7978845608 g (1 + 0.044715 g^2))) (src/transformer/cpu_backend.c:27-29, without its
    rounding of g and of the result to half precision)."""
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * g * (1.0 + 0.044715 * g * g)))


def relu2(g: torch.Tensor) -> torch.Tensor:
    """max(g, 0)^2 (src/transformer/cpu_backend.c:349-350)."""
    return torch.clamp(g, min=0.0) ** 2


GATE_ACTIVATIONS = {"silu": silu, "gelu_pytorch_tanh": gelu_tanh, "gelu_tanh": gelu_tanh, "relu2": relu2}


def swiglu(g: torch.Tensor, u: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """hb[i] = act(hb[i]) * hb2[i], act = silu for this architecture (src/transformer/cpu_backend.c:365-391)."""
    return GATE_ACTIVATIONS[act](g) * u


def linear(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor | None = None) -> torch.Tensor:
    """out[row] = sum_col W[row, col] * x[col], W row-major [out, in]
    (src/quant/f32_scalar.c:4-32, src/model.c:157-158); a bias, where the model has the
    tensor, is added after the product (src/transformer/cpu.c:871-873)."""
    y = x.to(F32) @ w.to(F32).t()
    return y if b is None else y + b.to(F32)


def feed_forward(xb: torch.Tensor, wg, wu, wd, round_to=None, bg=None, bu=None, bd=None, act: str = "silu") -> torch.Tensor:
    """gate, up -> act(gate)*up -> down (src/transformer/cpu.c:1270-1303)."""
    g = _rt(linear(xb, wg, bg), round_to)
    u = _rt(linear(xb, wu, bu), round_to)
    h = _rt(swiglu(g, u, act), round_to)
    return _rt(linear(h, wd, bd), round_to)


# ----------------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------------

def decoder_layer(x, positions, W, l, c, inv_freq, round_to=None, window=None):
    """norm -> q,k,v -> rope -> attention over all earlier positions -> o -> add ->
    norm -> gate/up -> act*up -> down -> add (src/transformer/cpu.c:536-939, :1247-1303)."""
    p = f"model.layers.{l}."
    T = x.shape[0]
    H, Hkv, hs = c["heads"], c["kv_heads"], c["head_dim"]
    xb = _rt(rmsnorm(x, W[p + "input_layernorm.weight"], c["eps"]), round_to)
    b = lambda name: W.get(p + name)              # optional bias tensors (Llama checkpoints have none)
    q = _rt(linear(xb, W[p + "self_attn.q_proj.weight"], b("self_attn.q_proj.bias")), round_to).view(T, H, hs)
    k = _rt(linear(xb, W[p + "self_attn.k_proj.weight"], b("self_attn.k_proj.bias")), round_to).view(T, Hkv, hs)
    v = _rt(linear(xb, W[p + "self_attn.v_proj.weight"], b("self_attn.v_proj.bias")), round_to).view(T, Hkv, hs)
    q = _rt(apply_rope(q, positions, inv_freq), round_to)
    k = _rt(apply_rope(k, positions, inv_freq), round_to)     # the cache holds rotated keys
    scale = 1.0 / math.sqrt(hs)                               # src/model_arch.c:141-145
    o = _rt(attention(q, k, v, scale, window).reshape(T, H * hs), round_to)
    x = x + _rt(linear(o, W[p + "self_attn.o_proj.weight"], b("self_attn.o_proj.bias")), round_to)
    xb = _rt(rmsnorm(x, W[p + "post_attention_layernorm.weight"], c["eps"]), round_to)
    x = x + feed_forward(xb, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"],
                         W[p + "mlp.down_proj.weight"], round_to, b("mlp.gate_proj.bias"), b("mlp.up_proj.bias"),
                         b("mlp.down_proj.bias"), c.get("act", "silu"))
    return x


def forward(c: dict, W: dict, tokens, round_to=None, pos0: int = 0, emb_scale: float = 1.0,
            softcap: float = 0.0) -> torch.Tensor:
    """Logits [T, vocab] (float32) of one whole sequence.  Embedding row, layers, final
    norm, output matrix or the embedding matrix when tied
    (src/model_embed.c:6-28, src/transformer.c:128-169, src/transformer/logits.c:249-314).
    emb_scale multiplies the embedding row (src/model_embed.c:23-27) and softcap > 0 bounds the
    logits, tanh(logit / cap) * cap (src/transformer/logits.c:325-333); this architecture uses neither."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(pos0, pos0 + tokens.numel())
    inv_freq = rope_inv_freq(c["head_dim"], c["theta"], c["rope_scaling"])
    x = W["model.embed_tokens.weight"][tokens].to(F32) * emb_scale
    for l in range(c["layers"]):
        x = decoder_layer(x, positions, W, l, c, inv_freq, round_to)
    xn = _rt(rmsnorm(x, W["model.norm.weight"], c["eps"]), round_to)
    out_w = W["model.embed_tokens.weight"] if c["tied"] else W["lm_head.weight"]
    logits = linear(xn, out_w)
    if softcap > 0.0:
        logits = torch.tanh(logits * (1.0 / softcap)) * softcap
    return logits


# ----------------------------------------------------------------------------------
# sampler (src/sampler.c) and a generation loop without a cache (src/generate.c:110-234)
# ----------------------------------------------------------------------------------

class XorShift64Star:
    """state ^= state>>12; ^= state<<25; ^= state>>27; high 32 bits of state*0x2545F4914F6CDD1D;
    float = (u32 >> 8) / 2^24 (src/sampler.c:6-15, include/sampler.h:6-7); seed 0 -> 42
    (src/sampler.c:22)."""
    MASK = (1 << 64) - 1

    def __init__(self, seed: int):
        self.state = (seed or 42) & self.MASK

    def next_u32(self) -> int:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & self.MASK
        s ^= s >> 27
        self.state = s
        return ((s * 0x2545F4914F6CDD1D) & self.MASK) >> 32

    def next_float(self) -> float:
        return (self.next_u32() >> 8) / 16777216.0


def apply_repeat_penalty(logits: torch.Tensor, recent: list, penalty: float) -> torch.Tensor:
    """each distinct recent token once: logit > 0 ? /p : *p (src/sampler.c:137-157)."""
    out = logits.clone()
    seen = set()
    for tok in recent:
        if tok in seen or not (0 <= tok < out.numel()):
            continue
        seen.add(tok)
        out[tok] = out[tok] / penalty if out[tok] > 0 else out[tok] * penalty
    return out


def sample(logits: torch.Tensor, temperature: float, top_p: float, rng: XorShift64Star,
           recent: list | None = None, penalty: float = 1.0) -> int:
    """src/sampler.c:137-172: penalty, then argmax at temperature 0 (first index of the
    maximum, src/sampler_backend.c:129-134), else logits/T, softmax with a float32 sum,
    and the cdf walk `r < cdf`; top-p (0 < p < 1): drop below (1-p)/(n-1), sort
    descending, cut where the cumulative sum exceeds p, walk r*cumulative."""
    x = logits.to(F32).clone()
    n = x.numel()
    if penalty != 1.0 and recent:
        x = apply_repeat_penalty(x, recent, penalty)
    if temperature == 0.0:
        return int(torch.argmax(x))            # torch returns the first maximal index
    x = x / temperature
    p = torch.exp(x - x.max())
    p = p / p.sum()
    if top_p <= 0.0 or top_p >= 1.0:
        r = rng.next_float()
        cdf = torch.cumsum(p, 0)
        idx = torch.nonzero(r < cdf)
        return int(idx[0]) if idx.numel() else n - 1
    if n == 1:
        return 0
    cutoff = (1.0 - top_p) / (n - 1)
    cand = torch.nonzero(p >= cutoff)[:, 0]
    order = torch.argsort(p[cand], descending=True, stable=True)
    cand = cand[order]
    cp = p[cand]
    cum = 0.0
    last = cand.numel() - 1
    for i in range(cand.numel()):
        cum += float(cp[i])
        if cum > top_p:
            last = i
            break
    r = rng.next_float() * cum
    cdf = 0.0
    for i in range(last + 1):
        cdf += float(cp[i])
        if r < cdf:
            return int(cand[i])
    return int(cand[last])


def generate(c: dict, W: dict, prompt, max_new: int, temperature: float = 0.0, top_p: float = 0.9,
             seed: int = 42, stop_ids=(), penalty: float = 1.0, window: int = 64,
             round_to=None) -> list:
    """Sample from the logits of the last position; a stop token ends the sequence and
    is not emitted; after max_new tokens no further forward is run
    (src/generate.c:156-160, :212-213, :227-229).  Prompt tokens feed the penalty ring
    (src/main.c:1648-1650).  The whole sequence is run again for every token."""
    rng = XorShift64Star(seed)
    seq = list(prompt)
    recent = list(prompt)[-window:] if penalty != 1.0 else []
    out = []
    while len(out) < max_new:
        logits = forward(c, W, seq, round_to)[-1]
        tok = sample(logits, temperature, top_p, rng, recent, penalty)
        if tok in stop_ids:
            break
        out.append(tok)
        seq.append(tok)
        if penalty != 1.0:
            recent = (recent + [tok])[-window:]
    return out
