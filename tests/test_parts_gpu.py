"""Each part alone against the plain implementation; the order of layers as data (a layer named
twice, a layer that reads another layer's cache); and toy parts defined here, registered, built
and stepped without a change to the library's files: a mixer with a state of its own, a
feed-forward with routing, another position encoding, another norm and another arrangement of
a layer's parts."""
import json
import math
import os
import random
from dataclasses import asdict, dataclass

import pytest
import torch

import plain_llama as pl
from conftest import TOL, part_close, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _rand(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def _ctx(cache, slots, n_new, dtype, tokens=None):
    """A StepContext and block tables for hand-driven parts, the way the engine makes them."""
    from bitnet_c_amd.engine.step import StepContext
    pos0 = [cache.length(s) for s in slots]
    cache.reserve(slots, n_new)
    positions, seq_index = [], []
    for i, (p, n) in enumerate(zip(pos0, n_new)):
        positions += list(range(p, p + n))
        seq_index += [i] * n
    T = sum(n_new)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    ctx = StepContext(torch.device(DEV), dtype, i32(tokens or [0] * T), i32(positions), i32(seq_index),
                      i32([p + n for p, n in zip(pos0, n_new)]), i32(list(range(T))), i32(slots),
                      all(n == 1 for n in n_new), slots, n_new, pos0)
    tables = {g: cache.block_table(g, slots).to(DEV) for g in range(len(cache.groups))}
    return ctx, tables, max(p + n for p, n in zip(pos0, n_new))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_and_feed_forward_parts(dtype):
    from bitnet_c_amd.parts import FEED_FORWARDS, NORMS, PartSpec
    norm = NORMS.build(PartSpec.of("rmsnorm", dim=72, eps=1e-4))
    w = _rand((72,), 1) + 1.0
    norm.load({"weight": w}, DEV, dtype)
    x = _rand((9, 72), 2, 2.0)
    assert part_close(norm.apply(x.to(DEV), None, dtype).float(), pl.rmsnorm(x, w, 1e-4), dtype)
    ffn = FEED_FORWARDS.build(PartSpec.of("swiglu", hidden=72, intermediate=100))
    assert {k: v.shape for k, v in ffn.tensors().items()} == {"w_gate": (100, 72), "w_up": (100, 72), "w_down": (72, 100)}
    t = {"w_gate": _rand((100, 72), 3, 0.1).to(dtype), "w_up": _rand((100, 72), 4, 0.1).to(dtype),
         "w_down": _rand((72, 100), 5, 0.1).to(dtype)}
    ffn.load(t, DEV, dtype)
    rt = None if dtype == torch.float32 else dtype
    for T in (1, 9, 70):                                        # decode-sized and prompt-sized products
        h = _rand((T, 72), 6).to(dtype)
        got = ffn.forward(h.to(DEV), None)
        want = pl.feed_forward(h.float(), t["w_gate"].float(), t["w_up"].float(), t["w_down"].float(), rt)
        exact = pl.feed_forward(h.float(), t["w_gate"].float(), t["w_up"].float(), t["w_down"].float())
        assert part_close(got.float(), want, dtype, exact), T
    # a feed-forward with biases
    fb = FEED_FORWARDS.build(PartSpec.of("swiglu", hidden=72, intermediate=100, bias=True))
    tb = dict(t, b_gate=_rand((100,), 7, 0.1), b_up=_rand((100,), 8, 0.1), b_down=_rand((72,), 9, 0.1))
    fb.load(tb, DEV, dtype)
    h = _rand((5, 72), 10).to(dtype)
    def with_bias(r):
        g = r(r(pl.linear(h.float(), t["w_gate"])) + tb["b_gate"])
        u = r(r(pl.linear(h.float(), t["w_up"])) + tb["b_up"])
        return r(r(pl.linear(r(pl.swiglu(g, u)), t["w_down"])) + tb["b_down"])
    exact = with_bias(lambda x: x)
    want = with_bias((lambda x: x) if dtype == torch.float32 else (lambda x: x.to(dtype).float()))
    assert part_close(fb.forward(h.to(DEV), None).float(), want, dtype, exact)


@pytest.mark.parametrize("T", [8, 40, 64, 128, 200])
def test_a_feed_forward_s_last_product_reaches_the_stream_in_every_form(T):
    """bfloat16: at 8 rows the last product adds itself to the stream and leaves the norm deferred, at 40, 64 and 128
    rows it comes as partial sums over ranges of K that the kernels of the next norm add up, at 200 rows as a
    tensor.  The stream and the normed rows are the plain formulas' in every form; a norm that knows only tensors
    (defined here) gets the sum formed for it."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.parts import FEED_FORWARDS, NORMS, LazyDelta, PartSpec, ResidualStream
    dtype, D, F = torch.bfloat16, 1024, 2048                     # K = 2,048 columns of the last product: four ranges
    ffn = FEED_FORWARDS.build(PartSpec.of("swiglu", hidden=D, intermediate=F))
    t = {"w_gate": _rand((F, D), 3, 0.05).to(dtype), "w_up": _rand((F, D), 4, 0.05).to(dtype),
         "w_down": _rand((D, F), 5, 0.05).to(dtype)}
    ffn.load(t, DEV, dtype)
    norm = NORMS.build(PartSpec.of("rmsnorm", dim=D, eps=1e-5))
    nw = _rand((D,), 6) * 0.2 + 1.0
    norm.load({"weight": nw}, DEV, dtype)
    h, x0 = _rand((T, D), 7).to(dtype), _rand((T, D), 8, 2.0)
    delta = ffn.forward(h.to(DEV), None, lazy_ok=True)
    kind = LazyDelta if T <= 16 else ops.PartialSums if 17 <= T <= 128 else torch.Tensor
    assert isinstance(delta, kind), type(delta)
    if kind is ops.PartialSums:
        assert delta.slabs.shape[0] == 4
    act = pl.swiglu(pl.linear(h.float(), t["w_gate"].float()).to(dtype).float(), pl.linear(h.float(), t["w_up"].float()).to(dtype).float())
    exact_x = x0.double() + pl.linear(act.to(dtype).float(), t["w_down"].float()).double()

    class TensorsOnlyNorm:
        weight, eps = norm.weight, norm.eps

        def apply(self, x, d, out_dtype, rows=None):
            assert d is None or isinstance(d, torch.Tensor)
            return ops.add_rmsnorm(x, d, self.weight, self.eps, out_dtype, rows)

    for n in (norm, TensorsOnlyNorm()):
        stream = ResidualStream(x0.clone().to(DEV))
        stream.add(ffn.forward(h.to(DEV), None, lazy_ok=True))
        got = stream.normed(n, dtype, consumer=None)
        assert stream.pending is None
        # the activations of the last product differ from the plain ones by one bf16 step here and there, and the plain
        # path at 200 rows rounds the product to bf16 before it is added
        assert rel_err(stream.x, exact_x.float()) < 2e-2
        assert part_close(got.float(), pl.rmsnorm(exact_x.float(), nw, 1e-5).to(dtype).float(), dtype,
                          pl.rmsnorm(exact_x.float(), nw, 1e-5))
    if 17 <= T <= 128:
        # a consumer that applies the norm itself gets it undone: one kernel forms the sum and leaves the factor
        stream = ResidualStream(x0.clone().to(DEV))
        stream.add(ffn.forward(h.to(DEV), None, lazy_ok=True))
        pre = stream.normed(norm, dtype, consumer=ffn)
        assert isinstance(pre, ops.DeferredNorm) and stream.pending is None
        assert rel_err(stream.x, exact_x.float()) < 2e-2
        assert part_close(pre.materialize().float(), pl.rmsnorm(exact_x.float(), nw, 1e-5).to(dtype).float(), dtype,
                          pl.rmsnorm(exact_x.float(), nw, 1e-5))
        # and the feed-forward that consumes it gives what it gives for the normed rows
        plain_in = pl.rmsnorm(exact_x.float(), nw, 1e-5)
        want = pl.feed_forward(plain_in.to(dtype).float(), t["w_gate"].float(), t["w_up"].float(), t["w_down"].float(), dtype)
        exact = pl.feed_forward(plain_in, t["w_gate"].float(), t["w_up"].float(), t["w_down"].float())
        assert part_close(ffn.forward(pre, None).float(), want, dtype, exact)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv,hs,window,pos_kind", [(6, 2, 32, 0, "rope"), (4, 4, 16, 40, "rope"), (3, 1, 24, 0, "none")])
def test_attention_part_alone(dtype, H, Hkv, hs, window, pos_kind):
    """The mixer with its own cache entry: prompts of unequal lengths, then tokens one by one,
    against plain attention over the whole sequences."""
    from bitnet_c_amd.cache import PagedCache
    from bitnet_c_amd.parts import MIXERS, PartSpec
    hidden, scale = 48, 0.2
    pos = PartSpec.of("rope", head_dim=hs, theta=5000.0, rope_dims=hs // 2) if pos_kind == "rope" else PartSpec.of("none")
    att = MIXERS.build(PartSpec.of("attention", hidden=hidden, n_heads=H, n_kv_heads=Hkv, head_dim=hs, scale=scale,
                                   position=pos, window=window))
    t = {k: _rand(v.shape, 20 + i, 0.15).to(dtype) for i, (k, v) in enumerate(att.tensors().items())}
    att.load(t, DEV, dtype)
    cache = PagedCache([att.cache_need()], [None], 64 * 8, dtype=dtype, device=DEV)
    lens = [70, 5, 130]
    hs_in = [_rand((n, hidden), 30 + i).to(dtype) for i, n in enumerate(lens)]
    slots = [cache.alloc_slot() for _ in lens]
    got = [[] for _ in lens]
    fed = [n - 3 for n in lens]
    ctx, tables, max_len = _ctx(cache, slots, fed, dtype)
    out = att.forward(torch.cat([h[:f] for h, f in zip(hs_in, fed)]).to(DEV), ctx, cache.view(0, tables, max_len))
    cache.commit(slots, fed)
    o = 0
    for i, f in enumerate(fed):
        got[i].append(out[o:o + f])
        o += f
    for step in range(3):
        ctx, tables, max_len = _ctx(cache, slots, [1] * 3, dtype)
        out = att.forward(torch.stack([h[f + step] for h, f in zip(hs_in, fed)]).to(DEV), ctx,
                          cache.view(0, tables, max_len))
        cache.commit(slots, [1] * 3)
        for i in range(3):
            got[i].append(out[i:i + 1])
    rt = (lambda x: x) if dtype == torch.float32 else (lambda x: x.to(dtype).float())
    inv = pl.rope_inv_freq(hs, 5000.0, None, hs // 2) if pos_kind == "rope" else torch.zeros(0)
    for i, n in enumerate(lens):
        h = hs_in[i].float()
        p = torch.arange(n)
        q = rt(pl.apply_rope(rt(pl.linear(h, t["wq"])).view(n, H, hs), p, inv))
        k = rt(pl.apply_rope(rt(pl.linear(h, t["wk"])).view(n, Hkv, hs), p, inv))
        v = rt(pl.linear(h, t["wv"])).view(n, Hkv, hs)
        a = rt(pl.attention(q, k, v, scale, window or None).reshape(n, H * hs))
        want = rt(pl.linear(a, t["wo"]))
        assert part_close(torch.cat(got[i]).float(), want, dtype), i


def _tiny_folder(tmp_path, dtype=torch.float32):
    from bitnet_c_amd.config import LlamaConfig
    from bitnet_c_amd.weights import write_model_folder
    from conftest import TINY_A
    d = str(tmp_path / "m")
    write_model_folder(d, LlamaConfig.from_dict(dict(TINY_A, num_hidden_layers=3)), 3, dtype)
    return d


def test_the_order_of_layers_is_data(tmp_path):
    """A schedule that names a layer twice (shared weights, a cache entry each) equals the plain
    model with that layer's weights copied; an entry that reads an earlier entry's cache attends
    over that entry's keys and values with its own queries."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import load_config
    from bitnet_c_amd.engine import DecoderModel, ScheduleEntry
    from bitnet_c_amd.weights import load_tensors
    from dataclasses import replace
    folder = _tiny_folder(tmp_path)
    arch, cfg = load_config(folder)
    plan = arch.build_plan(cfg)
    tensors = load_tensors(folder, plan.expected_tensors())
    c, W = pl.read_config(folder), pl.read_weights(folder)
    toks = [random.Random(5).randrange(256) for _ in range(80)]

    def run(schedule):
        model = DecoderModel(replace(plan, schedule=schedule), torch.float32, DEV)
        model.load(tensors)
        eng = Engine(model, max_tokens=256)
        s = eng.new_sequence()
        a = eng.step([StepEntry(s, toks[:70], list(range(70)))])
        b = [eng.step([StepEntry(s, [t], [0])]) for t in toks[70:]]
        return torch.cat([a] + b), eng

    # layers 0, 1, 1, 2
    got, eng = run([ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(2)])
    assert eng.cache.groups[0].k.shape[0] == 4                   # four cache entries for three layers
    W4 = {k: v for k, v in W.items() if ".layers." not in k}
    for new, old in enumerate([0, 1, 1, 2]):
        for k, v in W.items():
            if f".layers.{old}." in k:
                W4[k.replace(f".layers.{old}.", f".layers.{new}.")] = v
    assert rel_err(got, pl.forward(dict(c, layers=4), W4, toks)) < TOL[torch.float32]

    # layer 2 reads the cache of entry 0: plain version written out here
    got, eng = run([ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2, kv_from=0)])
    assert eng.cache.groups[0].k.shape[0] == 2                   # the third entry has no storage
    x = W["model.embed_tokens.weight"][toks]
    pos = torch.arange(len(toks))
    inv = pl.rope_inv_freq(c["head_dim"], c["theta"])
    keep = {}
    for l in range(3):
        p = f"model.layers.{l}."
        xb = pl.rmsnorm(x, W[p + "input_layernorm.weight"], c["eps"])
        q = pl.apply_rope(pl.linear(xb, W[p + "self_attn.q_proj.weight"]).view(-1, 4, 16), pos, inv)
        if l < 2:
            k = pl.apply_rope(pl.linear(xb, W[p + "self_attn.k_proj.weight"]).view(-1, 2, 16), pos, inv)
            v = pl.linear(xb, W[p + "self_attn.v_proj.weight"]).view(-1, 2, 16)
            keep[l] = (k, v)
        else:
            k, v = keep[0]
        o = pl.attention(q, k, v, 0.25).reshape(len(toks), 64)
        x = x + pl.linear(o, W[p + "self_attn.o_proj.weight"])
        xb = pl.rmsnorm(x, W[p + "post_attention_layernorm.weight"], c["eps"])
        x = x + pl.feed_forward(xb, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"], W[p + "mlp.down_proj.weight"])
    want = pl.linear(pl.rmsnorm(x, W["model.norm.weight"], c["eps"]), W["lm_head.weight"])
    assert rel_err(got, want) < TOL[torch.float32]


def test_an_entry_reads_another_entry_s_blocked_pages(tmp_path):
    """bfloat16 at the head size and grouping of the benchmark shape (128, four query heads per kv head): the cache keeps
    blocked pages, which only the matrix-core kernels read.  A schedule whose third entry runs layer 1's weights again
    over the keys and values of entry 0 (it writes nothing): a prompt of 150 tokens whole, and 100 of them followed by 50
    one by one (the decode kernel then reads the pages without storing into them), against the plain computation."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import LlamaConfig, load_config
    from bitnet_c_amd.engine import DecoderModel, ScheduleEntry
    from bitnet_c_amd.weights import load_tensors, write_model_folder
    from conftest import TINY_E
    from dataclasses import replace
    folder = str(tmp_path / "e")
    write_model_folder(folder, LlamaConfig.from_dict(TINY_E), 21, torch.bfloat16)
    arch, cfg = load_config(folder)
    plan = arch.build_plan(cfg)
    plan = replace(plan, schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1, kv_from=0)])
    model = DecoderModel(plan, torch.bfloat16, DEV)
    model.load(load_tensors(folder, plan.expected_tensors()))
    eng = Engine(model, max_tokens=512)
    assert eng.cache.groups[0].blocked and eng.cache.groups[0].k.shape[0] == 2
    c, W = pl.read_config(folder), pl.read_weights(folder)
    H, Hkv, hd, D = c["heads"], c["kv_heads"], c["head_dim"], c["dim"]
    toks = [random.Random(6).randrange(c["vocab"]) for _ in range(150)]
    s = eng.new_sequence()
    whole = eng.step([StepEntry(s, toks, list(range(150)))])
    eng.release(s)
    s = eng.new_sequence()
    first = eng.step([StepEntry(s, toks[:100], list(range(100)))])
    rest = [eng.step([StepEntry(s, [t], [0])]) for t in toks[100:]]
    eng.release(s)
    eng.cache.check()
    r = lambda x: x.to(torch.bfloat16).float()
    x = W["model.embed_tokens.weight"].float()[toks]
    pos = torch.arange(len(toks))
    inv = pl.rope_inv_freq(hd, c["theta"])
    keep = None
    for e, l in enumerate([0, 1, 1]):
        p = f"model.layers.{l}."
        xb = r(pl.rmsnorm(x, W[p + "input_layernorm.weight"].float(), c["eps"]))
        q = r(pl.apply_rope(r(pl.linear(xb, W[p + "self_attn.q_proj.weight"].float())).view(-1, H, hd), pos, inv))
        if e < 2:
            k = r(pl.apply_rope(r(pl.linear(xb, W[p + "self_attn.k_proj.weight"].float())).view(-1, Hkv, hd), pos, inv))
            v = r(pl.linear(xb, W[p + "self_attn.v_proj.weight"].float())).view(-1, Hkv, hd)
            if e == 0:
                keep = (k, v)
        else:
            k, v = keep
        o = r(pl.attention(q, k, v, hd ** -0.5).reshape(len(toks), H * hd))
        x = x + pl.linear(o, W[p + "self_attn.o_proj.weight"].float())
        xb = r(pl.rmsnorm(x, W[p + "post_attention_layernorm.weight"].float(), c["eps"]))
        x = x + pl.feed_forward(xb, W[p + "mlp.gate_proj.weight"].float(), W[p + "mlp.up_proj.weight"].float(),
                                W[p + "mlp.down_proj.weight"].float())
    want = pl.linear(r(pl.rmsnorm(x, W["model.norm.weight"].float(), c["eps"])), W["model.embed_tokens.weight"].float())
    assert rel_err(whole, want) < TOL[torch.bfloat16]
    assert rel_err(torch.cat([first] + rest), want) < TOL[torch.bfloat16]


# ---------------------------------------------------------------------------------------
# a toy architecture, defined here: layers alternate between attention and a mixer that keeps
# a running decayed sum of its inputs per sequence; nothing of it lives in the library
# ---------------------------------------------------------------------------------------

def _register_toy():
    from bitnet_c_amd.config import Architecture, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.engine import LayerPlan, ModelPlan, ScheduleEntry
    from bitnet_c_amd.parts import MIXERS, CacheNeed, ParamSpec, Part, PartSpec, StateNeed

    if "decay_sum" not in MIXERS:
        @MIXERS.register("decay_sum")
        class DecaySum(Part):
            """s_t = decay * s_{t-1} + h_t ;  out_t = W s_t."""

            def __init__(self, hidden, decay):
                self.hidden, self.decay = hidden, decay

            def tensors(self):
                return {"w": ParamSpec((self.hidden, self.hidden))}

            def load(self, tensors, device, dtype):
                self.w = tensors["w"].to(dtype).to(device)

            def cache_need(self):
                return CacheNeed(state=StateNeed((self.hidden,), torch.float32))

            def forward(self, h, ctx, kv):
                out = torch.empty_like(h)
                for slot, (r0, n) in zip(ctx.slots, ctx.row_ranges()):
                    s = kv.state[slot]
                    for t in range(r0, r0 + n):                 # strictly in order inside a sequence
                        s = self.decay * s + h[t].float()
                        out[t] = (self.w.float() @ s).to(h.dtype)
                    kv.state[slot] = s
                return out

    @dataclass(frozen=True)
    class ToyConfig:
        vocab_size: int
        hidden_size: int
        n_layers: int
        decay: float
        model_type: str = "toy_decay"

        @staticmethod
        def from_dict(raw):
            return ToyConfig(raw["vocab_size"], raw["hidden_size"], raw["n_layers"], raw["decay"])

        def to_dict(self):
            return asdict(self)

    def build(c):
        norm = PartSpec.of("rmsnorm", dim=c.hidden_size, eps=1e-5)
        ffn = PartSpec.of("swiglu", hidden=c.hidden_size, intermediate=2 * c.hidden_size)
        att = PartSpec.of("attention", hidden=c.hidden_size, n_heads=2, n_kv_heads=1, head_dim=c.hidden_size // 2,
                          scale=(c.hidden_size // 2) ** -0.5,
                          position=PartSpec.of("rope", head_dim=c.hidden_size // 2, theta=100.0))
        dec = PartSpec.of("decay_sum", hidden=c.hidden_size, decay=c.decay)
        layers = []
        for i in range(c.n_layers):
            mixer = att if i % 2 == 0 else dec
            blk = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
            from bitnet_c_amd.parts import BLOCKS
            names = {local: f"layers.{i}.{local}" for local in BLOCKS.build(blk).tensors()}
            layers.append(LayerPlan(block=blk, names=names))
        return ModelPlan(vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
                         schedule=[ScheduleEntry(i) for i in range(c.n_layers)], final_norm=norm,
                         embedding_name="embed.weight", final_norm_names={"weight": "norm.weight"},
                         lm_head_name="head.weight")

    if "toy_decay" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_decay", ToyConfig, build))
    return ToyConfig


def test_a_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.weights import write_model_folder
    ToyConfig = _register_toy()
    cfg = ToyConfig(vocab_size=40, hidden_size=32, n_layers=3, decay=0.9)
    folder = write_model_folder(str(tmp_path / "toy"), cfg, 11, torch.float32)
    assert json.load(open(os.path.join(folder, "config.json")))["model_type"] == "toy_decay"
    eng = Engine.from_folder(folder, dtype=torch.float32, max_tokens=512)       # chosen by config.json
    assert not eng.use_graphs and list(eng.cache.states) == [1]
    assert eng.cache.states[1].shape[1:] == (32,) and len(eng.cache.groups) == 1

    # the plain version of the toy model
    from safetensors.torch import load_file
    W = load_file(os.path.join(folder, "model.safetensors"))

    def plain(toks):
        x = W["embed.weight"][toks]
        n = len(toks)
        pos = torch.arange(n)
        for l in range(3):
            p = f"layers.{l}."
            xb = pl.rmsnorm(x, W[p + "mixer_norm.weight"], 1e-5)
            if l % 2 == 0:
                inv = pl.rope_inv_freq(16, 100.0)
                q = pl.apply_rope(pl.linear(xb, W[p + "mixer.wq"]).view(n, 2, 16), pos, inv)
                k = pl.apply_rope(pl.linear(xb, W[p + "mixer.wk"]).view(n, 1, 16), pos, inv)
                v = pl.linear(xb, W[p + "mixer.wv"]).view(n, 1, 16)
                x = x + pl.linear(pl.attention(q, k, v, 0.25).reshape(n, 32), W[p + "mixer.wo"])
            else:
                s, rows = torch.zeros(32), []
                for t in range(n):
                    s = 0.9 * s + xb[t]
                    rows.append(W[p + "mixer.w"] @ s)
                x = x + torch.stack(rows)
            xb = pl.rmsnorm(x, W[p + "ffn_norm.weight"], 1e-5)
            x = x + pl.feed_forward(xb, W[p + "ffn.w_gate"], W[p + "ffn.w_up"], W[p + "ffn.w_down"])
        return pl.linear(pl.rmsnorm(x, W["norm.weight"], 1e-5), W["head.weight"])

    rnd = random.Random(12)
    reqs = [[rnd.randrange(40) for _ in range(n)] for n in (20, 7, 33)]
    # a batch of unequal prompts, then one token each; the state is carried from step to step
    slots = [eng.new_sequence() for _ in reqs]
    fed = [len(r) - 4 for r in reqs]
    out = eng.step([StepEntry(s, r[:f], list(range(f))) for s, r, f in zip(slots, reqs, fed)])
    got, o = [[] for _ in reqs], 0
    for i, f in enumerate(fed):
        got[i].append(out[o:o + f])
        o += f
    for k in range(4):
        out = eng.step([StepEntry(s, [r[f + k]], [0]) for s, r, f in zip(slots, reqs, fed)])
        for i in range(3):
            got[i].append(out[i:i + 1])
    for i, r in enumerate(reqs):
        assert rel_err(torch.cat(got[i]), plain(r)) < TOL[torch.float32], i
    # a slot that is used again starts from a zero state
    eng.release(slots[0])
    s = eng.new_sequence()
    assert s == slots[0]
    again = eng.step([StepEntry(s, reqs[1], list(range(7)))])
    assert rel_err(again, plain(reqs[1])) < TOL[torch.float32]


def test_a_state_mixer_that_addresses_its_state_on_the_device_decodes_under_graphs(tmp_path):
    """The same toy recurrence written against the step's device-side slot ids (ctx.slot_ids) instead of the
    host's slot list, and declared so (StateNeed.device_addressed): its decode steps are captured and
    replayed, padding rows read and write the state row that no sequence owns, and the logits are those of
    the eager engine, bit for bit, with sequences that end at different steps and a slot that is used again."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import Architecture, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.engine import LayerPlan, ModelPlan, ScheduleEntry
    from bitnet_c_amd.parts import BLOCKS, MIXERS, CacheNeed, ParamSpec, Part, PartSpec, StateNeed
    from bitnet_c_amd.weights import write_model_folder

    if "decay_sum_dev" not in MIXERS:
        @MIXERS.register("decay_sum_dev")
        class DecaySumDev(Part):
            """s_t = decay * s_{t-1} + h_t ;  out_t = W s_t, the state addressed by ctx.slot_ids."""

            def __init__(self, hidden, decay):
                self.hidden, self.decay = hidden, decay

            def tensors(self):
                return {"w": ParamSpec((self.hidden, self.hidden))}

            def load(self, tensors, device, dtype):
                self.w = tensors["w"].to(dtype).to(device)

            def cache_need(self):
                return CacheNeed(state=StateNeed((self.hidden,), torch.float32, device_addressed=True))

            def forward(self, h, ctx, kv):
                ids = ctx.slot_ids.long()
                if ctx.is_decode:                                   # one row a sequence: no host loop, capturable
                    s = self.decay * kv.state.index_select(0, ids) + h.float()
                    kv.state.index_copy_(0, ids, s)
                    return (s @ self.w.float().t()).to(h.dtype)
                out = torch.empty_like(h)
                for b, (r0, n) in enumerate(ctx.row_ranges()):
                    s = kv.state[ids[b]]
                    for t in range(r0, r0 + n):
                        s = self.decay * s + h[t].float()
                        out[t] = (self.w.float() @ s).to(h.dtype)
                    kv.state[ids[b]] = s
                return out

    @dataclass(frozen=True)
    class DevConfig:
        vocab_size: int
        hidden_size: int
        model_type: str = "toy_decay_dev"

        @staticmethod
        def from_dict(raw):
            return DevConfig(raw["vocab_size"], raw["hidden_size"])

        def to_dict(self):
            return asdict(self)

    def build(c):
        norm = PartSpec.of("rmsnorm", dim=c.hidden_size, eps=1e-5)
        ffn = PartSpec.of("swiglu", hidden=c.hidden_size, intermediate=2 * c.hidden_size)
        att = PartSpec.of("attention", hidden=c.hidden_size, n_heads=2, n_kv_heads=1, head_dim=c.hidden_size // 2,
                          scale=(c.hidden_size // 2) ** -0.5,
                          position=PartSpec.of("rope", head_dim=c.hidden_size // 2, theta=100.0))
        dec = PartSpec.of("decay_sum_dev", hidden=c.hidden_size, decay=0.8)
        layers = []
        for i, mixer in enumerate((dec, att, dec)):
            blk = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
            layers.append(LayerPlan(block=blk, names={local: f"layers.{i}.{local}" for local in BLOCKS.build(blk).tensors()}))
        return ModelPlan(vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
                         schedule=[ScheduleEntry(i) for i in range(3)], final_norm=norm,
                         embedding_name="embed.weight", final_norm_names={"weight": "norm.weight"},
                         lm_head_name="head.weight")

    if "toy_decay_dev" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_decay_dev", DevConfig, build))
    folder = write_model_folder(str(tmp_path / "toydev"), DevConfig(vocab_size=50, hidden_size=32), 13, torch.float32)
    rnd = random.Random(14)
    reqs = [[rnd.randrange(50) for _ in range(n)] for n in (20, 9, 33)]
    n_dec = [12, 3, 7]
    outs = []
    for graphs in (True, False):
        eng = Engine.from_folder(folder, dtype=torch.float32, max_tokens=512, use_graphs=graphs)
        assert eng.use_graphs == graphs and sorted(eng.cache.states) == [0, 2]
        got = []
        for _ in range(2):                                  # the second round uses the first one's slots again
            slots = [eng.new_sequence() for _ in reqs]
            fed = [len(r) - d for r, d in zip(reqs, n_dec)]
            eng.step([StepEntry(s, r[:f], []) for s, r, f in zip(slots, reqs, fed)])
            live = list(range(3))
            while live:
                got.append(eng.step([StepEntry(slots[i], [reqs[i][fed[i]]], [0]) for i in live]).clone())
                for i in live:
                    fed[i] += 1
                for i in [i for i in live if fed[i] == len(reqs[i])]:
                    eng.release(slots[i])
                live = [i for i in live if fed[i] < len(reqs[i])]
        if graphs:
            assert sorted(eng._graphs) == [1, 2, 4]         # three rows are a graph of four: one padding row
            # the padding row worked on the spare state row and on no sequence's
            assert float(eng.cache.states[0][eng.cache.padding_slot].abs().sum()) > 0
        outs.append(got)
    assert len(outs[0]) == len(outs[1]) == 24
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert torch.equal(torch.cat(outs[0][:12]), torch.cat(outs[0][12:]))      # the second round equals the first


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_an_architecture_with_an_embedding_multiplier_and_a_logit_softcap(tmp_path, dtype):
    """Two fields of the plan, set by a toy architecture's builder: the embedding row times sqrt(hidden) before the
    first block, the logits bounded by cap * tanh(logits / cap).  Prompts and decoded tokens (replayed from graphs)
    against the plain implementation with the same two numbers."""
    from dataclasses import replace
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import Architecture, LlamaConfig, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.config.llama_plan import build_llama_plan
    from bitnet_c_amd.weights import write_model_folder
    from conftest import TINY_D
    scale, cap = math.sqrt(TINY_D["hidden_size"]), 0.4

    class CappedConfig(LlamaConfig):
        @staticmethod
        def from_dict(raw):
            return CappedConfig(**{k: v for k, v in vars(LlamaConfig.from_dict(raw)).items()})

        def to_dict(self):
            return dict(LlamaConfig.to_dict(self), model_type="toy_capped", architectures=["ToyCapped"])

    if "toy_capped" not in _ARCHITECTURES:
        register_architecture(Architecture(
            "toy_capped", CappedConfig,
            lambda c: replace(build_llama_plan(c), embedding_multiplier=math.sqrt(c.hidden_size), logit_softcap=cap)))
    cfg = CappedConfig.from_dict(dict(TINY_D, model_type="toy_capped"))
    folder = write_model_folder(str(tmp_path / "capped"), cfg, 15, dtype)
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=1024)
    assert eng.model.plan.logit_softcap == cap and eng.use_graphs
    c, W = pl.read_config(folder), pl.read_weights(folder)
    rounded = torch.bfloat16 if dtype == torch.bfloat16 else None
    rnd = random.Random(16)
    reqs = [[rnd.randrange(cfg.vocab_size) for _ in range(n)] for n in (40, 7, 71)]
    slots = [eng.new_sequence() for _ in reqs]
    out = eng.step([StepEntry(s, r[:-5], list(range(len(r) - 5))) for s, r in zip(slots, reqs)])
    got, o = [[] for _ in reqs], 0
    for i, r in enumerate(reqs):
        got[i].append(out[o:o + len(r) - 5])
        o += len(r) - 5
    for k in range(5):
        out = eng.step([StepEntry(s, [r[len(r) - 5 + k]], [0]) for s, r in zip(slots, reqs)])
        for i in range(3):
            got[i].append(out[i:i + 1].clone())
    for i, r in enumerate(reqs):
        want = pl.forward(c, W, r, rounded, emb_scale=scale, softcap=cap)
        assert float(want.abs().max()) > 0.5 * cap                          # the cap bites
        assert rel_err(torch.cat(got[i]), want) < TOL[dtype], i
        assert rel_err(pl.forward(c, W, r, rounded, emb_scale=scale), want) > 10 * TOL[dtype]
        assert rel_err(pl.forward(c, W, r, rounded, softcap=cap), want) > 10 * TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_an_architecture_without_a_final_norm_and_with_a_bias_on_its_output_matrix(tmp_path, dtype):
    """The model's skeleton is the plan's to say as well: a toy architecture's builder drops the norm in front of the
    output matrix and names a bias for it.  The folder then holds no final norm and one bias tensor; prompts, decoded
    tokens (from graphs) and a prompt step from its graph equal the plain layers followed by W x + b on the stream itself."""
    from dataclasses import replace
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import Architecture, LlamaConfig, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.config.llama_plan import build_llama_plan
    from bitnet_c_amd.weights import write_model_folder
    from conftest import TINY_A

    class BareConfig(LlamaConfig):
        def to_dict(self):
            return dict(LlamaConfig.to_dict(self), model_type="toy_bare_head", architectures=["ToyBareHead"])

    if "toy_bare_head" not in _ARCHITECTURES:
        register_architecture(Architecture(
            "toy_bare_head", BareConfig,
            lambda c: replace(build_llama_plan(c), final_norm=None, final_norm_names={}, lm_head_bias_name="lm_head.bias")))
    cfg = BareConfig.from_dict(dict(TINY_A, model_type="toy_bare_head"))
    folder = write_model_folder(str(tmp_path / "bare"), cfg, 25, dtype)
    from safetensors.torch import load_file
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    assert "model.norm.weight" not in names and "lm_head.bias" in names
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=1024)
    assert eng.model.final_norm is None and eng.prompt_graphs
    c, W = pl.read_config(folder), pl.read_weights(folder)
    rt = torch.bfloat16 if dtype == torch.bfloat16 else None
    r_ = (lambda x: x) if rt is None else (lambda x: x.to(rt).float())

    def plain(toks):
        x = W["model.embed_tokens.weight"][torch.tensor(toks)].float()
        inv = pl.rope_inv_freq(c["head_dim"], c["theta"], c["rope_scaling"])
        for l in range(c["layers"]):
            x = pl.decoder_layer(x, torch.arange(len(toks)), W, l, c, inv, rt)
        return pl.linear(r_(x), W["lm_head.weight"].float(), W["lm_head.bias"].float())

    rnd = random.Random(26)
    reqs = [[rnd.randrange(cfg.vocab_size) for _ in range(n)] for n in (30, 9)]
    for round_ in range(3):                       # the third round's prompt step is a replay of the second's graph
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([StepEntry(s, r[:-3], list(range(len(r) - 3))) for s, r in zip(slots, reqs)])
        got, o = [[] for _ in reqs], 0
        for i, r in enumerate(reqs):
            got[i].append(out[o:o + len(r) - 3])
            o += len(r) - 3
        for k in range(3):
            out = eng.step([StepEntry(s, [r[len(r) - 3 + k]], [0]) for s, r in zip(slots, reqs)])
            for i in range(2):
                got[i].append(out[i:i + 1].clone())
        for i, r in enumerate(reqs):
            want = plain(r)
            assert rel_err(torch.cat(got[i]), want) < TOL[dtype], (round_, i)
            assert rel_err(pl.forward(c, dict(W, **{"model.norm.weight": torch.ones(c["dim"])}), r, rt), want) > 10 * TOL[dtype]
        for s in slots:
            eng.release(s)
    assert eng._prompt_graphs and eng._graphs


def test_a_windowed_group_beside_a_full_one_through_the_engine(tmp_path):
    """A toy architecture whose odd layers see only the last 70 positions: two cache groups with
    storage of their own; the windowed one gives pages back while sequences grow, and the logits
    match plain attention with the same window, for prompts and for decoding (with graphs)."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.config import Architecture, LlamaConfig, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.config.llama_plan import build_llama_plan
    from bitnet_c_amd.engine import LayerPlan
    from bitnet_c_amd.parts import PartSpec
    from bitnet_c_amd.weights import write_model_folder
    from dataclasses import replace
    W = 70

    def build(c):
        plan = build_llama_plan(c)
        layers = []
        for i, lp in enumerate(plan.layers):
            if i % 2 == 1:
                blk = dict(lp.block.params)
                blk["mixer"] = PartSpec.of(blk["mixer"].kind, **dict(dict(blk["mixer"].params), window=W))
                lp = LayerPlan(block=PartSpec.of(lp.block.kind, **blk), names=lp.names)
            layers.append(lp)
        return replace(plan, layers=layers)

    class WinConfig(LlamaConfig):
        def to_dict(self):
            return dict(super().to_dict(), model_type="toy_window", architectures=["ToyWindow"])

    if "toy_window" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_window", LlamaConfig, build))
    from conftest import TINY_A
    for dtype in (torch.float32, torch.bfloat16):
        base = LlamaConfig.from_dict(dict(TINY_A, num_hidden_layers=4, head_dim=64, num_attention_heads=2,
                                          num_key_value_heads=1, hidden_size=64))
        cfg = WinConfig(**{f: getattr(base, f) for f in base.__dataclass_fields__})
        folder = write_model_folder(str(tmp_path / f"win{dtype}"), cfg, 9, dtype)
        eng = Engine.from_folder(folder, dtype=dtype, max_tokens=64 * 12)
        assert len(eng.cache.groups) == 2 and sorted(g.need.window for g in eng.cache.groups) == [0, W]
        c, Wt = pl.read_config(folder), pl.read_weights(folder)
        rt = None if dtype == torch.float32 else torch.bfloat16
        rnd = random.Random(3)
        reqs = [[rnd.randrange(256) for _ in range(n)] for n in (300, 150)]

        def plain(toks):
            x = Wt["model.embed_tokens.weight"][toks]
            pos = torch.arange(len(toks))
            inv = pl.rope_inv_freq(c["head_dim"], c["theta"])
            for l in range(4):
                x = pl.decoder_layer(x, pos, Wt, l, c, inv, rt, W if l % 2 == 1 else None)
            xn = pl._rt(pl.rmsnorm(x, Wt["model.norm.weight"], c["eps"]), rt)
            return pl.linear(xn, Wt["lm_head.weight"])

        slots = [eng.new_sequence() for _ in reqs]
        fed = [len(r) - 40 for r in reqs]
        out = eng.step([StepEntry(s, r[:f], list(range(f))) for s, r, f in zip(slots, reqs, fed)])
        got, o = [[] for _ in reqs], 0
        for i, f in enumerate(fed):
            got[i].append(out[o:o + f])
            o += f
        for k in range(40):
            out = eng.step([StepEntry(s, [r[f + k]], [0]) for s, r, f in zip(slots, reqs, fed)])
            for i in range(2):
                got[i].append(out[i:i + 1])
            eng.cache.check()
        full = [g for g in eng.cache.groups if g.need.window == 0][0]
        win = [g for g in eng.cache.groups if g.need.window == W][0]
        assert sum(p >= 0 for p in full.pages[slots[0]]) == 5 and sum(p >= 0 for p in win.pages[slots[0]]) == 2
        for i, r in enumerate(reqs):
            assert rel_err(torch.cat(got[i]), plain(r)) < TOL[dtype], (dtype, i)
        for s in slots:
            eng.release(s)
        eng.cache.check()
        assert win.pool.n_free == win.pool.n_pages


def _register_routed_toy():
    """A feed-forward with routing (two experts, the better router logit wins) and another position
    encoding (keys and queries at odd positions change their sign), both defined here."""
    from bitnet_c_amd import ops
    from bitnet_c_amd.config import Architecture, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.engine import LayerPlan, ModelPlan, ScheduleEntry
    from bitnet_c_amd.parts import BLOCKS, FEED_FORWARDS, POSITION_ENCODINGS, ParamSpec, Part, PartSpec
    from bitnet_c_amd.parts.position import PositionEncoding

    if "two_experts" not in FEED_FORWARDS:
        @FEED_FORWARDS.register("two_experts")
        class TwoExperts(Part):
            def __init__(self, hidden, intermediate):
                self.hidden = hidden
                spec = PartSpec.of("swiglu", hidden=hidden, intermediate=intermediate)
                self.experts = [FEED_FORWARDS.build(spec), FEED_FORWARDS.build(spec)]     # library parts inside

            def tensors(self):
                t = {"router": ParamSpec((2, self.hidden))}
                for e, part in enumerate(self.experts):
                    t.update({f"e{e}.{k}": v for k, v in part.tensors().items()})
                return t

            def load(self, tensors, device, dtype):
                self.router = (64.0 * tensors["router"].float()).to(device)              # router logits in float32, decisive
                for e, part in enumerate(self.experts):
                    part.load({k[3:]: v for k, v in tensors.items() if k.startswith(f"e{e}.")}, device, dtype)

            def forward(self, h, ctx):
                logits = h.float() @ self.router.t()
                first = (logits[:, 0] >= logits[:, 1])[:, None]
                # a toy: both experts run on every row and the router picks (no shapes that depend on data,
                # so that decode steps can be replayed from graphs)
                return torch.where(first, self.experts[0].forward(h, ctx), self.experts[1].forward(h, ctx))

    if "parity_sign" not in POSITION_ENCODINGS:
        @POSITION_ENCODINGS.register("parity_sign")
        class ParitySign(PositionEncoding):
            def __init__(self, head_dim=0):
                pass

            def fusable(self, hs):
                return False, None                                   # no kernel knows this encoding

            def encode_and_store(self, qkv, ctx, H, Hkv, hs, kv):
                sign = (1 - 2 * (ctx.positions & 1)).to(qkv.dtype)[:, None]
                qkv[:, :(H + Hkv) * hs] *= sign
                ops.rope_kv_write(qkv, ctx.positions, H, Hkv, hs, rope_dims=0,
                                  seq_index=ctx.seq_index if kv.writes else None,
                                  block_table=kv.block_table if kv.writes else None,
                                  k_pages=kv.k_pages if kv.writes else None,
                                  v_pages=kv.v_pages if kv.writes else None)

    @dataclass(frozen=True)
    class RoutedConfig:
        vocab_size: int
        hidden_size: int
        n_layers: int
        model_type: str = "toy_routed"

        @staticmethod
        def from_dict(raw):
            return RoutedConfig(raw["vocab_size"], raw["hidden_size"], raw["n_layers"])

        def to_dict(self):
            return asdict(self)

    def build(c):
        norm = PartSpec.of("rmsnorm", dim=c.hidden_size, eps=1e-5)
        ffn = PartSpec.of("two_experts", hidden=c.hidden_size, intermediate=40)
        att = PartSpec.of("attention", hidden=c.hidden_size, n_heads=3, n_kv_heads=1, head_dim=16, scale=0.25,
                          position=PartSpec.of("parity_sign"))
        layers = []
        for i in range(c.n_layers):
            blk = PartSpec.of("prenorm", mixer=att, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
            names = {local: f"layers.{i}.{local}" for local in BLOCKS.build(blk).tensors()}
            layers.append(LayerPlan(block=blk, names=names))
        return ModelPlan(vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
                         schedule=[ScheduleEntry(i) for i in range(c.n_layers)], final_norm=norm,
                         embedding_name="embed.weight", final_norm_names={"weight": "norm.weight"},
                         lm_head_name="head.weight")

    if "toy_routed" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_routed", RoutedConfig, build))
    return RoutedConfig


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_toy_feed_forward_with_routing_and_another_position_encoding(tmp_path, dtype):
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.weights import write_model_folder
    RoutedConfig = _register_routed_toy()
    cfg = RoutedConfig(vocab_size=50, hidden_size=48, n_layers=2)
    folder = write_model_folder(str(tmp_path / "routed"), cfg, 17, dtype)
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=512)
    assert eng.use_graphs                                            # no state: decode steps are replayed
    from safetensors.torch import load_file
    W = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    rt = None if dtype == torch.float32 else dtype
    r_ = lambda x: x if rt is None else x.to(rt).float()

    def plain(toks):
        x = W["embed.weight"][toks]
        n = len(toks)
        sign = (1 - 2 * (torch.arange(n) % 2)).float()[:, None, None]
        routes = []
        for l in range(2):
            p = f"layers.{l}."
            xb = r_(pl.rmsnorm(x, W[p + "mixer_norm.weight"], 1e-5))
            q = r_(r_(pl.linear(xb, W[p + "mixer.wq"])).view(n, 3, 16) * sign)
            k = r_(r_(pl.linear(xb, W[p + "mixer.wk"])).view(n, 1, 16) * sign)
            v = r_(pl.linear(xb, W[p + "mixer.wv"])).view(n, 1, 16)
            x = x + r_(pl.linear(r_(pl.attention(q, k, v, 0.25).reshape(n, 48)), W[p + "mixer.wo"]))
            xb = r_(pl.rmsnorm(x, W[p + "ffn_norm.weight"], 1e-5))
            logits = xb @ (64.0 * W[p + "ffn.router"]).t()
            routes.append(logits[:, 0] - logits[:, 1])
            ys = [pl.feed_forward(xb, W[p + f"ffn.e{e}.w_gate"], W[p + f"ffn.e{e}.w_up"], W[p + f"ffn.e{e}.w_down"], rt)
                  for e in range(2)]
            x = x + torch.where((logits[:, 0] >= logits[:, 1])[:, None], ys[0], ys[1])
        return pl.linear(r_(pl.rmsnorm(x, W["norm.weight"], 1e-5)), W["head.weight"]), torch.stack(routes)

    rnd = random.Random(20)      # with these requests no router decision is closer than 0.18 (typical margin: 6)
    reqs = [[rnd.randrange(50) for _ in range(n)] for n in (21, 6, 34)]
    slots = [eng.new_sequence() for _ in reqs]
    fed = [len(r) - 5 for r in reqs]
    out = eng.step([StepEntry(s, r[:f], list(range(f))) for s, r, f in zip(slots, reqs, fed)])
    got, o = [[] for _ in reqs], 0
    for i, f in enumerate(fed):
        got[i].append(out[o:o + f])
        o += f
    for k in range(5):
        out = eng.step([StepEntry(s, [r[f + k]], [0]) for s, r, f in zip(slots, reqs, fed)])
        for i in range(3):
            got[i].append(out[i:i + 1])
    used = set()
    for i, r in enumerate(reqs):
        want, margin = plain(r)
        assert float(margin.abs().min()) > 0.05                        # no decision on a knife's edge
        used |= set((margin > 0).flatten().tolist())
        assert rel_err(torch.cat(got[i]), want) < TOL[dtype], i
    assert used == {True, False}                                       # both experts were chosen somewhere


def _register_parallel_toy():
    """Another norm (mean taken out before the root mean square) and another arrangement of a layer's parts (mixer
    and feed-forward read the same normed stream and both add to it), both defined here."""
    from bitnet_c_amd.config import Architecture, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.engine import LayerPlan, ModelPlan, ScheduleEntry
    from bitnet_c_amd.parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, ParamSpec, Part, PartSpec

    if "centered" not in NORMS:
        @NORMS.register("centered")
        class CenteredNorm(Part):
            # neither deferrable nor takes_partial_sums: the stream hands it tensors, with every sum formed

            def __init__(self, dim, eps):
                self.dim, self.eps = dim, eps

            def tensors(self):
                return {"weight": ParamSpec((self.dim,), init="ones")}

            def load(self, tensors, device, dtype):
                self.weight = tensors["weight"].float().to(device)

            def apply(self, x, delta, out_dtype, rows=None):
                if rows is None:
                    if delta is not None:
                        x.add_(delta.float())                       # the norm's kernel is where the sum is formed
                    xs = x
                else:
                    xs = x[rows.long()] if delta is None else x[rows.long()] + delta[rows.long()].float()
                c = xs - xs.mean(dim=1, keepdim=True)
                return (c * torch.rsqrt((c * c).mean(dim=1, keepdim=True) + self.eps) * self.weight).to(out_dtype)

    if "parallel" not in BLOCKS:
        @BLOCKS.register("parallel")
        class ParallelBlock(Part):
            def __init__(self, mixer, ffn, norm):
                self.mixer, self.ffn, self.norm = MIXERS.build(mixer), FEED_FORWARDS.build(ffn), NORMS.build(norm)

            def children(self):
                return {"mixer": self.mixer, "ffn": self.ffn, "norm": self.norm}

            def tensors(self):
                return {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}

            def load(self, tensors, device, dtype):
                for cn, c in self.children().items():
                    c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)

            def cache_need(self):
                return self.mixer.cache_need()

            def forward(self, stream, ctx, kv):
                h = stream.normed(self.norm, ctx.act_dtype)
                a = self.mixer.forward(h, ctx, kv)
                f = self.ffn.forward(h, ctx)
                stream.add(a)
                stream.add(f)

    @dataclass(frozen=True)
    class ParallelConfig:
        vocab_size: int
        hidden_size: int
        n_layers: int
        model_type: str = "toy_parallel"

        @staticmethod
        def from_dict(raw):
            return ParallelConfig(raw["vocab_size"], raw["hidden_size"], raw["n_layers"])

        def to_dict(self):
            return asdict(self)

    def build(c):
        norm = PartSpec.of("centered", dim=c.hidden_size, eps=1e-3)
        ffn = PartSpec.of("swiglu", hidden=c.hidden_size, intermediate=56)
        att = PartSpec.of("attention", hidden=c.hidden_size, n_heads=4, n_kv_heads=2, head_dim=12, scale=0.3,
                          position=PartSpec.of("none"))
        layers = []
        for i in range(c.n_layers):
            blk = PartSpec.of("parallel", mixer=att, ffn=ffn, norm=norm)
            names = {local: f"layers.{i}.{local}" for local in BLOCKS.build(blk).tensors()}
            layers.append(LayerPlan(block=blk, names=names))
        return ModelPlan(vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
                         schedule=[ScheduleEntry(i) for i in range(c.n_layers)], final_norm=norm,
                         embedding_name="embed.weight", final_norm_names={"weight": "norm.weight"},
                         lm_head_name="head.weight")

    if "toy_parallel" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_parallel", ParallelConfig, build))
    return ParallelConfig


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_toy_norm_and_another_arrangement_of_a_layer(tmp_path, dtype):
    """A norm and a block arrangement defined in this file (registered, built from a folder, stepped in a batch of
    unequal prompts and then token by token from graphs) against a plain computation of the same formulas."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.weights import write_model_folder
    ParallelConfig = _register_parallel_toy()
    cfg = ParallelConfig(vocab_size=60, hidden_size=40, n_layers=3)
    folder = write_model_folder(str(tmp_path / "parallel"), cfg, 23, dtype)
    eng = Engine.from_folder(folder, dtype=dtype, max_tokens=512)
    assert eng.use_graphs
    from safetensors.torch import load_file
    W = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    rt = None if dtype == torch.float32 else dtype
    r_ = lambda x: x if rt is None else x.to(rt).float()

    def centered(x, w):
        c = x - x.mean(dim=1, keepdim=True)
        return c * torch.rsqrt((c * c).mean(dim=1, keepdim=True) + 1e-3) * w

    def plain(toks):
        x = W["embed.weight"][toks]
        n = len(toks)
        for l in range(3):
            p = f"layers.{l}."
            xb = r_(centered(x, W[p + "norm.weight"]))
            q = r_(pl.linear(xb, W[p + "mixer.wq"])).view(n, 4, 12)
            k = r_(pl.linear(xb, W[p + "mixer.wk"])).view(n, 2, 12)
            v = r_(pl.linear(xb, W[p + "mixer.wv"])).view(n, 2, 12)
            a = r_(pl.linear(r_(pl.attention(q, k, v, 0.3).reshape(n, 48)), W[p + "mixer.wo"]))
            f = pl.feed_forward(xb, W[p + "ffn.w_gate"], W[p + "ffn.w_up"], W[p + "ffn.w_down"], rt)
            x = x + a + f                                          # both read the same xb, both add
        return pl.linear(r_(centered(x, W["norm.weight"])), W["head.weight"])

    rnd = random.Random(31)
    reqs = [[rnd.randrange(60) for _ in range(n)] for n in (19, 3, 70)]
    slots = [eng.new_sequence() for _ in reqs]
    fed = [len(r) - 2 for r in reqs]
    out = eng.step([StepEntry(s, r[:f], list(range(f))) for s, r, f in zip(slots, reqs, fed)])
    got, o = [[] for _ in reqs], 0
    for i, f in enumerate(fed):
        got[i].append(out[o:o + f])
        o += f
    for k in range(2):
        out = eng.step([StepEntry(s, [r[f + k]], [0]) for s, r, f in zip(slots, reqs, fed)])
        for i in range(3):
            got[i].append(out[i:i + 1])
    assert eng.graphs_built >= 1
    for i, r in enumerate(reqs):
        assert rel_err(torch.cat(got[i]), plain(r)) < TOL[dtype], (dtype, i)
    # the residual order matters: a sequential layer (the feed-forward reading the stream after the mixer's add)
    # gives other logits, so the comparison above does tell the two arrangements apart
    def sequential(toks):
        x = W["embed.weight"][toks]
        n = len(toks)
        for l in range(3):
            p = f"layers.{l}."
            xb = centered(x, W[p + "norm.weight"])
            q, k, v = (pl.linear(xb, W[p + "mixer." + t]).view(n, h, 12) for t, h in (("wq", 4), ("wk", 2), ("wv", 2)))
            x = x + pl.linear(pl.attention(q, k, v, 0.3).reshape(n, 48), W[p + "mixer.wo"])
            xb = centered(x, W[p + "norm.weight"])
            x = x + pl.feed_forward(xb, W[p + "ffn.w_gate"], W[p + "ffn.w_up"], W[p + "ffn.w_down"], None)
        return pl.linear(centered(x, W["norm.weight"]), W["head.weight"])
    apart = rel_err(sequential(reqs[0]), plain(reqs[0]))
    assert apart > 0.03 and apart > 4 * rel_err(torch.cat(got[0]), plain(reqs[0])), apart


# ---------------------------------------------------------------------------------------
# the layout of a cache page is the mixer's to say (KVNeed): values wider than keys, and the
# library's own attention over values that lie like the keys in bfloat16
# ---------------------------------------------------------------------------------------

def test_a_toy_mixer_whose_values_are_wider_than_its_keys(tmp_path):
    """One-head attention with keys of 8 and values of 24 columns, written in the test with torch over the pages
    that the cache gives it: the cache allocates what the need says ([.., PAGE, 24] beside [.., PAGE, 8]) and nothing
    in the library is edited for it.  Prompts of unequal lengths, tokens one by one, a slot that is used again."""
    from bitnet_c_amd import Engine, StepEntry
    from bitnet_c_amd.cache import PAGE
    from bitnet_c_amd.config import Architecture, register_architecture
    from bitnet_c_amd.config.base import _ARCHITECTURES
    from bitnet_c_amd.engine import LayerPlan, ModelPlan, ScheduleEntry
    from bitnet_c_amd.parts import BLOCKS, MIXERS, CacheNeed, KVNeed, ParamSpec, Part, PartSpec
    from bitnet_c_amd.weights import write_model_folder
    DK, DV = 8, 24

    if "wide_values" not in MIXERS:
        @MIXERS.register("wide_values")
        class WideValues(Part):
            def __init__(self, hidden):
                self.hidden = hidden

            def tensors(self):
                return {"wq": ParamSpec((DK, self.hidden)), "wk": ParamSpec((DK, self.hidden)),
                        "wv": ParamSpec((DV, self.hidden)), "wo": ParamSpec((self.hidden, DV))}

            def load(self, tensors, device, dtype):
                self.w = {k: v.float().to(device) for k, v in tensors.items()}

            def cache_need(self):
                return CacheNeed(kv=KVNeed(1, DK, v_head_dim=DV, v_layout="rows"))

            def forward(self, h, ctx, kv):
                assert kv.v_transposed is False and kv.v_pages.shape[1:] == (1, PAGE, DV)
                x = h.float()
                q, k, v = x @ self.w["wq"].t(), x @ self.w["wk"].t(), x @ self.w["wv"].t()
                pos, seq = ctx.positions.long(), ctx.seq_index.long()
                page = kv.block_table.long()[seq, pos // PAGE]
                kv.k_pages[page, 0, pos % PAGE] = k.to(kv.k_pages.dtype)
                kv.v_pages[page, 0, pos % PAGE] = v.to(kv.v_pages.dtype)
                out = torch.empty((h.shape[0], DV), dtype=torch.float32, device=h.device)
                for b, ((r0, n), p0) in enumerate(zip(ctx.row_ranges(), ctx.pos0)):
                    L = p0 + n
                    pages = kv.block_table.long()[b, :(L + PAGE - 1) // PAGE]
                    K = kv.k_pages[pages, 0].reshape(-1, DK)[:L].float()
                    V = kv.v_pages[pages, 0].reshape(-1, DV)[:L].float()
                    sc = (q[r0:r0 + n] @ K.t()) * DK ** -0.5
                    keys = torch.arange(L, device=h.device)[None, :]
                    sc = sc.masked_fill(keys > (p0 + torch.arange(n, device=h.device))[:, None], float("-inf"))
                    out[r0:r0 + n] = torch.softmax(sc, dim=-1) @ V
                return (out @ self.w["wo"].t()).to(h.dtype)

    @dataclass(frozen=True)
    class WideConfig:
        vocab_size: int
        hidden_size: int
        model_type: str = "toy_wide_values"

        @staticmethod
        def from_dict(raw):
            return WideConfig(raw["vocab_size"], raw["hidden_size"])

        def to_dict(self):
            return asdict(self)

    def build(c):
        norm = PartSpec.of("rmsnorm", dim=c.hidden_size, eps=1e-5)
        ffn = PartSpec.of("swiglu", hidden=c.hidden_size, intermediate=2 * c.hidden_size)
        att = PartSpec.of("attention", hidden=c.hidden_size, n_heads=2, n_kv_heads=1, head_dim=DK,
                          scale=DK ** -0.5, position=PartSpec.of("rope", head_dim=DK, theta=100.0))
        layers = []
        for i, mixer in enumerate((PartSpec.of("wide_values", hidden=c.hidden_size), att)):
            blk = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
            layers.append(LayerPlan(block=blk, names={n: f"layers.{i}.{n}" for n in BLOCKS.build(blk).tensors()}))
        return ModelPlan(vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
                         schedule=[ScheduleEntry(0), ScheduleEntry(1)], final_norm=norm, embedding_name="embed.weight",
                         final_norm_names={"weight": "norm.weight"}, lm_head_name="head.weight")

    if "toy_wide_values" not in _ARCHITECTURES:
        register_architecture(Architecture("toy_wide_values", WideConfig, build))
    folder = write_model_folder(str(tmp_path / "wide"), WideConfig(vocab_size=50, hidden_size=32), 21, torch.float32)
    eng = Engine.from_folder(folder, dtype=torch.float32, max_tokens=512, use_graphs=False)
    # two groups: the toy mixer's pages (values of 24 columns) and the attention's (keys and values of 8)
    shapes = sorted((tuple(g.k.shape[2:]), tuple(g.v.shape[2:])) for g in eng.cache.groups)
    assert shapes == [((1, PAGE, DK), (1, PAGE, DK)), ((1, PAGE, DK), (1, PAGE, DV))]

    from safetensors.torch import load_file
    W = load_file(os.path.join(folder, "model.safetensors"))

    def plain(toks):
        x = W["embed.weight"][toks]
        n = len(toks)
        pos = torch.arange(n)
        for l in range(2):
            p = f"layers.{l}."
            xb = pl.rmsnorm(x, W[p + "mixer_norm.weight"], 1e-5)
            if l == 0:
                q, k, v = (pl.linear(xb, W[p + "mixer.w" + c]) for c in "qkv")
                sc = (q @ k.t()) * DK ** -0.5
                sc = sc.masked_fill(torch.arange(n)[None, :] > torch.arange(n)[:, None], float("-inf"))
                o = pl.softmax(sc) @ v                                  # [n, DV]: one head, values of their own width
            else:
                inv = pl.rope_inv_freq(DK, 100.0)
                q = pl.apply_rope(pl.linear(xb, W[p + "mixer.wq"]).view(n, 2, DK), pos, inv)
                k = pl.apply_rope(pl.linear(xb, W[p + "mixer.wk"]).view(n, 1, DK), pos, inv)
                o = pl.attention(q, k, pl.linear(xb, W[p + "mixer.wv"]).view(n, 1, DK), DK ** -0.5).reshape(n, 2 * DK)
            x = x + pl.linear(o, W[p + "mixer.wo"])
            xb = pl.rmsnorm(x, W[p + "ffn_norm.weight"], 1e-5)
            x = x + pl.feed_forward(xb, W[p + "ffn.w_gate"], W[p + "ffn.w_up"], W[p + "ffn.w_down"])
        return pl.linear(pl.rmsnorm(x, W["norm.weight"], 1e-5), W["head.weight"])

    rnd = random.Random(22)
    reqs = [[rnd.randrange(50) for _ in range(n)] for n in (70, 9, 131)]
    for round_ in range(2):                                   # the second round runs in slots that were used before
        slots = [eng.new_sequence() for _ in reqs]
        fed = [len(r) - 3 for r in reqs]
        out = eng.step([StepEntry(s, r[:f], list(range(f))) for s, r, f in zip(slots, reqs, fed)])
        got, o = [[] for _ in reqs], 0
        for i, f in enumerate(fed):
            got[i].append(out[o:o + f])
            o += f
        for k in range(3):
            out = eng.step([StepEntry(s, [r[f + k]], [0]) for s, r, f in zip(slots, reqs, fed)])
            for i in range(3):
                got[i].append(out[i:i + 1])
        for i, r in enumerate(reqs):
            assert rel_err(torch.cat(got[i]), plain(r)) < TOL[torch.float32], (round_, i)
        for s in slots:
            eng.release(s)
        eng.cache.check()
        reqs = reqs[::-1]


@pytest.mark.parametrize("dtype,layout", [(torch.bfloat16, "rows"), (torch.float32, "transposed"), (torch.bfloat16, "transposed")])
@pytest.mark.parametrize("hs", [64, 24])
def test_the_attention_part_over_the_layout_that_is_not_its_kernels_own(dtype, layout, hs):
    """An attention whose need names another layout than its kernels would pick (bfloat16 values lying like the keys,
    float32 values turned, bfloat16 values turned at a head size where the kernels would keep blocked pages): the cache
    write and the vector kernel take either, the matrix-core kernels are not used, and the result is the plain
    attention's."""
    from bitnet_c_amd.cache import PAGE, PagedCache
    from bitnet_c_amd.parts import MIXERS, CacheNeed, KVNeed, PartSpec
    from bitnet_c_amd.parts.attention import Attention

    class OtherLayout(Attention):
        def cache_need(self):
            return CacheNeed(kv=KVNeed(self.Hkv, self.hs, self.window, v_layout=layout))

    H, Hkv, hidden, scale = 4, 2, 48, 0.2
    att = OtherLayout(hidden, H, Hkv, hs, scale, PartSpec.of("rope", head_dim=hs, theta=5000.0))
    t = {k: _rand(v.shape, 40 + i, 0.15).to(dtype) for i, (k, v) in enumerate(att.tensors().items())}
    att.load(t, DEV, dtype)
    cache = PagedCache([att.cache_need()], [None], 64 * 8, dtype=dtype, device=DEV)
    assert cache.groups[0].v.shape[2:] == ((Hkv, hs, PAGE) if layout == "transposed" else (Hkv, PAGE, hs))
    lens = [70, 5, 130]
    hs_in = [_rand((n, hidden), 50 + i).to(dtype) for i, n in enumerate(lens)]
    slots = [cache.alloc_slot() for _ in lens]
    got = [[] for _ in lens]
    fed = [n - 3 for n in lens]
    ctx, tables, max_len = _ctx(cache, slots, fed, dtype)
    out = att.forward(torch.cat([h[:f] for h, f in zip(hs_in, fed)]).to(DEV), ctx, cache.view(0, tables, max_len))
    cache.commit(slots, fed)
    o = 0
    for i, f in enumerate(fed):
        got[i].append(out[o:o + f])
        o += f
    for step in range(3):
        ctx, tables, max_len = _ctx(cache, slots, [1] * 3, dtype)
        out = att.forward(torch.cat([h[f + step:f + step + 1] for h, f in zip(hs_in, fed)]).to(DEV), ctx,
                          cache.view(0, tables, max_len))
        cache.commit(slots, [1] * 3)
        for i in range(3):
            got[i].append(out[i:i + 1])
    rt = None if dtype == torch.float32 else dtype
    r = (lambda x: x) if rt is None else (lambda x: x.to(rt).float())
    inv = pl.rope_inv_freq(hs, 5000.0)
    for i, n in enumerate(lens):
        h = hs_in[i].float()
        pos = torch.arange(n)

        def whole(r):
            q = r(pl.apply_rope(r(pl.linear(h, t["wq"].float())).view(n, H, hs), pos, inv))
            k = r(pl.apply_rope(r(pl.linear(h, t["wk"].float())).view(n, Hkv, hs), pos, inv))
            v = r(pl.linear(h, t["wv"].float())).view(n, Hkv, hs)
            return r(pl.linear(r(pl.attention(q, k, v, scale).reshape(n, H * hs)), t["wo"].float()))
        assert part_close(torch.cat(got[i]).float(), whole(r), dtype, whole(lambda x: x)), i
