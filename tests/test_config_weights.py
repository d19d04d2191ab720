"""Configuration, registry, weight files and their errors (no GPU)."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B


def test_llama_config_defaults_and_derived_sizes():
    from bitnet_c_amd.config import LlamaConfig
    c = LlamaConfig.from_dict(dict(vocab_size=100, hidden_size=64, intermediate_size=96, num_hidden_layers=2,
                                   num_attention_heads=4, max_position_embeddings=32))
    # defaults of the reference's loader: kv heads = heads, theta 10000, eps 1e-5, head = hidden/heads
    assert (c.num_key_value_heads, c.rope_theta, c.rms_norm_eps, c.head_dim) == (4, 10000.0, 1e-5, 16)
    assert c.tie_word_embeddings is False and c.rope_scaling is None
    b = LlamaConfig.from_dict(TINY_B)
    assert (b.q_dim, b.kv_dim, b.head_dim) == (120, 120, 24) and b.rope_scaling.factor == 8.0
    assert LlamaConfig.from_dict(b.to_dict()) == b


@pytest.mark.parametrize("patch,word", [
    (dict(num_key_value_heads=3), "multiple"), (dict(hidden_size=0), "positive"), (dict(vocab_size=-1), "positive"),
    (dict(hidden_act="gelu"), "hidden_act"), (dict(head_dim=15), "even"), (dict(head_dim=258), "attention kernels take"),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), "yarn"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=8.0)), "low_freq_factor"),
    (dict(num_hidden_layers=None), "num_hidden_layers"), (dict(hidden_size=66, num_attention_heads=4), "head_dim"),
])
def test_config_errors_name_the_key(patch, word):
    from bitnet_c_amd.config import ConfigError, LlamaConfig
    raw = dict(TINY_A)
    raw.update(patch)
    raw = {k: v for k, v in raw.items() if v is not None}
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(raw)
    assert word in str(e.value)


def test_registry_chooses_by_config_json_and_has_no_default(tmp_path):
    from bitnet_c_amd.config import (Architecture, ConfigError, LlamaConfig, architecture_for, load_config,
                                     register_architecture)
    assert architecture_for(dict(model_type="llama")).name == "llama"
    assert architecture_for(dict(architectures=["LlamaForCausalLM"])).name == "llama"
    with pytest.raises(ConfigError) as e:
        architecture_for(dict(model_type="mamba"))
    assert "mamba" in str(e.value) and "llama" in str(e.value)
    with pytest.raises(ValueError):
        register_architecture(Architecture("llama", LlamaConfig, lambda c: None))
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "llama" and cfg.hidden_size == 64
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "nothing"))


def test_plan_is_data_and_names_every_tensor():
    from bitnet_c_amd.config import LlamaConfig, architecture_for
    for raw, n_tensors, n_params in ((TINY_A, 2 * 9 + 3, None), (TINY_B, 3 * 9 + 2, None)):
        c = LlamaConfig.from_dict(raw)
        plan = architecture_for(raw).build_plan(c)
        exp = plan.expected_tensors()
        assert len(exp) == n_tensors
        assert [e.layer for e in plan.schedule] == list(range(c.num_hidden_layers))
        assert exp["model.layers.0.self_attn.k_proj.weight"].shape == (c.kv_dim, c.hidden_size)
        assert exp["model.layers.1.mlp.down_proj.weight"].shape == (c.hidden_size, c.intermediate_size)
        assert exp["model.norm.weight"].init == "ones"
        assert ("lm_head.weight" in exp) == (not c.tie_word_embeddings)
    # the constants of the parts come from the configuration alone
    mixer = dict(plan.layers[0].block.params)["mixer"]
    assert dict(mixer.params)["scale"] == pytest.approx(24 ** -0.5)
    assert dict(dict(mixer.params)["position"].params)["theta"] == 500000.0


def test_random_weights_folder_round_trip(tmp_path):
    from safetensors.torch import load_file
    from bitnet_c_amd.config import LlamaConfig, load_config
    from bitnet_c_amd.weights import load_tensors, write_model_folder
    c = LlamaConfig.from_dict(TINY_A)
    d1, d2, d3 = (str(tmp_path / n) for n in "abc")
    write_model_folder(d1, c, 0, torch.bfloat16)
    write_model_folder(d2, c, 0, torch.bfloat16)
    write_model_folder(d3, c, 1, torch.float32)
    arch, cfg = load_config(d1)
    assert cfg == c
    t1 = load_tensors(d1, arch.build_plan(cfg).expected_tensors())
    t2 = load_tensors(d2, arch.build_plan(cfg).expected_tensors())
    t3 = load_tensors(d3, arch.build_plan(cfg).expected_tensors())
    lib = load_file(os.path.join(d1, "model.safetensors"))          # an independent reader sees the same file
    assert set(lib) == set(t1) and all(torch.equal(lib[k], t1[k]) for k in t1)
    for k in t1:
        assert torch.equal(t1[k], t2[k])                              # same seed, same values
    w = t1["model.layers.1.mlp.up_proj.weight"]
    assert w.dtype == torch.bfloat16 and abs(float(w.float().std()) - 0.02) < 0.002
    assert t1["model.norm.weight"].dtype == torch.float32 and bool((t1["model.norm.weight"] == 1).all())
    assert t3["lm_head.weight"].dtype == torch.float32               # a tensor stored in 32 bits stays so
    assert not torch.equal(t3["lm_head.weight"], t1["lm_head.weight"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    from safetensors.torch import load_file, save_file
    from bitnet_c_amd.config import LlamaConfig, load_config
    from bitnet_c_amd.weights import WeightError, load_tensors, write_model_folder
    d = str(tmp_path / "m")
    write_model_folder(d, LlamaConfig.from_dict(TINY_A), 0, torch.float32)
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["model.layers.0.mlp.up_proj.weight"], t["model.norm.weight"]
    t["model.layers.7.extra.weight"] = torch.zeros(3)
    t["lm_head.weight"] = torch.zeros(256, 63)
    t["model.layers.1.self_attn.k_proj.weight"] = torch.zeros(64, 32)
    save_file(t, path)
    arch, cfg = load_config(d)
    with pytest.raises(WeightError) as e:
        load_tensors(d, arch.build_plan(cfg).expected_tensors())
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert [w[0] for w in err.wrong_shape] == ["lm_head.weight", "model.layers.1.self_attn.k_proj.weight"]
    msg = str(err)
    for word in ("missing (2)", "unexpected (1)", "wrong shape (2)", "[256, 63]", "[256, 64]"):
        assert word in msg
    with pytest.raises(WeightError):
        load_tensors(str(tmp_path / "empty"), {})


def test_host_dtypes(tmp_path):
    from bitnet_c_amd.weights import TensorSpec, load_tensors, write_file
    d = str(tmp_path)
    write_file(os.path.join(d, "model.safetensors"), {
        "a": torch.ones(2, 2, dtype=torch.float16), "b": torch.ones(2, dtype=torch.bfloat16),
        "c": torch.arange(3, dtype=torch.int64), "d": torch.ones(1, dtype=torch.float32)})
    t = load_tensors(d, {"a": TensorSpec("a", (2, 2)), "b": TensorSpec("b", (2,)), "c": TensorSpec("c", (3,)),
                         "d": TensorSpec("d", (1,)), "e": TensorSpec("e", (9,), optional=True)})
    assert [t[k].dtype for k in "abcd"] == [torch.float32, torch.bfloat16, torch.int32, torch.float32]
    assert "e" not in t


def test_damaged_files_are_refused(tmp_path):
    from bitnet_c_amd.weights import SafetensorsError, SafetensorsFile, write_file
    p = str(tmp_path / "x.safetensors")
    write_file(p, {"w": torch.arange(12, dtype=torch.float32).view(3, 4)})
    with SafetensorsFile(p) as f:
        assert torch.equal(f.read("w"), torch.arange(12, dtype=torch.float32).view(3, 4))
    raw = open(p, "rb").read()
    for name, blob in (("short", raw[:-8]),                                   # data cut off
                       ("hdr", struct.pack("<Q", 10 ** 9) + raw[8:]),         # header length past the end
                       ("tiny", raw[:4]),
                       ("json", raw[:8] + b"{" * (len(raw) - 8))):
        q = str(tmp_path / f"{name}.safetensors")
        open(q, "wb").write(blob)
        with pytest.raises(SafetensorsError):
            SafetensorsFile(q)
    (hlen,) = struct.unpack("<Q", raw[:8])
    hdr = json.loads(raw[8:8 + hlen])
    hdr["w"]["shape"] = [3, 5]                                                # shape that does not fit the bytes
    blob = json.dumps(hdr).encode()
    open(p, "wb").write(struct.pack("<Q", len(blob)) + blob + raw[8 + hlen:])
    with pytest.raises(SafetensorsError):
        SafetensorsFile(p)


def test_sharded_folder(tmp_path):
    from bitnet_c_amd.weights import TensorSpec, load_tensors, write_file
    d = str(tmp_path)
    write_file(os.path.join(d, "model-00001-of-00002.safetensors"), {"a": torch.ones(2)})
    write_file(os.path.join(d, "model-00002-of-00002.safetensors"), {"b": torch.zeros(3)})
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": {"a": "model-00001-of-00002.safetensors", "b": "model-00002-of-00002.safetensors"}}, f)
    t = load_tensors(d, {"a": TensorSpec("a", (2,)), "b": TensorSpec("b", (3,))})
    assert float(t["a"].sum()) == 2.0 and t["b"].shape == (3,)


def test_a_model_is_read_tensor_by_tensor_without_holding_it(tmp_path):
    """open_tensors gives views of the mapped files and release() lets their pages go: walking a sharded folder of
    24 tensors of 4 MB the way a model is uploaded (take a layer's tensors, use them, release them) raises the
    process's peak memory by less than two tensors, where reading the folder whole (load_tensors) raises it by the
    folder's size.  Measured in a fresh process with resource.getrusage, whose peak only ever grows."""
    import subprocess
    import sys
    from bitnet_c_amd.weights import write_file
    d = str(tmp_path)
    names, wm = [], {}
    for shard in range(3):
        fn = f"model-0000{shard + 1}-of-00003.safetensors"
        part = {f"t{shard}_{i}": torch.full((1024, 1024), float(8 * shard + i), dtype=torch.float32) for i in range(8)}
        write_file(os.path.join(d, fn), part)
        names += list(part)
        wm.update({n: fn for n in part})
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    script = f"""
import resource, sys, torch
sys.path.insert(0, {os.path.dirname(os.path.dirname(os.path.abspath(__file__)))!r})
from bitnet_c_amd.weights import TensorSpec, load_tensors, open_tensors
names = {names!r}
exp = {{n: TensorSpec(n, (1024, 1024)) for n in names}}
peak = lambda: resource.getrusage(resource.RUSAGE_SELF).ru_maxrss * 1024
torch.zeros(1 << 20).sum()                       # whatever the first use of torch brings in
p0 = peak()
total = 0.0
with open_tensors({d!r}, exp) as src:
    for i in range(0, len(names), 2):            # two tensors at a time, as a layer's
        pair = [src[n] for n in names[i:i + 2]]
        total += sum(float(t.sum()) for t in pair)
        del pair
        src.release(names[i:i + 2])
p1 = peak()
whole = load_tensors({d!r}, exp)
p2 = peak()
print(total, p1 - p0, p2 - p1)
"""
    out = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-2000:]
    total, streamed, held = (float(v) for v in out.stdout.split())
    assert total == sum(range(24)) * 1024 * 1024
    one = 4 << 20
    assert streamed <= 2 * 2 * one + (4 << 20), streamed      # two tensors in use at a time, and some slack
    assert held >= 16 * one, held                              # the measure can tell: the whole folder is 24 tensors


def test_views_of_the_map_are_the_file_s_bytes(tmp_path):
    from bitnet_c_amd.weights import SafetensorsFile, TensorSpec, open_tensors, write_file
    d = str(tmp_path)
    a = torch.arange(5, dtype=torch.bfloat16)                  # 10 bytes: what follows it is not aligned for 4-byte types
    b = torch.arange(12, dtype=torch.float32).view(3, 4)
    h = torch.arange(6, dtype=torch.float16).view(2, 3)
    write_file(os.path.join(d, "model.safetensors"), {"a": a, "b": b, "h": h})
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        assert torch.equal(f.view("a"), a) and torch.equal(f.view("b"), b)
    with open_tensors(d, {"a": TensorSpec("a", (5,)), "b": TensorSpec("b", (3, 4)), "h": TensorSpec("h", (2, 3))}) as src:
        assert set(src) == {"a", "b", "h"} and len(src) == 3 and "zz" not in src
        assert torch.equal(src["b"], b) and src["h"].dtype == torch.float32 and torch.equal(src["h"], h.float())
        kept = src["a"]
        src.release(["a", "b", "zz"])                          # advice only; the bytes are read again when asked for
        assert torch.equal(src["a"], a)
    assert torch.equal(kept, a)                                # a view that outlives the source keeps the map alive


def test_rope_frequencies_match_the_plain_implementation():
    import plain_llama as pl
    from bitnet_c_amd.parts.position import rope_frequencies
    sc = TINY_B["rope_scaling"]
    assert torch.equal(rope_frequencies(24, 500000.0, sc), pl.rope_inv_freq(24, 500000.0, sc))
    assert torch.equal(rope_frequencies(16, 10000.0), pl.rope_inv_freq(16, 10000.0))
    big = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
               original_max_position_embeddings=8192)
    assert torch.equal(rope_frequencies(128, 500000.0, big), pl.rope_inv_freq(128, 500000.0, big))


def test_ops_fail_loudly_without_a_gpu():
    from bitnet_c_amd import ops
    if torch.cuda.is_available():
        pytest.skip("a GPU is here")
    with pytest.raises(ops.KernelError):
        ops.linear(torch.zeros(2, 8), torch.zeros(4, 8))
    with pytest.raises(ops.KernelError):
        ops.argmax(torch.zeros(1, 4))
