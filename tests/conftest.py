import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations of the architecture that differ in every size and option.
TINY_A = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=256, hidden_size=64, intermediate_size=172, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, max_position_embeddings=512,
    rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY_B = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=389, hidden_size=120, intermediate_size=328, num_hidden_layers=3,
    num_attention_heads=5, num_key_value_heads=5, head_dim=24, max_position_embeddings=1024,
    rope_theta=500000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64))
# a third one: head_dim that is not hidden/heads, three query heads per kv head, biases
TINY_C = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=131, hidden_size=72, intermediate_size=100, num_hidden_layers=1,
    num_attention_heads=6, num_key_value_heads=2, head_dim=32, max_position_embeddings=2048,
    rope_theta=20000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
# a fourth one with the optional bias tensors on every projection, and head size 64 (matrix-core attention)
TINY_D = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=200, hidden_size=128, intermediate_size=264, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, head_dim=64, max_position_embeddings=1024,
    rope_theta=100000.0, rms_norm_eps=1e-5, tie_word_embeddings=False, attention_bias=True, mlp_bias=True)
# a fifth one with the head size and grouping of the benchmark shape (128, four query heads per kv head)
TINY_E = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=300, hidden_size=192, intermediate_size=520, num_hidden_layers=2,
    num_attention_heads=8, num_key_value_heads=2, head_dim=128, max_position_embeddings=2048,
    rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=True)
# one layer with eight kv heads: a batch of 40 is more attention workgroups than the chip has CUs
TINY_F = dict(
    model_type="llama", architectures=["LlamaForCausalLM"],
    vocab_size=150, hidden_size=80, intermediate_size=136, num_hidden_layers=1,
    num_attention_heads=16, num_key_value_heads=8, head_dim=64, max_position_embeddings=512,
    rope_theta=10000.0, rms_norm_eps=1e-5, tie_word_embeddings=False)
TINY = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}
SEEDS = {"A": 0, "B": 2, "C": 5, "D": 7, "E": 11, "F": 13}


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """name, dtype -> a model folder with random weights, made on demand in a temporary folder."""
    from bitnet_c_amd.config import LlamaConfig
    from bitnet_c_amd.weights import write_model_folder
    made = {}

    def get(name: str, dtype=torch.float32) -> str:
        key = (name, dtype)
        if key not in made:
            d = tmp_path_factory.mktemp(f"tiny{name}_{str(dtype).split('.')[-1]}")
            write_model_folder(str(d), LlamaConfig.from_dict(TINY[name]), SEEDS[name], dtype)
            made[key] = str(d)
        return made[key]
    return get


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest absolute difference over the root mean square of the reference."""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.numel() == 0:
        return 0.0
    rms = float(ref.pow(2).mean().sqrt())
    return float((got - ref).abs().max()) / max(rms, 1e-30)


# Bounds, fixed before the first run: float32 differs from the plain implementation by
# summation order only; bfloat16 by the rounding of activations to 8 bits of mantissa at
# every part's boundary (the plain implementation rounds at the same places).
TOL = {torch.float32: 1e-4, torch.bfloat16: 3e-2}


def part_close(got: torch.Tensor, want: torch.Tensor, dtype, exact: torch.Tensor = None) -> bool:
    """For a part whose output is stored in `dtype`; `want` is the plain implementation with its
    tensors rounded to `dtype` where a part stores them.
    float32: as for logits.
    bfloat16, short paths (one or two roundings): an element may differ from `want` by one unit in
    the last place (2^-7 of its size) plus 1e-2 of the rms for the inner roundings.
    bfloat16 with `exact` (the plain implementation without any rounding): the two sides round at
    different places (a fused kernel keeps float32 where the plain one stores bfloat16), so they are
    compared by their distance to the exact result: the part is at most twice as far from it as the
    rounded plain implementation is, plus one rounding of the largest element."""
    if dtype == torch.float32:
        return rel_err(got, want) < TOL[dtype]
    if exact is not None:
        e_got, e_want = rel_err(got, exact), rel_err(want, exact)
        ok = e_got <= 2.0 * e_want + 2.0 ** -8
        if not ok:
            print(f"part_close: part is {e_got} from the exact result, the rounded plain one {e_want}")
        return ok
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    rms = float(want.pow(2).mean().sqrt())
    excess = (got - want).abs() - (want.abs() * 2.0 ** -7 + 1e-2 * rms)
    if bool((excess > 0).any()):
        i = int(excess.argmax())
        print(f"part_close: worst element {i}: got {float(got.flatten()[i])} want {float(want.flatten()[i])} "
              f"rms {rms} excess {float(excess.max())}")
        return False
    return True
