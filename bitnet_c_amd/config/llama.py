"""Configuration of the Llama-style dense decoder, read from its config.json keys.

Fields and defaults follow the reference's loader (src/model.c:238-310): kv heads
default to heads (:252-254), rope_theta to 10000 (:259-260), the norm's eps to 1e-5
(:264-266), head size to hidden/heads unless given (:285-287); heads must be a multiple
of kv heads (:299-302).  The reference's SIMD-only checks (hidden % 128, head % 16;
:303-310) are properties of its kernels, not of the architecture and are not taken over; the one limit of the kernels here that a
config.json can break (a head size above BN_MAX_HEAD_DIM of csrc/common.h) is reported with the other errors.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass
from typing import Optional

from ..csrc.build import header_constant
from .base import ConfigError, _positive_int


# config.json's names of the gate activation -> the feed-forward part's.  Which of them a config.json may name is the
# architecture's decision (LlamaConfig.GATE_ACTIVATIONS): the reference's registry fixes SiLU for this one
# (src/model_arch.c:807-810); the other kinds exist for architectures that declare them.
HIDDEN_ACTS = {"silu": "silu", "gelu_pytorch_tanh": "gelu_tanh", "gelu_tanh": "gelu_tanh", "relu2": "relu2"}
MAX_HEAD_DIM = header_constant("BN_MAX_HEAD_DIM")      # the kernels' limit, read from their header (no kernel is loaded for it)


@dataclass(frozen=True)
class RopeScaling:
    rope_type: str                          # "llama3" (or "default": none)
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @staticmethod
    def from_dict(raw: Optional[dict]) -> Optional["RopeScaling"]:
        if raw is None:
            return None
        if not isinstance(raw, dict):
            raise ConfigError(f"config.json: rope_scaling must be an object, got {raw!r}")
        kind = raw.get("rope_type", raw.get("type"))
        if kind in (None, "default"):
            return None
        if kind != "llama3":
            raise ConfigError(f"config.json: rope_scaling.rope_type {kind!r} is not supported "
                              f"(supported: 'llama3', 'default')")
        try:
            rs = RopeScaling(
                rope_type="llama3",
                factor=float(raw["factor"]),
                low_freq_factor=float(raw["low_freq_factor"]),
                high_freq_factor=float(raw["high_freq_factor"]),
                original_max_position_embeddings=int(raw["original_max_position_embeddings"]),
            )
        except KeyError as e:
            raise ConfigError(f"config.json: rope_scaling (llama3) lacks key {e.args[0]!r}") from None
        if rs.factor <= 0 or rs.original_max_position_embeddings <= 0:
            raise ConfigError("config.json: rope_scaling factor and original_max_position_embeddings "
                              "must be positive")
        if rs.high_freq_factor <= rs.low_freq_factor:
            raise ConfigError("config.json: rope_scaling high_freq_factor must exceed low_freq_factor")
        return rs


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-5
    tie_word_embeddings: bool = False
    rope_scaling: Optional[RopeScaling] = None
    hidden_act: str = "silu"
    attention_bias: bool = False
    mlp_bias: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[object] = None    # an int or a list of ints
    model_type: str = "llama"

    # the values of hidden_act that this architecture takes; a configuration class of another architecture of the
    # family (a subclass) widens it
    GATE_ACTIVATIONS = ("silu",)

    @classmethod
    def from_dict(cls, raw: dict) -> "LlamaConfig":
        hidden = _positive_int(raw, "hidden_size")
        heads = _positive_int(raw, "num_attention_heads")
        kv_heads = raw.get("num_key_value_heads")
        kv_heads = heads if kv_heads in (None, 0) else _positive_int(raw, "num_key_value_heads")
        head_dim = raw.get("head_dim")
        if head_dim in (None, 0):
            if hidden % heads:
                raise ConfigError(f"config.json: hidden_size {hidden} is not a multiple of "
                                  f"num_attention_heads {heads} and no head_dim is given")
            head_dim = hidden // heads
        else:
            head_dim = _positive_int(raw, "head_dim")
        if heads % kv_heads:
            raise ConfigError(f"config.json: num_attention_heads {heads} is not a multiple of "
                              f"num_key_value_heads {kv_heads}")
        if head_dim % 2:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even (rotation pairs)")
        if head_dim > MAX_HEAD_DIM:
            raise ConfigError(f"config.json: head_dim {head_dim} is more than the attention kernels take "
                              f"(every even head size up to {MAX_HEAD_DIM})")
        act = raw.get("hidden_act", "silu")
        if act not in HIDDEN_ACTS or act not in cls.GATE_ACTIVATIONS:
            raise ConfigError(f"config.json: hidden_act {act!r} is not supported by this architecture "
                              f"(supported: {sorted(cls.GATE_ACTIVATIONS)})")
        theta = raw.get("rope_theta")
        theta = 10000.0 if theta in (None, 0) else float(theta)
        eps = raw.get("rms_norm_eps")
        eps = 1e-5 if eps in (None, 0) else float(eps)
        if not (theta > 0 and math.isfinite(theta)) or not (eps > 0 and math.isfinite(eps)):
            raise ConfigError("config.json: rope_theta and rms_norm_eps must be positive and finite")
        return cls(
            vocab_size=_positive_int(raw, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_positive_int(raw, "intermediate_size"),
            num_hidden_layers=_positive_int(raw, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            max_position_embeddings=_positive_int(raw, "max_position_embeddings"),
            rope_theta=theta,
            rms_norm_eps=eps,
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            rope_scaling=RopeScaling.from_dict(raw.get("rope_scaling")),
            hidden_act=act,
            attention_bias=bool(raw.get("attention_bias", False)),
            mlp_bias=bool(raw.get("mlp_bias", False)),
            bos_token_id=raw.get("bos_token_id"),
            eos_token_id=raw.get("eos_token_id"),
            model_type=str(raw.get("model_type", "llama")),
        )

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = ["LlamaForCausalLM"]
        if self.rope_scaling is None:
            d["rope_scaling"] = None
        return d

    # derived sizes (the reference's head_size / kv_dim / kv_mul, include/model_config.h:30-36)
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def stop_ids(self):
        e = self.eos_token_id
        if e is None:
            return ()
        return tuple(e) if isinstance(e, (list, tuple)) else (int(e),)
