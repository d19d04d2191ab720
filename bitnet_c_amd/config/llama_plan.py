"""The Llama-style dense decoder as a plan: per layer a pre-norm block of RMSNorm,
grouped-query attention with rotary encoding, RMSNorm and a SwiGLU feed-forward; every
layer once, in order; final RMSNorm; output matrix or the tied embedding.

Tensor names of the model folder against the roles the reference loads for this
architecture (src/model_arch.c:45-97, src/model.c:436-913):
  token_embd -> model.embed_tokens.weight        output_norm -> model.norm.weight
  output -> lm_head.weight (absent when tied, src/model.c:453-493)
  blk.N.attn_norm -> model.layers.N.input_layernorm.weight
  blk.N.attn_{q,k,v,output} -> model.layers.N.self_attn.{q,k,v,o}_proj.weight
  blk.N.ffn_norm -> model.layers.N.post_attention_layernorm.weight
  blk.N.ffn_{gate,up,down} -> model.layers.N.mlp.{gate,up,down}_proj.weight
"""
from __future__ import annotations

import math
from dataclasses import asdict

from ..engine.plan import LayerPlan, ModelPlan, ScheduleEntry
from ..parts.base import PartSpec
from .base import Architecture, register_architecture
from .llama import HIDDEN_ACTS, LlamaConfig


def build_llama_plan(c: LlamaConfig) -> ModelPlan:
    scaling = asdict(c.rope_scaling) if c.rope_scaling is not None else None
    position = PartSpec.of("rope", head_dim=c.head_dim, theta=c.rope_theta, scaling=scaling)
    mixer = PartSpec.of("attention", hidden=c.hidden_size, n_heads=c.num_attention_heads,
                        n_kv_heads=c.num_key_value_heads, head_dim=c.head_dim,
                        scale=1.0 / math.sqrt(c.head_dim),          # src/model_arch.c:141-145
                        position=position, bias=c.attention_bias)
    ffn = PartSpec.of("swiglu", hidden=c.hidden_size, intermediate=c.intermediate_size, bias=c.mlp_bias,
                      activation=HIDDEN_ACTS[c.hidden_act])
    norm = PartSpec.of("rmsnorm", dim=c.hidden_size, eps=c.rms_norm_eps)
    block = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm)
    layers = []
    for i in range(c.num_hidden_layers):
        p = f"model.layers.{i}."
        names = {
            "mixer_norm.weight": p + "input_layernorm.weight",
            "mixer.wq": p + "self_attn.q_proj.weight", "mixer.wk": p + "self_attn.k_proj.weight",
            "mixer.wv": p + "self_attn.v_proj.weight", "mixer.wo": p + "self_attn.o_proj.weight",
            "mixer.bq": p + "self_attn.q_proj.bias", "mixer.bk": p + "self_attn.k_proj.bias",
            "mixer.bv": p + "self_attn.v_proj.bias", "mixer.bo": p + "self_attn.o_proj.bias",
            "ffn_norm.weight": p + "post_attention_layernorm.weight",
            "ffn.w_gate": p + "mlp.gate_proj.weight", "ffn.w_up": p + "mlp.up_proj.weight",
            "ffn.w_down": p + "mlp.down_proj.weight",
            "ffn.b_gate": p + "mlp.gate_proj.bias", "ffn.b_up": p + "mlp.up_proj.bias",
            "ffn.b_down": p + "mlp.down_proj.bias",
        }
        layers.append(LayerPlan(block=block, names=names))
    plan = ModelPlan(
        vocab_size=c.vocab_size, hidden_size=c.hidden_size, layers=layers,
        schedule=[ScheduleEntry(i) for i in range(c.num_hidden_layers)],
        final_norm=norm, embedding_name="model.embed_tokens.weight",
        final_norm_names={"weight": "model.norm.weight"},
        lm_head_name=None if c.tie_word_embeddings else "lm_head.weight",
        max_positions=c.max_position_embeddings, stop_ids=c.stop_ids())
    plan.validate()
    return plan


LLAMA = register_architecture(Architecture(name="llama", config_cls=LlamaConfig, build_plan=build_llama_plan,
                                           aliases=("LlamaForCausalLM",)))
