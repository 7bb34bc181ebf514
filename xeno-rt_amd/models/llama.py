"""Llama / Qwen3 dense decoder, described in parts.

Layer stack of the reference (crates/xrt-models/src/llama.rs:433-613):
L identical pre-norm blocks of grouped-query attention with rotary positions
and a SwiGLU feed-forward, a final RMSNorm and an output head that may be tied
to the embedding. Qwen3 differs by a per-head RMSNorm of q and k (llama.rs:489-496).
Tensor names are those of the checkpoints' safetensors files.
"""
from __future__ import annotations

from ..config import LlamaConfig, register_architecture
from ..parts import Attention, Embedding, GatedMLP, OutputHead, PreNormBlock, RMSNorm, Rotary
from .decoder import ModelSpec


MOST_TABLE_POSITIONS = 131072          # 64 MB of cosines and sines at a head size of 128


def build_llama(config: LlamaConfig) -> ModelSpec:
    c = config
    embedding = Embedding("model.embed_tokens.", c.vocab_size, c.hidden_size)
    layers = []
    # one rotation for all layers. With head norms a decode step's attention finishes q and k itself and reads the
    # positions' cosines and sines from a table (positions * head_dim * 4 bytes, made once when the model is bound;
    # at most MOST_TABLE_POSITIONS: a step with a longer sequence takes the two kernels)
    rotary = Rotary(c.rope_dim, c.rope_theta, scale=c.rope_scale,
                    table_positions=min(c.max_position_embeddings, MOST_TABLE_POSITIONS) if c.qk_norm and c.rope_dim == c.head_dim else 0)
    for index in range(c.num_hidden_layers):
        p = f"model.layers.{index}."
        mixer = Attention(
            p + "self_attn.", c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
            position=rotary,
            qk_norm=c.qk_norm, qk_norm_eps=c.rms_norm_eps)          # same eps as the block norms (llama.rs:1028)
        layers.append(PreNormBlock(
            RMSNorm(p + "input_layernorm.", c.hidden_size, c.rms_norm_eps),
            mixer,
            RMSNorm(p + "post_attention_layernorm.", c.hidden_size, c.rms_norm_eps),
            GatedMLP(p + "mlp.", c.hidden_size, c.intermediate_size, "silu")))
    final_norm = RMSNorm("model.norm.", c.hidden_size, c.rms_norm_eps)
    head = OutputHead("lm_head.", c.vocab_size, c.hidden_size,
                      tied_to=embedding if c.tie_word_embeddings else None)
    return ModelSpec(config=c, embedding=embedding, layers=layers, final_norm=final_norm, head=head)


register_architecture("LlamaForCausalLM", LlamaConfig, build_llama)
register_architecture("Qwen3ForCausalLM", LlamaConfig, build_llama)
