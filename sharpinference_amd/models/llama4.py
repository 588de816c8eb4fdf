"""Llama 4 (text): the configuration's options turned into parts, layer by layer.

The reference runs Llama 4 as a flag set on its generic decoder (reference:
src/SharpInference.Core/ModelGraph.cs:292-301: no rotary every 4th layer, sigmoid gating,
weightless QK norm; interleaved rotary pairs because the architecture is absent from the NEOX
list, 308-328).  Here each of those is a choice of part or of a part's argument, made per
layer from config.json:

* rotary layers: interleaved rotary (llama3 scaling if configured), weightless per-head norm
  if ``use_qk_norm``, attention confined to the chunk of ``attention_chunk_size``;
* layers without rotary: all keys, queries scaled by the position-dependent temperature if
  ``attn_temperature_tuning``;
* ``hidden_act`` names the gated unit's activation of every feed-forward, ``attention_bias``
  gives the four attention projections biases;
* layer L carries experts iff (L + 1) % interleave_moe_layer_step == 0 (top-k sigmoid router
  scaling the expert input, plus the shared expert), otherwise the dense feed-forward of
  width ``intermediate_size_mlp``.
"""
from __future__ import annotations

from ..cache.spec import WINDOW_CHUNK, WINDOW_NONE
from ..config.llama4 import Llama4TextConfig
from ..parts.attention import Attention
from ..parts.block import PreNormBlock
from ..parts.feedforward import DenseSwiGLU, MoESwiGLU
from ..parts.model import DecoderModel
from ..parts.norm import RMSNorm
from ..parts.position import RotaryInterleaved
from ..registry import register_architecture


def build_llama4(cfg: Llama4TextConfig) -> DecoderModel:
    cfg.validate()
    rotary = RotaryInterleaved(cfg.head_dim, cfg.rope_theta, cfg.rope_scaling)
    blocks = []
    for layer in range(cfg.num_hidden_layers):
        if cfg.uses_rope(layer):
            mixer = Attention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                              rotary=rotary, qk_norm_eps=cfg.rms_norm_eps if cfg.use_qk_norm else None,
                              q_temperature=None, window_kind=WINDOW_CHUNK, window=cfg.attention_chunk_size,
                              bias=cfg.attention_bias)
        else:
            temp = (cfg.floor_scale, cfg.attn_scale) if cfg.attn_temperature_tuning else None
            mixer = Attention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                              rotary=None, qk_norm_eps=None, q_temperature=temp, window_kind=WINDOW_NONE,
                              bias=cfg.attention_bias)
        if cfg.is_moe_layer(layer):
            ffn = MoESwiGLU(cfg.hidden_size, cfg.num_local_experts, cfg.num_experts_per_tok, cfg.intermediate_size,
                            shared_intermediate=cfg.intermediate_size, gate="sigmoid", renormalise=False,
                            score_on_input=True, activation=cfg.activation)
        else:
            ffn = DenseSwiGLU(cfg.hidden_size, cfg.intermediate_size_mlp, activation=cfg.activation)
        blocks.append(PreNormBlock(RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), mixer,
                                   RMSNorm(cfg.hidden_size, cfg.rms_norm_eps), ffn))
    return DecoderModel(cfg.vocab_size, cfg.hidden_size, blocks, RMSNorm(cfg.hidden_size, cfg.rms_norm_eps),
                        tie_embeddings=cfg.tie_word_embeddings, config=cfg)


register_architecture("Llama4ForCausalLM", Llama4TextConfig, build_llama4)
# A multimodal folder names the container class; of it this engine runs the text decoder alone
# (its keys sit under text_config, its tensors under a prefix that the loader strips; the other
# towers' tensors are passed over).
register_architecture("Llama4ForConditionalGeneration", Llama4TextConfig, build_llama4)
