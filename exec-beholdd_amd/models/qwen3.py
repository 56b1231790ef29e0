"""Qwen3 dense: a pre-norm decoder of GQA attention (per-head q/k RMSNorm, split-half RoPE) and
SwiGLU feed-forwards, final RMSNorm, tied or separate head.

Tensor names and shapes (ours <- the reference's GGUF names, crates/beholdd-model/src/qwen3moe.rs:919-960):
  model.embed_tokens.weight [V, D]                      <- token_embd.weight
  model.layers.N.input_layernorm.weight [D]             <- blk.N.attn_norm.weight
  model.layers.N.self_attn.{q,k,v}_proj.weight          <- blk.N.attn_{q,k,v}.weight
  model.layers.N.self_attn.{q,k}_norm.weight [head_dim] <- blk.N.attn_{q,k}_norm.weight
  model.layers.N.self_attn.o_proj.weight [D, H*head_dim]<- blk.N.attn_output.weight
  model.layers.N.post_attention_layernorm.weight [D]    <- blk.N.ffn_norm.weight
  model.layers.N.mlp.{gate,up,down}_proj.weight         <- blk.N.ffn_{gate,up,down}.weight
  model.norm.weight [D]                                 <- output_norm.weight
  lm_head.weight [V, D] (absent when tied)              <- output.weight
"""

from __future__ import annotations

from ..config.qwen3 import Qwen3Config
from ..registry import register_architecture
from .decoder import build_decoder


def build_qwen3(config: Qwen3Config):
    return build_decoder(config, position_encoding="rope")


register_architecture("Qwen3ForCausalLM", Qwen3Config, build_qwen3)
