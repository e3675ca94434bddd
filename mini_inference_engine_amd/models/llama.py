"""Llama dense decoder assembled from parts.

Layer formulas and tensor names as inference_engine/model.py:96-113,161-185:
per layer input_layernorm -> self_attn (q/k/v/o_proj, rotary half-split, GQA,
scale 1/sqrt(head_dim)) -> post_attention_layernorm -> mlp (gate/up/down_proj,
SiLU); model.norm; lm_head or the tied embedding.  Everything here is
construction: sizes and constants come from LlamaConfig only.
"""
from __future__ import annotations

from ..config.model_config import LlamaConfig
from ..config.registry import register_architecture
from ..parts import (Attention, DecoderSpec, Embedding, LMHead, PreNormBlock, RMSNorm, RotaryHalfSplit, SwiGLU)


def build_llama(cfg: LlamaConfig) -> DecoderSpec:
    h = cfg.hidden_size
    rope = RotaryHalfSplit(cfg.head_dim, cfg.rope_theta, cfg.max_position_embeddings)
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        layers.append(PreNormBlock(
            norm_mixer=RMSNorm(h, cfg.rms_norm_eps, f"{p}.input_layernorm.weight"),
            mixer=Attention(h, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
                            scale=cfg.head_dim ** -0.5, position=rope, prefix=f"{p}.self_attn"),
            norm_feed_forward=RMSNorm(h, cfg.rms_norm_eps, f"{p}.post_attention_layernorm.weight"),
            feed_forward=SwiGLU(h, cfg.intermediate_size, prefix=f"{p}.mlp"),
        ))
    embedding = Embedding(cfg.vocab_size, h, "model.embed_tokens.weight")
    head = LMHead(cfg.vocab_size, h, "lm_head.weight", tied_to=embedding if cfg.tie_word_embeddings else None)
    ignore = [r".*\.rotary_emb\.inv_freq"]
    if cfg.tie_word_embeddings:
        ignore.append(r"lm_head\.weight")
    return DecoderSpec(embedding=embedding, layers=layers, final_norm=RMSNorm(h, cfg.rms_norm_eps, "model.norm.weight"),
                       head=head, ignore_tensors=tuple(ignore), stop_token_ids=tuple(cfg.eos_token_id),
                       max_position=cfg.max_position_embeddings, vocab_size=cfg.vocab_size)


# Named sizes: the two tiny configurations of the tests, the benchmark's layer sizes, and two larger models' sizes.
SHAPES = {
    "tiny-a": dict(vocab_size=256, hidden_size=64, intermediate_size=176, num_hidden_layers=2, num_attention_heads=4,
                   num_key_value_heads=2, head_dim=16, rms_norm_eps=1e-5, rope_theta=10000.0,
                   max_position_embeddings=128, tie_word_embeddings=False),
    "tiny-b": dict(vocab_size=384, hidden_size=96, intermediate_size=256, num_hidden_layers=3, num_attention_heads=3,
                   num_key_value_heads=1, head_dim=32, rms_norm_eps=1e-6, rope_theta=500000.0,
                   max_position_embeddings=256, tie_word_embeddings=True),
    "tinyllama": dict(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_hidden_layers=22,
                      num_attention_heads=32, num_key_value_heads=4, head_dim=64, rms_norm_eps=1e-5,
                      rope_theta=10000.0, max_position_embeddings=2048, tie_word_embeddings=False),
    "llama2-7b": dict(vocab_size=32000, hidden_size=4096, intermediate_size=11008, num_hidden_layers=32,
                      num_attention_heads=32, num_key_value_heads=32, head_dim=128, rms_norm_eps=1e-5,
                      rope_theta=10000.0, max_position_embeddings=4096, tie_word_embeddings=False),
    "llama3-8b": dict(vocab_size=128256, hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
                      num_attention_heads=32, num_key_value_heads=8, head_dim=128, rms_norm_eps=1e-5,
                      rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False),
}

register_architecture("LlamaForCausalLM", LlamaConfig, build_llama, model_type="llama", shapes=SHAPES, replace=True)
