"""The dense Llama decoder put together from parts (models/src/llama.rs:384-504 of the reference).

Every layer is a pre-norm block of RMSNorm, grouped-query attention with rotary positions, RMSNorm and a SwiGLU
feed-forward; the head is tied to the embedding when ``tie_word_embeddings`` says so.  Tensor names are the
checkpoint's own (models/src/llama.rs:481-489, 414-421, 322-325, 372-374).
"""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..config.registry import register_architecture
from ..parts.base import make_part
from ..parts.embedding import OutputHead, TokenEmbedding
from .spec import ModelSpec


def build_llama(cfg: LlamaConfig) -> ModelSpec:
    hd = cfg.head_size
    scaling = None
    if cfg.rope_scaling is not None and cfg.rope_scaling.rope_type == "llama3":
        scaling = {k: v for k, v in cfg.rope_scaling.to_dict().items() if k != "rope_type"}
    layers = []
    for i in range(cfg.num_hidden_layers):
        position = make_part("position", "rotary", head_size=hd, theta=cfg.rope_theta,
                             max_positions=cfg.max_position_embeddings, scaling=scaling)
        mixer = make_part("mixer", "attention", width=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                          num_kv_heads=cfg.num_key_value_heads, head_size=hd, position=position,
                          window=cfg.sliding_window)
        ffn = make_part("feed_forward", "swiglu", width=cfg.hidden_size, intermediate=cfg.intermediate_size)
        block = make_part("block", "pre_norm",
                          norm1=make_part("norm", "rmsnorm", width=cfg.hidden_size, eps=cfg.rms_norm_eps),
                          mixer=mixer,
                          norm2=make_part("norm", "rmsnorm", width=cfg.hidden_size, eps=cfg.rms_norm_eps),
                          feed_forward=ffn)
        layers.append((f"model.layers.{i}", block))
    embedding = TokenEmbedding(cfg.vocab_size, cfg.hidden_size)
    head = OutputHead(cfg.hidden_size, cfg.vocab_size, tied_to=embedding if cfg.tie_word_embeddings else None)
    ignorable = [r"model\.layers\.\d+\.self_attn\.rotary_emb\.inv_freq"]
    if cfg.tie_word_embeddings:
        ignorable.append(r"lm_head\.weight")  # the reference ignores it too when tied (models/src/llama.rs:482-486)
    return ModelSpec(width=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
                     embedding=("model.embed_tokens", embedding), layers=layers,
                     final_norm=("model.norm", make_part("norm", "rmsnorm", width=cfg.hidden_size,
                                                         eps=cfg.rms_norm_eps)),
                     head=("lm_head", head), eos_token_ids=cfg.eos_token_id, ignorable=tuple(ignorable))


for _name in LlamaConfig.architectures:
    register_architecture(_name, LlamaConfig, build_llama, replace=True)
