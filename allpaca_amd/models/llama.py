"""The dense llama decoder described with parts (LlamaForCausalLM / "llama").

Layer l: pre-norm arrangement of grouped-query attention with rotary positions
and a SwiGLU feed-forward, RMS norms, then a final norm and a linear head that
may be tied to the embedding (crates/allpaca-core/src/model.rs:7904-8044 for the
tensor names, 8301-8792 for the order of operations)."""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    scaling = None
    if cfg.rope_scaling is not None:
        s = cfg.rope_scaling
        scaling = dict(rope_type=s.rope_type, factor=s.factor, low_freq_factor=s.low_freq_factor,
                       high_freq_factor=s.high_freq_factor,
                       original_max_position_embeddings=s.original_max_position_embeddings)
    position = PartSpec("rope", dict(head_dim=cfg.head_dim, theta=cfg.rope_theta, scaling=scaling))
    norm = dict(size=cfg.hidden_size, eps=cfg.rms_norm_eps)
    blocks = []
    for l in range(cfg.num_hidden_layers):
        blocks.append(BlockSpec(
            arrangement="pre_norm",
            weight_prefix=f"model.layers.{l}.",
            parts={
                "mixer_norm": PartSpec("rmsnorm", norm, "input_layernorm."),
                "mixer": PartSpec("attention", dict(hidden_size=cfg.hidden_size, num_heads=cfg.num_attention_heads,
                                                    num_kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim,
                                                    position=position), "self_attn."),
                "ffn_norm": PartSpec("rmsnorm", norm, "post_attention_layernorm."),
                "ffn": PartSpec("swiglu", dict(hidden_size=cfg.hidden_size,
                                               intermediate_size=cfg.intermediate_size), "mlp."),
            }))
    forbidden, copies = {}, {}
    if cfg.tie_word_embeddings:
        forbidden["lm_head.weight"] = "tie_word_embeddings is true, the head is the embedding matrix"
        copies["lm_head.weight"] = "model.embed_tokens.weight"
    return ModelSpec(
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("token_table", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size),
                           "model.embed_tokens."),
        blocks=blocks,
        plan=[PlanEntry(l) for l in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", norm, "model.norm."),
        head=PartSpec("linear", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                                     tied=cfg.tie_word_embeddings), "lm_head."),
        forbidden=forbidden,
        copies=copies,
        ignored_suffixes=(".rotary_emb.inv_freq",),   # a table of rotation frequencies that older writers stored
    )


ARCHITECTURES.register(("LlamaForCausalLM", "llama"), Architecture("llama", LlamaConfig.from_dict, llama_spec))
