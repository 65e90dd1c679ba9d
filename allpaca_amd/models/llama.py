"""The dense llama decoder described with parts (LlamaForCausalLM / "llama").

Layer l: pre-norm arrangement of grouped-query attention with rotary positions
and a SwiGLU feed-forward, RMS norms, then a final norm and a linear head that
may be tied to the embedding (crates/allpaca-core/src/model.rs:7904-8044 for the
tensor names, 8301-8792 for the order of operations)."""
from __future__ import annotations

from ..config.llama import LlamaConfig
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, PlanEntry
from . import ARCHITECTURES, Architecture


# Names under which a file may hold the tensors, in the reference's order of trial: GGUF-style first, then the names
# of HF checkpoints, then those without the `model.` prefix, then a few older spellings
# (crates/allpaca-safetensors/src/names.rs:26-107).  Only names: the layout is that of HF checkpoints whatever the
# name (rows of q and k are not permuted; the rotation pairs i with i + d/2).
_LAYER_ALIASES = {
    "input_layernorm.weight": ("blk.{i}.attn_norm.weight", "model.layers.{i}.input_layernorm.weight",
                               "layers.{i}.input_layernorm.weight", "model.layers.{i}.rms_1.weight"),
    "self_attn.q_proj.weight": ("blk.{i}.attn_q.weight", "model.layers.{i}.self_attn.q_proj.weight",
                                "layers.{i}.self_attn.q_proj.weight"),
    "self_attn.k_proj.weight": ("blk.{i}.attn_k.weight", "model.layers.{i}.self_attn.k_proj.weight",
                                "layers.{i}.self_attn.k_proj.weight"),
    "self_attn.v_proj.weight": ("blk.{i}.attn_v.weight", "model.layers.{i}.self_attn.v_proj.weight",
                                "layers.{i}.self_attn.v_proj.weight"),
    "self_attn.o_proj.weight": ("blk.{i}.attn_output.weight", "model.layers.{i}.self_attn.o_proj.weight",
                                "layers.{i}.self_attn.o_proj.weight"),
    "post_attention_layernorm.weight": ("blk.{i}.ffn_norm.weight", "model.layers.{i}.post_attention_layernorm.weight",
                                        "layers.{i}.post_attention_layernorm.weight", "model.layers.{i}.rms_2.weight"),
    "mlp.gate_proj.weight": ("blk.{i}.ffn_gate.weight", "model.layers.{i}.mlp.gate_proj.weight",
                             "layers.{i}.mlp.gate_proj.weight", "model.layers.{i}.mlp.w1.weight"),
    "mlp.up_proj.weight": ("blk.{i}.ffn_up.weight", "model.layers.{i}.mlp.up_proj.weight",
                           "layers.{i}.mlp.up_proj.weight", "model.layers.{i}.mlp.w3.weight"),
    "mlp.down_proj.weight": ("blk.{i}.ffn_down.weight", "model.layers.{i}.mlp.down_proj.weight",
                             "layers.{i}.mlp.down_proj.weight", "model.layers.{i}.mlp.w2.weight"),
}
_TOP_ALIASES = {
    "model.embed_tokens.weight": ("token_embd.weight", "model.embed_tokens.weight", "embed_tokens.weight",
                                  "model.model.embed_tokens.weight"),
    "model.norm.weight": ("output_norm.weight", "model.norm.weight", "model.model.norm.weight",
                          "model.final_layernorm.weight"),
    "lm_head.weight": ("output.weight", "lm_head.weight"),
}


def llama_aliases(n_layers: int) -> dict:
    out = {name: list(names) for name, names in _TOP_ALIASES.items()}
    for i in range(n_layers):
        for rest, names in _LAYER_ALIASES.items():
            out[f"model.layers.{i}.{rest}"] = [n.format(i=i) for n in names]
    return out


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
        aliases=llama_aliases(cfg.num_hidden_layers),
    )


ARCHITECTURES.register(("LlamaForCausalLM", "llama"), Architecture("llama", LlamaConfig.from_dict, llama_spec))
