"""The Llama dense decoder laid out of parts.

Everything here is data: which parts, with which sizes and constants from the
configuration, under which tensor names, in which order
(llama.cu/src/model/mod.rs:90-169 is the reference's version of this table).
"""
from __future__ import annotations

from ..config import LlamaConfig, register_architecture
from ..parts import ModelSpec, PartSpec, RunEntry


def llama_spec(cfg: LlamaConfig) -> ModelSpec:
    d = cfg.hidden_size

    def norm(name: str) -> PartSpec:
        # one epsilon for all norms: llama.cu/src/model/mod.rs:77,103-110,132-139,159-166
        return PartSpec("rmsnorm", {"size": d, "eps": cfg.rms_norm_eps}, name)

    layers = []
    for i in range(cfg.num_hidden_layers):
        position = PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                       "max_positions": cfg.max_position_embeddings,
                                       "interleaved": cfg.rope_interleaved})
        mixer = PartSpec("attention", {"hidden_size": d, "heads": cfg.num_attention_heads,
                                       "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                                       "scale": cfg.head_dim ** -0.5, "window": 0, "position": position},
                         "self_attn")
        ffn = PartSpec("swiglu", {"hidden_size": d, "intermediate_size": cfg.intermediate_size}, "mlp")
        layers.append(PartSpec("prenorm", {"norm1": norm("input_layernorm"), "mixer": mixer,
                                           "norm2": norm("post_attention_layernorm"), "ffn": ffn},
                               f"model.layers.{i}"))
    return ModelSpec(
        hidden_size=d, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("tokens", {"vocab_size": cfg.vocab_size, "hidden_size": d}, "model.embed_tokens"),
        layers=layers,
        run_order=[RunEntry(i) for i in range(cfg.num_hidden_layers)],
        final_norm=norm("model.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": d, "tied": cfg.tie_word_embeddings},
                      "lm_head"),
        eos_token_ids=cfg.eos_token_ids)


# files of this architecture may carry each layer's rotation frequencies, which are no weights (the tables are made
# from rope_theta)
register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, llama_spec,
                      ignored_tensors=[r".*\.rotary_emb\.inv_freq$"])
