"""The configuration of the Llama dense decoder.

The reference reads the same quantities from its model file's metadata, with the
same defaults (llama.cu/src/model/mod.rs:62-78): key/value heads default to the
number of heads, the head size to width / heads, the norm's epsilon to 1e-5 and the
rotation base to 1e4.  Here they come from config.json under its own key names.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Tuple

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class LlamaConfig:
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    rope_interleaved: bool = False
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: int = -1
    architecture: str = "LlamaForCausalLM"

    @staticmethod
    def from_dict(data: Dict[str, Any], where: str = "config.json") -> "LlamaConfig":
        r = KeyReader(data, where)
        hidden = r.integer("hidden_size")
        heads = r.integer("num_attention_heads")
        kv_heads = r.integer("num_key_value_heads", default=heads)
        if "head_dim" not in data or data["head_dim"] is None:
            if hidden % heads:
                raise ConfigError(f"{where}: 'hidden_size' {hidden} is no multiple of "
                                  f"'num_attention_heads' {heads} and there is no 'head_dim'")
        head_dim = r.integer("head_dim", default=hidden // heads)
        if heads % kv_heads:
            raise ConfigError(f"{where}: 'num_attention_heads' {heads} is no multiple of "
                              f"'num_key_value_heads' {kv_heads}")
        if head_dim % 2:
            raise ConfigError(f"{where}: 'head_dim' {head_dim} must be even (pairs are rotated)")
        # keys that would change the computation: the reference has none of these
        r.absent_or("hidden_act", ("silu",), "the feed-forward is SwiGLU")
        r.absent_or("rope_scaling", (), "the reference scales no rotation frequencies")
        r.absent_or("attention_bias", (False,), "Llama's projections have no bias")
        r.absent_or("mlp_bias", (False,), "Llama's projections have no bias")
        r.absent_or("sliding_window", (), "Llama attends to all earlier tokens")
        bos = data.get("bos_token_id")
        return LlamaConfig(
            num_hidden_layers=r.integer("num_hidden_layers"),
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=r.integer("intermediate_size"),
            vocab_size=r.integer("vocab_size"),
            max_position_embeddings=r.integer("max_position_embeddings"),
            rope_theta=r.number("rope_theta", default=1e4),
            rms_norm_eps=r.number("rms_norm_eps", default=1e-5),
            tie_word_embeddings=r.boolean("tie_word_embeddings", default=False),
            rope_interleaved=r.boolean("rope_interleaved", default=False),
            eos_token_ids=r.token_ids("eos_token_id"),
            bos_token_id=bos if isinstance(bos, int) and not isinstance(bos, bool) else -1,
        )

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "num_hidden_layers": self.num_hidden_layers,
            "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
        }
        if self.rope_interleaved:
            d["rope_interleaved"] = True
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id >= 0:
            d["bos_token_id"] = self.bos_token_id
        return d
