"""LlamaConfig: the keys of a Llama config.json, typed and checked.

Fields and checks follow the reference's Config (runtime/model.py:11-35) and
its loader's rejections (runtime/checkpoint.py:12-17), with ``head_dim`` as a
key of its own (the reference requires it to equal hidden/heads,
runtime/checkpoint.py:17; here any even size up to 256 in the projections'
shapes is allowed).
"""
from dataclasses import dataclass, asdict
from typing import Optional, Tuple

from .base import ConfigError

_REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads")


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    model_type = "llama"

    def __post_init__(self):
        sizes = (self.vocab_size, self.hidden_size, self.intermediate_size, self.num_hidden_layers,
                 self.num_attention_heads, self.num_key_value_heads, self.head_dim, self.max_position_embeddings)
        if any((not isinstance(v, int)) or isinstance(v, bool) or v <= 0 for v in sizes):
            raise ConfigError("model dimensions must be positive integers")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2 or self.head_dim > 256:
            raise ConfigError(f"head_dim {self.head_dim}: supported head sizes are even and at most 256")
        if not (self.rms_norm_eps >= 0) or not (self.rope_theta > 0):
            raise ConfigError("rms_norm_eps must be >= 0 and rope_theta > 0")

    @classmethod
    def from_dict(cls, raw):
        if raw.get("model_type", "llama") != "llama":
            raise ConfigError(f"model_type {raw.get('model_type')!r} is not llama")
        missing = [k for k in _REQUIRED if k not in raw]
        if missing:
            raise ConfigError(f"config.json lacks {missing}")
        if raw.get("rope_scaling"):
            raise ConfigError("rope_scaling is not supported (plain rotary embedding only)")
        if raw.get("attention_bias") or raw.get("mlp_bias"):
            raise ConfigError("biased projections (attention_bias, mlp_bias) are not supported")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"hidden_act {raw.get('hidden_act')!r}: only silu is supported")
        heads = raw["num_attention_heads"]
        head_dim = raw.get("head_dim")
        if head_dim is None:
            if raw["hidden_size"] % heads:
                raise ConfigError("hidden_size is not a multiple of num_attention_heads and head_dim is not given")
            head_dim = raw["hidden_size"] // heads
        eos = raw.get("eos_token_id")
        eos_ids = () if eos is None else tuple(eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        return cls(
            vocab_size=raw["vocab_size"], hidden_size=raw["hidden_size"], intermediate_size=raw["intermediate_size"],
            num_hidden_layers=raw["num_hidden_layers"], num_attention_heads=heads,
            num_key_value_heads=raw.get("num_key_value_heads") or heads, head_dim=head_dim,
            # defaults where config.json is silent are the reference's (runtime/model.py:19-21, checkpoint.py:38)
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-5)), rope_theta=float(raw.get("rope_theta", 10000.0)),
            max_position_embeddings=raw.get("max_position_embeddings", 2048),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=eos_ids, bos_token_id=raw.get("bos_token_id"))

    def to_dict(self):
        d = {k: v for k, v in asdict(self).items() if k not in ("eos_token_ids",)}
        d["model_type"] = "llama"
        d["architectures"] = ["LlamaForCausalLM"]
        d["hidden_act"] = "silu"
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if d.get("bos_token_id") is None:
            d.pop("bos_token_id", None)
        return d
