"""Typed configuration of the dense Llama decoder.

Keys, defaults and required keys follow the reference's reader
(models/config.go:15-49, :102-124): ``rope_theta`` defaults to 10000,
``rms_norm_eps`` to 1e-6, ``num_key_value_heads`` to the head count,
``head_dim`` to hidden/heads, ``eos_token_id`` to "none".  Where the reference
silently ignores an option that would change the result (rope scaling, biases,
another activation), this reader refuses it.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class LlamaConfig(ModelConfig):
    vocab_size: int = 0
    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    rope_theta: float = 10000.0
    rms_norm_eps: float = 1e-6
    max_position_embeddings: Optional[int] = None
    tie_word_embeddings: bool = False
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    torch_dtype: Optional[str] = None

    # ---------------------------------------------------------------- derived
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, raw: dict, where: str = "config.json") -> "LlamaConfig":
        r = KeyReader(raw, where)
        arch = (raw.get("architectures") or ["LlamaForCausalLM"])[0]

        hidden = r.positive_int("hidden_size")
        layers = r.positive_int("num_hidden_layers")
        heads = r.positive_int("num_attention_heads")
        vocab = r.positive_int("vocab_size")
        inter = r.positive_int("intermediate_size")
        kv_heads = r.positive_int("num_key_value_heads", heads)
        if r.has("head_dim"):
            head_dim = r.positive_int("head_dim")
        else:
            if hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size {hidden} is not a multiple of num_attention_heads "
                    f"{heads} and no 'head_dim' is given")
            head_dim = hidden // heads
        if heads % kv_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads {heads} is not a multiple of "
                f"num_key_value_heads {kv_heads}")
        if head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim {head_dim} must be even for rotary pairs")

        theta = 10000.0
        if r.has("rope_theta"):
            theta = r.positive_float("rope_theta")
        # transformers >= 5 nests the base in rope_parameters (models/config.go:56-99).
        if r.has("rope_parameters"):
            rp = raw["rope_parameters"]
            if not isinstance(rp, dict):
                raise ConfigError(f"{where}: 'rope_parameters' must be an object")
            rtype = rp.get("rope_type", rp.get("type"))
            if rtype not in (None, "", "default"):
                raise ConfigError(
                    f"{where}: rope_parameters.rope_type {rtype!r} is not supported "
                    f"(no rope scaling)")
            if rp.get("rope_theta") is not None:
                theta = KeyReader(rp, where + ":rope_parameters").positive_float("rope_theta")
        if r.has("rope_scaling"):
            rs = raw["rope_scaling"]
            rtype = rs.get("rope_type", rs.get("type")) if isinstance(rs, dict) else rs
            if rtype not in (None, "", "default"):
                raise ConfigError(
                    f"{where}: 'rope_scaling' = {rs!r} is not supported (no rope scaling)")

        eps = r.positive_float("rms_norm_eps", 1e-6)
        r.refuse_unless("hidden_act", ("silu", "swish"), "the feed-forward is SiLU-gated")
        r.refuse_unless("attention_bias", (False,), "projections have no bias")
        r.refuse_unless("mlp_bias", (False,), "projections have no bias")
        r.refuse_unless("pretraining_tp", (1,), "sliced projections are not implemented")
        r.refuse_unless("sliding_window", (0,), "Llama layers keep all keys")

        eos = raw.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, bool):
            raise ConfigError(f"{where}: 'eos_token_id' must be an integer or a list of integers")
        elif isinstance(eos, int):
            eos_ids = (eos,) if eos >= 0 else ()
        elif isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
            eos_ids = tuple(e for e in eos if e >= 0)
        else:
            raise ConfigError(f"{where}: 'eos_token_id' must be an integer or a list of integers")

        max_pos = r.positive_int("max_position_embeddings", None)
        bos = raw.get("bos_token_id")
        dtype = raw.get("torch_dtype", raw.get("dtype"))
        return cls(
            architecture=arch, vocab_size=vocab, hidden_size=hidden, intermediate_size=inter,
            num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv_heads,
            head_dim=head_dim, rope_theta=theta, rms_norm_eps=eps,
            max_position_embeddings=max_pos,
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            eos_token_ids=eos_ids, bos_token_id=bos if isinstance(bos, int) else None,
            torch_dtype=dtype if isinstance(dtype, str) else None,
        )

    def to_dict(self) -> dict:
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rope_theta": self.rope_theta,
            "rms_norm_eps": self.rms_norm_eps,
            "hidden_act": "silu",
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if len(self.eos_token_ids) == 1:
            d["eos_token_id"] = self.eos_token_ids[0]
        elif self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.torch_dtype is not None:
            d["torch_dtype"] = self.torch_dtype
        return d
