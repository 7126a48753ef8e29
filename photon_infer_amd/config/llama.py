"""Typed configuration of the Llama architecture, read from its config.json keys.

Reference: include/photon/arch/config.hpp:16-54 (ModelConfig / TransformerConfig) and
src/arch/config.cpp:13-49 (derived sizes: head_size = dim / head_num, kv_dim,
kv_mul).  The reference fixes the RoPE base (include/photon/ops/kernels/rope_kernel.hpp:72)
and the norm eps (src/io/checkpoint.cpp:117); here both come from the file, as do the
llama3 frequency-scaling constants that the reference lacks.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Mapping, Optional

from ..errors import ConfigError, UnsupportedModelError
from .base import ConfigReader, architecture_name


@dataclass(frozen=True)
class RopeScaling:
    """Frequency scaling rule of the rotary encoding.

    ``rope_type`` is "llama3" (piecewise rule with the four constants) or "linear"
    (all frequencies divided by ``factor``).
    """

    rope_type: str
    factor: float
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0
    original_max_position_embeddings: int = 0

    def to_dict(self) -> dict:
        d = {"rope_type": self.rope_type, "factor": self.factor}
        if self.rope_type == "llama3":
            d.update(
                low_freq_factor=self.low_freq_factor,
                high_freq_factor=self.high_freq_factor,
                original_max_position_embeddings=self.original_max_position_embeddings,
            )
        return d


@dataclass(frozen=True)
class LlamaConfig:
    architecture: str
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[RopeScaling]
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    bos_token_id: Optional[int] = None
    eos_token_ids: tuple = ()
    # Pairing of rotated elements: False = (x[j], x[j + head_dim/2]), the layout of
    # Llama model folders; True = (x[2j], x[2j+1]), the reference's layout
    # (include/photon/ops/kernels/rope_kernel.hpp:126-165).
    rope_interleaved: bool = False

    # ---- derived sizes (src/arch/config.cpp:27-29) ----
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def queries_per_kv(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    # ---- parsing ----
    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str = "config.json") -> "LlamaConfig":
        r = ConfigReader(raw, where)
        hidden = r.integer("hidden_size")
        heads = r.integer("num_attention_heads")
        kv_heads = r.integer("num_key_value_heads", heads)
        if heads % kv_heads != 0:
            raise ConfigError(
                f"{where}: num_attention_heads ({heads}) must be a multiple of "
                f"num_key_value_heads ({kv_heads})"
            )
        if r.has("head_dim"):
            head_dim = r.integer("head_dim")
        else:
            if hidden % heads != 0:
                raise ConfigError(
                    f"{where}: hidden_size ({hidden}) is not a multiple of num_attention_heads "
                    f"({heads}) and no head_dim is given"
                )
            head_dim = hidden // heads
        if head_dim % 2 != 0:
            raise ConfigError(f"{where}: head_dim must be even for rotary pairs, got {head_dim}")
        act = r.string("hidden_act", "silu")
        if act != "silu":
            raise UnsupportedModelError(f"{where}: hidden_act '{act}' is not supported (only 'silu')")
        for bias_key in ("attention_bias", "mlp_bias"):
            if r.boolean(bias_key, False):
                raise UnsupportedModelError(f"{where}: {bias_key}=true is not supported")
        eos = r.int_or_list("eos_token_id")
        bos = r.int_or_list("bos_token_id")
        return cls(
            architecture=architecture_name(raw, where),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size"),
            num_hidden_layers=r.integer("num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            vocab_size=r.integer("vocab_size"),
            max_position_embeddings=r.integer("max_position_embeddings"),
            rms_norm_eps=r.number("rms_norm_eps"),
            rope_theta=r.number("rope_theta", 10000.0),
            rope_scaling=_parse_rope_scaling(r.mapping("rope_scaling")),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            hidden_act=act,
            torch_dtype=r.string("torch_dtype", "bfloat16"),
            bos_token_id=bos[0] if bos else None,
            eos_token_ids=eos,
            rope_interleaved=r.boolean("rope_interleaved", False),
        )

    def to_dict(self) -> dict:
        """The config.json form; ``from_dict(to_dict())`` round-trips."""
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": self.hidden_act,
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.rope_interleaved:
            d["rope_interleaved"] = True
        return d

    def replace(self, **kw) -> "LlamaConfig":
        return dataclasses.replace(self, **kw)


def _parse_rope_scaling(r: Optional[ConfigReader]) -> Optional[RopeScaling]:
    if r is None:
        return None
    kind = r.string("rope_type", r.string("type", "default"))
    if kind == "default":
        return None
    if kind == "linear":
        return RopeScaling("linear", r.number("factor"))
    if kind == "llama3":
        low = r.number("low_freq_factor")
        high = r.number("high_freq_factor")
        if not high > low:
            raise ConfigError(
                f"{r.where}: high_freq_factor ({high}) must be greater than low_freq_factor ({low})"
            )
        return RopeScaling(
            "llama3",
            r.number("factor"),
            low,
            high,
            r.integer("original_max_position_embeddings"),
        )
    raise UnsupportedModelError(f"{r.where}: rope_type '{kind}' is not supported (llama3, linear, default)")
