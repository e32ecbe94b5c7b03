"""Typed configuration of the Qwen2.5 dense decoder, read from config.json.

Which keys exist, which are required and what is refused follows the
reference's Qwen2 loader (/root/reference/core/src/model/loader.cpp:628-685:
every size, the norm eps and the rope base are required) and its validity
check (/root/reference/core/src/model/config.cpp:21-49: heads divisible by kv
heads, rope base > 0, eps >= 0).  The head size is width / heads
(loader.cpp:662).  No size and no constant of config.json stands anywhere
else in the code: parts get them from here as parameters.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, read_key, token_id_list


@dataclass(frozen=True)
class RopeScaling:
    """Long-context frequency scaling, ``rope_scaling`` in config.json.

    ``kind`` is "linear" or "yarn".  Both become a per-pair divisor of the
    rotation angle; YaRN also multiplies the attention scores
    (/root/reference/core/src/model/loader.cpp:192-311).
    """
    kind: str
    factor: float
    original_max_position_embeddings: int
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    attention_factor: float = 1.0


@dataclass(frozen=True)
class Qwen2Config:
    architecture: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool = False
    use_sliding_window: bool = False
    hidden_act: str = "silu"
    rope_scaling: Optional[RopeScaling] = None
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    # ---- derived ---------------------------------------------------------
    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def q_width(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_key_value_heads * self.head_dim

    # ---- reading ---------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen2Config":
        arch = d.get("architectures") or ["Qwen2ForCausalLM"]
        rs = d.get("rope_scaling")
        scaling = None
        if rs is not None:
            if not isinstance(rs, Mapping):
                raise ConfigError("missing/invalid config key: rope_scaling (want an object or null)")
            kind = rs.get("rope_type", rs.get("type"))
            if kind in (None, "none", "default"):
                scaling = None
            elif kind in ("linear", "yarn"):
                scaling = RopeScaling(
                    kind=kind,
                    factor=read_key(rs, "factor", float),
                    original_max_position_embeddings=read_key(
                        rs, "original_max_position_embeddings", int,
                        read_key(d, "max_position_embeddings", int, 0)),
                    beta_fast=read_key(rs, "beta_fast", float, 32.0),
                    beta_slow=read_key(rs, "beta_slow", float, 1.0),
                    attention_factor=read_key(rs, "attention_factor", float, 1.0),
                )
            else:
                raise ConfigError(f"unsupported rope scaling type: {kind}")
        known = {
            "architectures", "vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
            "num_attention_heads", "num_key_value_heads", "rms_norm_eps", "rope_theta",
            "max_position_embeddings", "tie_word_embeddings", "use_sliding_window", "hidden_act",
            "rope_scaling", "eos_token_id", "bos_token_id", "torch_dtype", "head_dim",
        }
        cfg = cls(
            architecture=str(arch[0]),
            vocab_size=read_key(d, "vocab_size", int),
            hidden_size=read_key(d, "hidden_size", int),
            intermediate_size=read_key(d, "intermediate_size", int),
            num_hidden_layers=read_key(d, "num_hidden_layers", int),
            num_attention_heads=read_key(d, "num_attention_heads", int),
            num_key_value_heads=read_key(d, "num_key_value_heads", int),
            rms_norm_eps=read_key(d, "rms_norm_eps", float),
            rope_theta=read_key(d, "rope_theta", float),
            max_position_embeddings=read_key(d, "max_position_embeddings", int, 0),
            tie_word_embeddings=read_key(d, "tie_word_embeddings", bool, False),
            use_sliding_window=read_key(d, "use_sliding_window", bool, False),
            hidden_act=read_key(d, "hidden_act", str, "silu"),
            rope_scaling=scaling,
            eos_token_ids=token_id_list(d.get("eos_token_id"), "eos_token_id"),
            bos_token_id=read_key(d, "bos_token_id", int, None),
            torch_dtype=read_key(d, "torch_dtype", str, "bfloat16"),
            extra={k: v for k, v in d.items() if k not in known},
        )
        cfg.validate(explicit_head_dim=d.get("head_dim"))
        return cfg

    def validate(self, explicit_head_dim=None) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"missing/invalid config key: {key} (must be positive)")
        if self.max_position_embeddings < 0:
            raise ConfigError("missing/invalid config key: max_position_embeddings (must not be negative)")
        if self.hidden_size % self.num_attention_heads:
            raise ConfigError(
                f"inconsistent config: hidden_size {self.hidden_size} is not a multiple of "
                f"num_attention_heads {self.num_attention_heads}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"inconsistent config: num_attention_heads {self.num_attention_heads} is not a "
                f"multiple of num_key_value_heads {self.num_key_value_heads}")
        if explicit_head_dim is not None and explicit_head_dim != self.head_dim:
            raise ConfigError(
                f"inconsistent config: head_dim {explicit_head_dim} differs from "
                f"hidden_size / num_attention_heads = {self.head_dim}")
        if self.head_dim % 2:
            raise ConfigError(f"inconsistent config: head size {self.head_dim} is odd; rotation pairs need an even size")
        if not (self.rope_theta > 0.0) or not math.isfinite(self.rope_theta):
            raise ConfigError("missing/invalid config key: rope_theta (must be > 0)")
        if not (self.rms_norm_eps >= 0.0) or not math.isfinite(self.rms_norm_eps):
            raise ConfigError("missing/invalid config key: rms_norm_eps (must be >= 0)")
        if self.hidden_act != "silu":
            raise ConfigError(f"unsupported hidden_act: {self.hidden_act} (this architecture's feed-forward is SiLU-gated)")
        if self.use_sliding_window:
            raise ConfigError("unsupported: use_sliding_window=true (every layer of this architecture attends all keys)")
        if self.rope_scaling is not None:
            if not (self.rope_scaling.factor > 0.0):
                raise ConfigError("missing/invalid config key: rope_scaling.factor (must be > 0)")
            if self.rope_scaling.kind == "yarn" and self.rope_scaling.original_max_position_embeddings <= 0:
                raise ConfigError("missing/invalid config key: rope_scaling.original_max_position_embeddings")
        for t in self.eos_token_ids:
            if not 0 <= t < self.vocab_size:
                raise ConfigError(f"missing/invalid config key: eos_token_id ({t} is outside the vocabulary)")

    def to_dict(self) -> dict:
        """The config.json form (what :meth:`from_dict` reads back unchanged)."""
        d = dict(self.extra)
        d.update({
            "architectures": [self.architecture],
            "model_type": d.get("model_type", "qwen2"),
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "hidden_act": self.hidden_act,
            "torch_dtype": self.torch_dtype,
        })
        if self.rope_scaling is not None:
            d["rope_scaling"] = {
                "type": self.rope_scaling.kind,
                "factor": self.rope_scaling.factor,
                "original_max_position_embeddings": self.rope_scaling.original_max_position_embeddings,
                "beta_fast": self.rope_scaling.beta_fast,
                "beta_slow": self.rope_scaling.beta_slow,
                "attention_factor": self.rope_scaling.attention_factor,
            }
        else:
            d["rope_scaling"] = None
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        return d
