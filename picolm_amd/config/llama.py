"""Typed configuration of the dense Llama decoder, read from the keys of its config.json.

The keys and their defaults are those picolm reads in `load_config_safetensors`
(picolm/safetensors.c:65-78, :101-102) and `load_tokenizer_safetensors` (:309-331); what
picolm ignores but the checkpoint format carries (`max_position_embeddings`,
`rope_scaling`, `tie_word_embeddings`) is read here too.  Every size the engine uses comes
from an instance of `LlamaConfig`; nothing is a constant in code.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field


MAX_HEAD_DIM = 1024


class ConfigError(ValueError):
    """A config.json that cannot describe a model; the message names the key."""


@dataclass(frozen=True)
class RopeScaling:
    """`rope_scaling` block of kind "llama3": wavelength-dependent division of frequencies."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    def to_dict(self) -> dict:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }

    @staticmethod
    def from_dict(d) -> "RopeScaling | None":
        if d is None:
            return None
        if not isinstance(d, dict):
            raise ConfigError("rope_scaling: expected an object or null")
        kind = d.get("rope_type", d.get("type"))
        if kind in (None, "default"):
            return None
        if kind != "llama3":
            raise ConfigError(f"rope_scaling.rope_type: '{kind}' is not supported (known: llama3, default)")
        missing = [k for k in ("factor", "low_freq_factor", "high_freq_factor",
                               "original_max_position_embeddings") if k not in d]
        if missing:
            raise ConfigError("rope_scaling: missing " + ", ".join(missing))
        rs = RopeScaling("llama3", float(d["factor"]), float(d["low_freq_factor"]),
                         float(d["high_freq_factor"]), int(d["original_max_position_embeddings"]))
        if rs.factor <= 0:
            raise ConfigError("rope_scaling.factor: must be positive")
        if rs.high_freq_factor <= rs.low_freq_factor:
            raise ConfigError("rope_scaling: high_freq_factor must exceed low_freq_factor")
        if rs.original_max_position_embeddings <= 0:
            raise ConfigError("rope_scaling.original_max_position_embeddings: must be positive")
        return rs


_ROPE_STYLES = ("pairwise", "half")
_DTYPES = ("bfloat16", "float32", "float16")


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    num_hidden_layers: int
    vocab_size: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: RopeScaling | None
    max_position_embeddings: int
    tie_word_embeddings: bool
    bos_token_id: int
    eos_token_ids: tuple
    torch_dtype: str = "bfloat16"
    # How a head's dimensions pair up under rotation: "pairwise" (2i, 2i+1) is what
    # picolm applies to Llama (rope_type 0, picolm/tensor.c:3298); "half" is (i, i+d/2).
    rope_style: str = "pairwise"
    architectures: tuple = field(default=("LlamaForCausalLM",))

    # -- reading ---------------------------------------------------------------------------
    @staticmethod
    def from_dict(root: dict) -> "LlamaConfig":
        if not isinstance(root, dict):
            raise ConfigError("config.json: expected an object")
        d = root.get("text_config") if isinstance(root.get("text_config"), dict) else root

        def integer(key, default=None):
            v = d.get(key, default)
            if v is None:
                raise ConfigError(f"{key}: missing")
            if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
                raise ConfigError(f"{key}: expected an integer, got {v!r}")
            return int(v)

        # What this architecture's layers do not have.  picolm reads none of these keys (its layers
        # have no bias tensors, picolm/safetensors.c:242-277, and one activation,
        # picolm/tensor.c:3306-3315); a checkpoint that says otherwise would be computed wrongly.
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"{key}: true is not supported (the products of this architecture have no bias)")
        act = d.get("hidden_act", "silu")
        if act not in ("silu", "swish"):
            raise ConfigError(f"hidden_act: '{act}' is not supported (the feed-forward is silu(gate) * up)")
        H = integer("num_attention_heads")
        D = integer("hidden_size")
        if H <= 0:
            raise ConfigError("num_attention_heads: must be positive")
        head_dim = integer("head_dim", 0)
        if not head_dim:
            # picolm divides without a check (picolm/safetensors.c:75-76); a width that the heads
            # do not divide would give every head a silently smaller size
            if D % H:
                raise ConfigError(f"hidden_size: {D} is not divisible by num_attention_heads = {H}, and head_dim is not given")
            head_dim = D // H
        eps = float(d.get("rms_norm_eps") or 0.0) or 1e-6          # safetensors.c:77-78
        theta = float(d.get("rope_theta") or 0.0)
        if theta <= 0.0:
            theta = 10000.0                                         # safetensors.c:102
        eos = root.get("eos_token_id", d.get("eos_token_id", 2))   # safetensors.c:310
        if isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        elif eos is None:
            eos_ids = ()
        else:
            eos_ids = (int(eos),)
        bos = root.get("bos_token_id", d.get("bos_token_id", 1))   # safetensors.c:309
        archs = root.get("architectures") or d.get("architectures") or ["LlamaForCausalLM"]
        cfg = LlamaConfig(
            hidden_size=D,
            intermediate_size=integer("intermediate_size"),
            num_attention_heads=H,
            num_key_value_heads=integer("num_key_value_heads", 0) or H,
            num_hidden_layers=integer("num_hidden_layers"),
            vocab_size=integer("vocab_size"),
            head_dim=head_dim,
            rms_norm_eps=eps,
            rope_theta=theta,
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            max_position_embeddings=integer("max_position_embeddings", 4096),  # safetensors.c:495
            tie_word_embeddings=bool(d.get("tie_word_embeddings", root.get("tie_word_embeddings", False))),
            bos_token_id=1 if bos is None else int(bos),
            eos_token_ids=eos_ids,
            torch_dtype=str(d.get("torch_dtype", root.get("torch_dtype", "bfloat16"))),
            rope_style=str(d.get("rope_style", "pairwise")),
            architectures=tuple(archs),
        )
        cfg.validate()
        return cfg

    @staticmethod
    def from_json_file(path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path, "r", encoding="utf-8") as f:
            return LlamaConfig.from_dict(json.load(f))

    # -- checking --------------------------------------------------------------------------
    def validate(self) -> None:
        for key in ("hidden_size", "intermediate_size", "num_attention_heads", "num_key_value_heads",
                    "num_hidden_layers", "vocab_size", "head_dim", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key}: must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"num_key_value_heads: {self.num_key_value_heads} does not divide "
                f"num_attention_heads {self.num_attention_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"head_dim: {self.head_dim} is odd; rotation needs pairs")
        if self.head_dim > MAX_HEAD_DIM:
            # picolm's bound too (picolm/model_attention.c:163); here it is what a tile of the
            # attention kernels holds, and it is refused when the configuration is read
            raise ConfigError(f"head_dim: {self.head_dim} exceeds {MAX_HEAD_DIM}, the largest head the attention kernels take")
        if not (self.rms_norm_eps > 0.0):
            raise ConfigError("rms_norm_eps: must be positive")
        if self.rope_style not in _ROPE_STYLES:
            raise ConfigError(f"rope_style: '{self.rope_style}' is not one of {_ROPE_STYLES}")
        if self.torch_dtype not in _DTYPES:
            raise ConfigError(f"torch_dtype: '{self.torch_dtype}' is not one of {_DTYPES}")
        for e in self.eos_token_ids:
            if not 0 <= e < self.vocab_size:
                raise ConfigError(f"eos_token_id: {e} is outside the vocabulary of {self.vocab_size}")

    # -- writing ---------------------------------------------------------------------------
    def to_dict(self) -> dict:
        eos = list(self.eos_token_ids)
        return {
            "architectures": list(self.architectures),
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "num_hidden_layers": self.num_hidden_layers,
            "vocab_size": self.vocab_size,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.to_dict() if self.rope_scaling else None,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": eos[0] if len(eos) == 1 else eos,
            "torch_dtype": self.torch_dtype,
            "rope_style": self.rope_style,
        }

    # -- derived ---------------------------------------------------------------------------
    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def parameter_count(self) -> int:
        D, F, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers
        per_layer = D * (self.q_size + 2 * self.kv_size) + self.q_size * D + 3 * D * F + 2 * D
        head = 0 if self.tie_word_embeddings else V * D
        return V * D + L * per_layer + D + head
