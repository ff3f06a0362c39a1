"""LlamaConfig: the typed view of a Llama config.json.

Reference: field set of include/llmengine/config.hpp:9-31 and the parsing rules
of src/weights.cpp:55-121 (defaults: num_key_value_heads = num_attention_heads,
head_dim = hidden_size / num_attention_heads, rms_norm_eps 1e-5, rope_theta
10000, tie_word_embeddings false; `rope_parameters` wins over `rope_scaling`;
EOS ids are the union of config.json and generation_config.json).

Where the reference reads sizes without checking them, this parser checks and
names the key; options the engine does not implement (biases, another
activation, another rope type) are refused rather than ignored.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping

from .base import ConfigError, KeyReader


@dataclass(frozen=True)
class RopeScaling:
    """The llama3 wavelength-band scaling block (src/weights.cpp:81-96)."""

    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0
    original_max_position_embeddings: int = 0

    def to_dict(self) -> dict:
        return {
            "rope_type": "llama3",
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


def _parse_scaling(r: KeyReader) -> RopeScaling:
    s = RopeScaling(
        factor=r.number("factor", 1.0),
        low_freq_factor=r.number("low_freq_factor", 1.0),
        high_freq_factor=r.number("high_freq_factor", 1.0),
        original_max_position_embeddings=r.integer("original_max_position_embeddings", 0, minimum=0),
    )
    if s.factor <= 0 or s.low_freq_factor <= 0 or s.high_freq_factor <= 0:
        raise ConfigError(f"{r.where}: factor, low_freq_factor and high_freq_factor must be > 0")
    return s


def _rope_type(r: KeyReader) -> str | None:
    # Older files call the key "type".
    if r.has("rope_type"):
        return r.string("rope_type")
    if r.has("type"):
        return r.string("type")
    return None


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
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: RopeScaling | None = None
    tie_word_embeddings: bool = False
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    # --- derived -----------------------------------------------------------------
    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @property
    def max_pos(self) -> int:
        """Largest prompt + generated length a request may reach.

        The reference caps this at min(max_position_embeddings, original max,
        8192) (include/llmengine/config.hpp:39-45); here positions run to
        max_position_embeddings, since the rotation table is built that far.
        """
        return self.max_position_embeddings

    # --- parsing -----------------------------------------------------------------
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], generation_cfg: Mapping[str, Any] | None = None,
                  architecture: str = "LlamaForCausalLM") -> "LlamaConfig":
        r = KeyReader(cfg)
        hidden = r.integer("hidden_size", minimum=1)
        n_q = r.integer("num_attention_heads", minimum=1)
        n_kv = r.integer("num_key_value_heads", n_q, minimum=1)
        if hidden % n_q != 0 and not r.has("head_dim"):
            raise ConfigError(
                f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads {n_q} "
                "and no head_dim is given")
        head_dim = r.integer("head_dim", hidden // n_q, minimum=1)
        if n_q % n_kv != 0:
            raise ConfigError(
                f"config.json: num_attention_heads {n_q} is not a multiple of num_key_value_heads {n_kv}")
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even for rotary pairs")

        if r.has("attention_bias") and r.boolean("attention_bias"):
            raise ConfigError("config.json: attention_bias=true is not supported (projections have no bias)")
        if r.has("mlp_bias") and r.boolean("mlp_bias"):
            raise ConfigError("config.json: mlp_bias=true is not supported (projections have no bias)")
        if r.has("hidden_act") and r.string("hidden_act") != "silu":
            raise ConfigError(
                f"config.json: hidden_act={r.string('hidden_act')!r} is not supported (the MLP is SiLU-gated)")

        theta = r.number("rope_theta", 10000.0)
        scaling: RopeScaling | None = None
        rp = r.mapping("rope_parameters")
        rs = r.mapping("rope_scaling")
        if rp is not None:
            theta = rp.number("rope_theta", theta)
            kind = _rope_type(rp) or "default"
            if kind == "llama3":
                scaling = _parse_scaling(rp)
            elif kind != "default":
                raise ConfigError(f"config.json: rope_parameters.rope_type={kind!r} is not supported "
                                  "(known: 'default', 'llama3')")
        elif rs is not None:
            kind = _rope_type(rs)
            # A block without a type is read as llama3, as the reference does for any block.
            if kind in (None, "llama3"):
                scaling = _parse_scaling(rs)
            elif kind != "default":
                raise ConfigError(f"config.json: rope_scaling.rope_type={kind!r} is not supported "
                                  "(known: 'default', 'llama3')")
        if theta <= 0:
            raise ConfigError("config.json: rope_theta must be > 0")

        eos: list[int] = []

        def absorb(src: Mapping[str, Any] | None, where: str) -> None:
            if not src or src.get("eos_token_id") is None:
                return
            v = src["eos_token_id"]
            items = v if isinstance(v, list) else [v]
            for t in items:
                if isinstance(t, bool) or not isinstance(t, int):
                    raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers")
                if t not in eos:
                    eos.append(t)

        absorb(cfg, "config.json")
        absorb(generation_cfg, "generation_config.json")

        eps = r.number("rms_norm_eps", 1e-5)
        if eps < 0:
            raise ConfigError("config.json: rms_norm_eps must be >= 0")

        return cls(
            architecture=architecture,
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            num_hidden_layers=r.integer("num_hidden_layers", minimum=1),
            num_attention_heads=n_q,
            num_key_value_heads=n_kv,
            head_dim=head_dim,
            vocab_size=r.integer("vocab_size", minimum=1),
            max_position_embeddings=r.integer("max_position_embeddings", minimum=1),
            rms_norm_eps=eps,
            rope_theta=theta,
            rope_scaling=scaling,
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            eos_token_ids=tuple(sorted(eos)),
        )

    def to_dict(self) -> dict:
        """The config.json that parses back to this configuration."""
        d: dict[str, Any] = {
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
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids)
        return d
