"""The Llama 3 dense decoder: its configuration, read from the keys of its own
config.json, and its description as parts.

What the architecture is (reference: the ``GPT`` of yalis/external/model.py
configured by the Llama-3 entries of yalis/external/config.py:755-951): token
embedding, pre-norm blocks of grouped-query attention with half-split rotary
positions and a SwiGLU feed-forward, RMSNorm everywhere, an untied or tied
output head.  Fixed by the reference's code rather than by configuration: the
score scale 1/sqrt(head_dim) (yalis/attention/backend_impl/sdpa_and_flex.py:71-73),
rotary over the whole head (yalis/external/model.py:563-565), no biases.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.reader import ConfigError, KeyReader
from ..config.registry import register_architecture
from ..config.specs import LayerSpec, ModelSpec, PartSpec, RunEntry


@dataclass(frozen=True)
class RopeScaling:
    """config.json ``rope_scaling`` of type llama3; the reference's
    ``rope_adjustments`` (yalis/external/model.py:207-252: all four or none)."""

    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    rope_scaling: Optional[RopeScaling]
    eos_token_ids: Tuple[int, ...]
    torch_dtype: str

    @classmethod
    def from_dict(cls, raw: Dict[str, Any], strict: bool = False) -> "LlamaConfig":
        r = KeyReader(raw)
        hidden = r.integer("hidden_size", minimum=1)
        layers = r.integer("num_hidden_layers", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        # yalis/external/config.py:121-125: groups default to the head count
        kv_heads = r.integer("num_key_value_heads", default=heads, minimum=1)
        if heads % kv_heads != 0:
            raise ConfigError(
                f"config.json: num_attention_heads={heads} is not a multiple of num_key_value_heads={kv_heads}"
            )
        # yalis/external/config.py:108-110: head size defaults to hidden / heads
        head_dim = r.integer("head_dim", default=None, minimum=1)
        if head_dim is None:
            if hidden % heads != 0:
                raise ConfigError(
                    f"config.json: hidden_size={hidden} is not a multiple of num_attention_heads={heads} and no head_dim is given"
                )
            head_dim = hidden // heads
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim={head_dim} must be even for rotary pairs")
        inter = r.integer("intermediate_size", minimum=1)
        vocab = r.integer("vocab_size", minimum=1)
        eps = r.number("rms_norm_eps", positive=True)
        theta = r.number("rope_theta", default=10000.0, positive=True)
        max_pos = r.integer("max_position_embeddings", minimum=1)
        tied = r.boolean("tie_word_embeddings", default=False)
        r.require_value("hidden_act", ["silu"], default="silu")
        r.require_value("attention_bias", [False], default=False)
        r.require_value("mlp_bias", [False], default=False)
        r.require_value("sliding_window", [None], default=None)

        scaling = None
        rs = r.mapping("rope_scaling", default=None)
        if rs is not None:
            sr = KeyReader(rs, where="config.json rope_scaling")
            kind = sr.raw_value("rope_type", None) or sr.raw_value("type", None) or "default"
            sr.taken.update({"rope_type", "type"})
            if kind == "llama3":
                scaling = RopeScaling(
                    factor=sr.number("factor", positive=True),
                    low_freq_factor=sr.number("low_freq_factor"),
                    high_freq_factor=sr.number("high_freq_factor"),
                    original_max_position_embeddings=sr.integer(
                        "original_max_position_embeddings", minimum=1
                    ),
                )
                if scaling.high_freq_factor == scaling.low_freq_factor:
                    raise ConfigError(
                        "config.json rope_scaling: high_freq_factor must differ from low_freq_factor"
                    )
            elif kind != "default":
                raise ConfigError(
                    f"config.json rope_scaling: rope_type {kind!r} is not supported (supported: 'llama3', 'default')"
                )
            sr.finish(strict=True)

        eos = r.raw_value("eos_token_id", None)
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, list) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"config.json: 'eos_token_id' must be an integer or a list of them, got {eos!r}")
        dtype = raw.get("torch_dtype") or raw.get("dtype") or "bfloat16"
        r.finish(harmless=("rope_interleaved",), strict=strict)
        return cls(
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=inter,
            vocab_size=vocab,
            rms_norm_eps=eps,
            rope_theta=theta,
            max_position_embeddings=max_pos,
            tie_word_embeddings=tied,
            rope_scaling=scaling,
            eos_token_ids=eos_ids,
            torch_dtype=str(dtype),
        )

    def to_dict(self) -> Dict[str, Any]:
        """The config.json that reads back as this configuration."""
        d: Dict[str, Any] = {
            "architectures": [ARCHITECTURE_NAME],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
            "rope_scaling": None,
        }
        if self.rope_scaling is not None:
            d["rope_scaling"] = {"rope_type": "llama3", **asdict(self.rope_scaling)}
        if self.eos_token_ids:
            d["eos_token_id"] = (
                self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
            )
        return d


ARCHITECTURE_NAME = "LlamaForCausalLM"


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    """The model as parts.  Tensor names are the checkpoint's own
    (the reference renames them offline, yalis/external/convert_hf_checkpoint.py:705-736;
    here they are read as they are)."""
    rotary = PartSpec(
        "rotary",
        {
            "rotary_dim": cfg.head_dim,
            "theta": cfg.rope_theta,
            "pairing": "half",
            "scaling": None if cfg.rope_scaling is None else {"kind": "llama3", **asdict(cfg.rope_scaling)},
        },
    )

    def norm(name: str) -> PartSpec:
        return PartSpec(
            "rmsnorm",
            {"name": name, "size": cfg.hidden_size, "eps": cfg.rms_norm_eps, "unit_offset": False},
        )

    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}"
        mixer = PartSpec(
            "attention",
            {
                "prefix": f"{p}.self_attn",
                "hidden_size": cfg.hidden_size,
                "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads,
                "head_dim": cfg.head_dim,
                "scale": 1.0 / math.sqrt(cfg.head_dim),
                "window": None,
                "position": rotary,
            },
        )
        ffn = PartSpec(
            "gated_mlp",
            {
                "prefix": f"{p}.mlp",
                "hidden_size": cfg.hidden_size,
                "intermediate_size": cfg.intermediate_size,
                "activation": "silu",
            },
        )
        layers.append(
            LayerSpec.of(
                p,
                "prenorm",
                mixer_norm=norm(f"{p}.input_layernorm.weight"),
                mixer=mixer,
                feed_forward_norm=norm(f"{p}.post_attention_layernorm.weight"),
                feed_forward=ffn,
            )
        )
    spec = ModelSpec(
        architecture=ARCHITECTURE_NAME,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings,
        embedding=PartSpec(
            "token_embedding",
            {"name": "model.embed_tokens.weight", "vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size},
        ),
        layers=tuple(layers),
        run_order=tuple(RunEntry(layer=i) for i in range(cfg.num_hidden_layers)),
        final_norm=norm("model.norm.weight"),
        head=PartSpec(
            "lm_head",
            {
                "name": "lm_head.weight",
                "tied_to": "model.embed_tokens.weight" if cfg.tie_word_embeddings else None,
                "vocab_size": cfg.vocab_size,
                "hidden_size": cfg.hidden_size,
            },
        ),
        eos_token_ids=cfg.eos_token_ids,
    )
    spec.validate()
    return spec


register_architecture(ARCHITECTURE_NAME, LlamaConfig, build_llama_spec)
