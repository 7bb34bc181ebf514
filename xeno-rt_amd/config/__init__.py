"""Typed model configuration read from config.json, and the architecture registry.

The reference reads the same numbers from GGUF metadata
(crates/xrt-models/src/llama.rs:24-137); here they come from the keys that a
Llama / Qwen3 checkpoint folder carries in config.json. An architecture is
registered once under the name found in `architectures[0]`, with the class that
parses its configuration and the function that builds its model from parts.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Callable, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that is missing a key, or whose numbers do not fit together."""


def _require(raw: dict, key: str):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json: missing required key '{key}'")
    return raw[key]


def _positive_int(raw: dict, key: str) -> int:
    value = _require(raw, key)
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ConfigError(f"config.json: '{key}' must be a positive integer, found {value!r}")
    return value


@dataclass(frozen=True)
class LlamaConfig:
    """Sizes and constants of the Llama / Qwen3 dense decoder.

    Field for field the reference's LlamaConfig (llama.rs:24-39); the
    defaults of absent keys are the reference's (llama.rs:68-70, 95-102).
    """

    architecture: str
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
    qk_norm: bool
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    torch_dtype: str = "bfloat16"
    rope_dim: int = 0            # dims of a head that are rotated, the first ones (llama.rs:92-94); 0: the whole head
    rope_scale: float = 1.0      # what a position is multiplied by before it becomes an angle (llama.rs:103-106, rope.rs:25)

    def __post_init__(self):
        if self.rope_dim == 0:
            object.__setattr__(self, "rope_dim", self.head_dim)

    # Architectures that this class parses, and whether each norms q and k per head.
    QK_NORM_BY_ARCHITECTURE = {"LlamaForCausalLM": False, "Qwen3ForCausalLM": True}
    # what checkpoint folders of these architectures carry under `model_type`
    MODEL_TYPE_BY_ARCHITECTURE = {"LlamaForCausalLM": "llama", "Qwen3ForCausalLM": "qwen3"}

    @property
    def q_width(self) -> int:            # llama.rs:130-132
        return self.num_attention_heads * self.head_dim

    @property
    def kv_width(self) -> int:           # llama.rs:134-136
        return self.num_key_value_heads * self.head_dim

    @classmethod
    def from_dict(cls, raw: dict) -> "LlamaConfig":
        architectures = _require(raw, "architectures")
        if not isinstance(architectures, list) or not architectures:
            raise ConfigError("config.json: 'architectures' must be a non-empty list")
        architecture = architectures[0]
        if architecture not in cls.QK_NORM_BY_ARCHITECTURE:
            raise ConfigError(
                f"LlamaConfig parses {sorted(cls.QK_NORM_BY_ARCHITECTURE)}, found {architecture}")

        hidden = _positive_int(raw, "hidden_size")
        heads = _positive_int(raw, "num_attention_heads")            # llama.rs:71-75
        kv_heads = raw.get("num_key_value_heads")
        if kv_heads is None:
            kv_heads = heads                                          # llama.rs:68-70
        if isinstance(kv_heads, bool) or not isinstance(kv_heads, int) or kv_heads <= 0:
            raise ConfigError("config.json: attention head counts must be non-zero")
        if hidden % heads != 0:                                       # llama.rs:76-80
            raise ConfigError(
                f"config.json: hidden_size {hidden} is not divisible by num_attention_heads {heads}")
        if heads % kv_heads != 0:                                     # llama.rs:81-85
            raise ConfigError(
                f"config.json: num_attention_heads {heads} is not divisible by "
                f"num_key_value_heads {kv_heads}")
        head_dim = raw.get("head_dim")
        if head_dim is None:
            head_dim = hidden // heads                                # llama.rs:125-128
        if isinstance(head_dim, bool) or not isinstance(head_dim, int) or head_dim <= 0:
            raise ConfigError(f"config.json: 'head_dim' must be a positive integer, found {head_dim!r}")
        if head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even (rotary pairs)")

        model_type = raw.get("model_type")
        if model_type is not None and model_type != cls.MODEL_TYPE_BY_ARCHITECTURE[architecture]:
            raise ConfigError(f"config.json: model_type {model_type!r} does not belong to {architecture}")
        # The rotation's options. The reference has two beside the base: how many dims of a head are rotated
        # (llama.rs:92-94) and a number that multiplies every position (llama.rs:103-106, rope.rs:25: GGUF's
        # `rope.scale_linear`). In config.json these are `partial_rotary_factor` (a share of the head) and a linear
        # `rope_scaling` whose `factor` divides the positions, so the multiplier is 1 / factor. Newer folders carry all
        # of it, with the base, inside `rope_parameters`. Every other scaling rule is refused, never ignored.
        rope_scale, rotary_share = 1.0, raw.get("partial_rotary_factor")

        def linear_factor(rule: dict, where: str) -> float:
            kind = rule.get("rope_type", rule.get("type"))
            unknown = sorted(set(rule) - {"rope_type", "type", "factor", "rope_theta", "partial_rotary_factor"})
            if unknown:
                raise ConfigError(f"config.json: '{where}' has keys that are not supported: {unknown}")
            if kind in (None, "default"):
                if rule.get("factor") not in (None, 1, 1.0):
                    raise ConfigError(f"config.json: '{where}' has a factor without a rule (rope_type 'linear')")
                return 1.0
            if kind != "linear":
                raise ConfigError(f"config.json: rope_type {kind!r} is not supported (only 'default' and 'linear')")
            factor = rule.get("factor")
            if isinstance(factor, bool) or not isinstance(factor, (int, float)) or not factor > 0:
                raise ConfigError(f"config.json: '{where}' of type 'linear' needs a positive 'factor', found {factor!r}")
            return 1.0 / float(factor)

        rope_scaling = raw.get("rope_scaling")
        if rope_scaling not in (None, {}):
            if not isinstance(rope_scaling, dict):
                raise ConfigError("config.json: 'rope_scaling' must be an object or null")
            if "rope_theta" in rope_scaling or "partial_rotary_factor" in rope_scaling:
                raise ConfigError("config.json: 'rope_scaling' holds the rule and its factor only")
            rope_scale = linear_factor(rope_scaling, "rope_scaling")
        rope_parameters = raw.get("rope_parameters")
        if rope_parameters is not None:
            if not isinstance(rope_parameters, dict):
                raise ConfigError("config.json: 'rope_parameters' must be an object")
            inner_scale = linear_factor(rope_parameters, "rope_parameters")
            if rope_scaling not in (None, {}) and inner_scale != rope_scale:
                raise ConfigError("config.json: 'rope_scaling' and 'rope_parameters' disagree")
            rope_scale = inner_scale
            inner = rope_parameters.get("rope_theta")
            if inner is not None:
                if raw.get("rope_theta") is not None and float(raw["rope_theta"]) != float(inner):
                    raise ConfigError("config.json: 'rope_theta' and 'rope_parameters.rope_theta' disagree")
                raw = dict(raw, rope_theta=inner)
            inner_share = rope_parameters.get("partial_rotary_factor")
            if inner_share is not None:
                if rotary_share is not None and float(rotary_share) != float(inner_share):
                    raise ConfigError("config.json: 'partial_rotary_factor' and 'rope_parameters.partial_rotary_factor' disagree")
                rotary_share = inner_share
        rope_dim = head_dim
        if rotary_share is not None:
            if isinstance(rotary_share, bool) or not isinstance(rotary_share, (int, float)) or not 0 < rotary_share <= 1:
                raise ConfigError(f"config.json: 'partial_rotary_factor' must lie in (0, 1], found {rotary_share!r}")
            rope_dim = int(head_dim * float(rotary_share))
            if rope_dim < 2 or rope_dim % 2 != 0:
                raise ConfigError(f"config.json: partial_rotary_factor {rotary_share} of head_dim {head_dim} gives {rope_dim} "
                                  "rotated dims; an even number, two at least, is needed (rotary pairs)")
        activation = raw.get("hidden_act", "silu")
        if activation != "silu":
            raise ConfigError(f"config.json: hidden_act must be 'silu', found {activation!r}")
        for key in ("attention_bias", "mlp_bias"):
            if raw.get(key):
                raise ConfigError(f"config.json: '{key}' must be false or absent (the decoder has no biases)")
        if raw.get("use_sliding_window"):
            raise ConfigError("config.json: 'use_sliding_window' must be false or absent")

        eos = raw.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        bos = raw.get("bos_token_id")
        vocab = _positive_int(raw, "vocab_size")
        for token in eos_ids + (() if bos is None else (int(bos),)):
            if not 0 <= token < vocab:
                raise ConfigError(f"config.json: special token id {token} is outside the vocabulary {vocab}")

        eps = float(raw.get("rms_norm_eps", 1e-5))                    # llama.rs:95-98
        theta = float(raw.get("rope_theta", 10000.0))                 # llama.rs:99-102
        if not eps > 0.0:
            raise ConfigError(f"config.json: rms_norm_eps must be positive, found {eps}")
        if not theta > 0.0:
            raise ConfigError(f"config.json: rope_theta must be positive, found {theta}")

        return cls(
            architecture=architecture,
            vocab_size=vocab,
            hidden_size=hidden,
            intermediate_size=_positive_int(raw, "intermediate_size"),
            num_hidden_layers=_positive_int(raw, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=eps,
            rope_theta=theta,
            max_position_embeddings=_positive_int(raw, "max_position_embeddings"),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            qk_norm=cls.QK_NORM_BY_ARCHITECTURE[architecture],
            eos_token_ids=eos_ids,
            bos_token_id=None if bos is None else int(bos),
            torch_dtype=str(raw.get("torch_dtype", "bfloat16")),
            rope_dim=rope_dim,
            rope_scale=rope_scale,
        )

    def to_dict(self) -> dict:
        """The config.json that `from_dict` reads back to an equal object."""
        eos = list(self.eos_token_ids)
        return {
            "architectures": [self.architecture],
            "model_type": self.MODEL_TYPE_BY_ARCHITECTURE[self.architecture],
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "eos_token_id": None if not eos else (eos[0] if len(eos) == 1 else eos),
            "bos_token_id": self.bos_token_id,
            "torch_dtype": self.torch_dtype,
            **({} if self.rope_dim == self.head_dim else {"partial_rotary_factor": self.rope_dim / self.head_dim}),
            **({} if self.rope_scale == 1.0 else {"rope_scaling": {"rope_type": "linear", "factor": 1.0 / self.rope_scale}}),
        }


# ----------------------------------------------------------------------------
# registry: architecture name -> (configuration class, model builder)
# ----------------------------------------------------------------------------

@dataclass
class Architecture:
    name: str
    config_class: type
    build: Callable  # (config) -> models.ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build: Callable) -> None:
    """Make `name` (as in config.json's architectures[0]) known to the library.

    `config_class.from_dict(raw)` parses config.json; `build(config)` returns the
    description of the model in parts. Registering a name again replaces it.
    """
    _ARCHITECTURES[name] = Architecture(name, config_class, build)


def architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unsupported architecture '{name}'; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    # The built-in architectures register themselves when their module is imported.
    from ..models import llama  # noqa: F401


def parse_config(raw: dict):
    """config.json contents -> the typed configuration of its architecture."""
    architectures = raw.get("architectures")
    if not isinstance(architectures, list) or not architectures:
        raise ConfigError("config.json: 'architectures' must be a non-empty list")
    return architecture(architectures[0]).config_class.from_dict(raw)


def load_config(folder: str):
    """Read `folder/config.json`."""
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder}")
    with open(path) as handle:
        try:
            raw = json.load(handle)
        except json.JSONDecodeError as error:
            raise ConfigError(f"{path}: invalid JSON: {error}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return parse_config(raw)


def save_config(config, folder: str) -> None:
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(config.to_dict(), handle, indent=2)
        handle.write("\n")
