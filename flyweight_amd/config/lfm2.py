"""Typed configuration of LFM2 (``Lfm2ForCausalLM``), read from its config.json keys.

LFM2 is a hybrid of gated short-convolution blocks and grouped-query attention blocks
with a SwiGLU feed-forward in every block. The reference reads the same facts from GGUF
metadata (native/src/v2_runtime.cpp:2897-2899 ``.shortconv.l_cache``, :2992 the
per-layer KV-head array, :3195-3209 the LFM2 fix-ups) and builds its per-layer plan in
``build_lfm2_plan`` (native/src/v2_runtime.cpp:4164-4282). Here the keys are the ones the
architecture's own config.json spells.
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, asdict
from typing import Any, Dict, List, Mapping, Optional, Tuple

from . import json_reader
from .spec import (ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry,
                   default_schedule)

_ATTENTION_NAMES = ("full_attention", "attn", "attention")
_CONV_NAMES = ("conv", "short_conv", "shortconv")

_REQUIRED = (
    "vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
    "num_key_value_heads", "max_position_embeddings",
)
# Keys that may be absent, and what stands for them then. rope_theta: the reference's default
# (native/src/v2_runtime.cpp:4235); norm_eps: what its LFM2 fixture writes
# (tests/lfm2_gguf_fixture.py:243); conv_L_cache: the width every LFM2 shape named here has.
# Further: conv_bias false, tie_word_embeddings true, block_auto_adjust_ff_dim false.
DEFAULTS = {"norm_eps": 1e-5, "rope_theta": 1000000.0, "conv_L_cache": 3}


def _need(data: Mapping[str, Any], key: str) -> Any:
    if key not in data or data[key] is None:
        raise ConfigError(f"config.json is missing '{key}'")
    return data[key]


def _as_int(data: Mapping[str, Any], key: str) -> int:
    value = _need(data, key)
    if isinstance(value, bool) or not isinstance(value, int):
        if isinstance(value, float) and value.is_integer():
            return int(value)
        raise ConfigError(f"config.json key '{key}' must be an integer, found {value!r}")
    return value


def _with_defaults(data: Mapping[str, Any]) -> Dict[str, Any]:
    """The keys with their documented defaults filled in, and the feed-forward width under its
    one name: ``block_ff_dim`` is the architecture's original spelling of ``intermediate_size``."""
    filled = dict(data)
    for key, value in DEFAULTS.items():
        if filled.get(key) is None:
            filled[key] = value
    width, original = filled.get("intermediate_size"), filled.get("block_ff_dim")
    if width is not None and original is not None and width != original:
        raise ConfigError(f"'intermediate_size' ({width}) and 'block_ff_dim' ({original}) disagree")
    if width is None:
        if original is None:
            raise ConfigError("config.json is missing 'intermediate_size' (or 'block_ff_dim')")
        filled["intermediate_size"] = original
    return filled


def _as_float(data: Mapping[str, Any], key: str) -> float:
    value = _need(data, key)
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"config.json key '{key}' must be a number, found {value!r}")
    return float(value)


def _as_bool(data: Mapping[str, Any], key: str, default: bool) -> bool:
    value = data.get(key, None)
    if value is None:
        return default
    if not isinstance(value, bool):
        raise ConfigError(f"config.json key '{key}' must be true or false, found {value!r}")
    return value


@dataclass(frozen=True)
class Lfm2Config:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    intermediate_size: int
    norm_eps: float
    rope_theta: float
    conv_L_cache: int
    max_position_embeddings: int
    layer_types: Tuple[str, ...]                 # "conv" | "full_attention", one per block
    conv_bias: bool = False
    tie_word_embeddings: bool = True
    block_auto_adjust_ff_dim: bool = False
    block_ffn_dim_multiplier: Optional[float] = None
    block_multiple_of: Optional[int] = None
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None

    architecture = "Lfm2ForCausalLM"
    model_type = "lfm2"

    # ----- derived sizes ---------------------------------------------------------------
    @property
    def head_dim(self) -> int:
        # hidden/heads, as the reference fixes it (native/src/v2_runtime.cpp:4222)
        return self.hidden_size // self.num_attention_heads

    @property
    def ff_dim(self) -> int:
        """Effective SwiGLU width. With ``block_auto_adjust_ff_dim`` the configured
        width is taken to two thirds, scaled by ``block_ffn_dim_multiplier`` and
        rounded up to a multiple of ``block_multiple_of``; otherwise it is
        ``intermediate_size`` itself. (The reference reads the effective width off
        the gate tensor's shape, native/src/v2_runtime.cpp:3527-3534.)"""
        if not self.block_auto_adjust_ff_dim:
            return self.intermediate_size
        width = int(2 * self.intermediate_size / 3)
        if self.block_ffn_dim_multiplier is not None:
            width = int(self.block_ffn_dim_multiplier * width)
        multiple = self.block_multiple_of
        return multiple * ((width + multiple - 1) // multiple)

    @property
    def full_attn_idxs(self) -> Tuple[int, ...]:
        return tuple(i for i, kind in enumerate(self.layer_types) if kind == "full_attention")

    def is_attention(self, layer: int) -> bool:
        return self.layer_types[layer] == "full_attention"

    # ----- validation ------------------------------------------------------------------
    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                    "num_key_value_heads", "intermediate_size", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json key '{key}' must be positive, found {getattr(self, key)}")
        if self.hidden_size % self.num_attention_heads:
            raise ConfigError(
                f"hidden_size {self.hidden_size} is not a multiple of num_attention_heads "
                f"{self.num_attention_heads}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim {self.head_dim} must be even for rotary pairs")
        if self.conv_L_cache < 2:
            # the reference refuses l_cache < 2 (native/src/v2_runtime.cpp:3205-3207)
            raise ConfigError(f"conv_L_cache must be at least 2, found {self.conv_L_cache}")
        if not (self.norm_eps > 0 and math.isfinite(self.norm_eps)):
            raise ConfigError(f"norm_eps must be a positive number, found {self.norm_eps}")
        if not (self.rope_theta > 0 and math.isfinite(self.rope_theta)):
            raise ConfigError(f"rope_theta must be a positive number, found {self.rope_theta}")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(
                f"layer_types names {len(self.layer_types)} blocks but num_hidden_layers is "
                f"{self.num_hidden_layers}")
        if self.block_auto_adjust_ff_dim:
            if self.block_multiple_of is None or self.block_multiple_of <= 0:
                raise ConfigError("block_auto_adjust_ff_dim needs a positive 'block_multiple_of'")
            if self.block_ffn_dim_multiplier is not None and not self.block_ffn_dim_multiplier > 0:
                raise ConfigError("'block_ffn_dim_multiplier' must be positive")
        if self.ff_dim <= 0:
            raise ConfigError("effective feed-forward width is not positive")

    # ----- reading and writing ---------------------------------------------------------
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "Lfm2Config":
        if not isinstance(data, Mapping):
            raise ConfigError("config.json must hold a JSON object")
        for key in _REQUIRED:
            _need(data, key)
        data = _with_defaults(data)
        layers = _as_int(data, "num_hidden_layers")
        layer_types = _layer_types(data, layers)
        tie = _tie(data)
        multiplier = data.get("block_ffn_dim_multiplier")
        if multiplier is not None:
            multiplier = _as_float(data, "block_ffn_dim_multiplier")
        multiple = data.get("block_multiple_of")
        if multiple is not None:
            multiple = _as_int(data, "block_multiple_of")
        config = cls(
            vocab_size=_as_int(data, "vocab_size"),
            hidden_size=_as_int(data, "hidden_size"),
            num_hidden_layers=layers,
            num_attention_heads=_as_int(data, "num_attention_heads"),
            num_key_value_heads=_as_int(data, "num_key_value_heads"),
            intermediate_size=_as_int(data, "intermediate_size"),
            norm_eps=_as_float(data, "norm_eps"),
            rope_theta=_as_float(data, "rope_theta"),
            conv_L_cache=_as_int(data, "conv_L_cache"),
            max_position_embeddings=_as_int(data, "max_position_embeddings"),
            layer_types=layer_types,
            conv_bias=_as_bool(data, "conv_bias", False),
            tie_word_embeddings=tie,
            block_auto_adjust_ff_dim=_as_bool(data, "block_auto_adjust_ff_dim", False),
            block_ffn_dim_multiplier=multiplier,
            block_multiple_of=multiple,
            bos_token_id=_optional_id(data, "bos_token_id"),
            eos_token_id=_optional_id(data, "eos_token_id"),
        )
        config.validate()
        return config

    @classmethod
    def from_json_file(cls, path: str) -> "Lfm2Config":
        try:
            data = json_reader.parse_file(path)
        except json_reader.JsonError as error:
            raise ConfigError(f"{path}: {error}") from None
        return cls.from_dict(data)

    def to_dict(self) -> Dict[str, Any]:
        data = asdict(self)
        data["layer_types"] = list(self.layer_types)
        data["full_attn_idxs"] = list(self.full_attn_idxs)
        data["architectures"] = [self.architecture]
        data["model_type"] = self.model_type
        return {key: value for key, value in data.items() if value is not None}

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as handle:
            json.dump(self.to_dict(), handle, indent=2)

    # ----- lowering to parts -----------------------------------------------------------
    def model_spec(self) -> ModelSpec:
        """The list of layers, part by part, with every size as a parameter.

        Tensor names follow the architecture's checkpoint layout; the same tensors
        under the reference's GGUF names are listed in tests/lfm2_gguf_fixture.py:139-167
        of the reference."""
        hidden = self.hidden_size
        norm = {"eps": self.norm_eps, "size": hidden}
        layers: List[LayerSpec] = []
        for index in range(self.num_hidden_layers):
            base = f"model.layers.{index}."
            if self.is_attention(index):
                mixer = PartSpec("gqa_attention", {
                    "hidden_size": hidden,
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    "qk_norm": True,
                    "qk_norm_eps": self.norm_eps,
                    "window": None,
                    "softmax_scale": 1.0 / math.sqrt(self.head_dim),
                    "position": PartSpec("rotary_neox", {
                        "theta": self.rope_theta,
                        "rotary_dim": self.head_dim,
                        "head_dim": self.head_dim,
                    }),
                    "names": {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "out_proj",
                              "q_norm": "q_layernorm", "k_norm": "k_layernorm"},
                }, prefix=base + "self_attn.")
            else:
                mixer = PartSpec("short_conv", {
                    "hidden_size": hidden,
                    "kernel_size": self.conv_L_cache,
                    "bias": self.conv_bias,
                }, prefix=base + "conv.")
            layers.append(LayerSpec(
                arrangement="pre_norm_residual",
                mixer_norm=PartSpec("rmsnorm", norm, prefix=base + "operator_norm."),
                mixer=mixer,
                ffn_norm=PartSpec("rmsnorm", norm, prefix=base + "ffn_norm."),
                ffn=PartSpec("swiglu", {
                    "hidden_size": hidden,
                    "intermediate_size": self.ff_dim,
                    "names": {"gate": "w1", "up": "w3", "down": "w2"},
                }, prefix=base + "feed_forward."),
            ))
        spec = ModelSpec(
            architecture=self.architecture,
            hidden_size=hidden,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            layers=tuple(layers),
            schedule=default_schedule(self.num_hidden_layers),
            final_norm=PartSpec("rmsnorm", norm, prefix="model.embedding_norm."),
            embedding_name="model.embed_tokens.weight",
            lm_head_name=None if self.tie_word_embeddings else "lm_head.weight",
            bos_token_id=self.bos_token_id,
            eos_token_id=self.eos_token_id,
        )
        spec.validate()
        return spec


def _optional_id(data: Mapping[str, Any], key: str) -> Optional[int]:
    value = data.get(key)
    if value is None:
        return None
    if isinstance(value, list):     # some checkpoints list several end tokens
        value = value[0] if value else None
    if value is None:
        return None
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json key '{key}' must be an integer, found {value!r}")
    return value


def _tie(data: Mapping[str, Any]) -> bool:
    values = {key: data[key] for key in ("tie_word_embeddings", "tie_embedding")
              if data.get(key) is not None}
    for key, value in values.items():
        if not isinstance(value, bool):
            raise ConfigError(f"config.json key '{key}' must be true or false, found {value!r}")
    if len(set(values.values())) > 1:
        raise ConfigError("'tie_word_embeddings' and 'tie_embedding' disagree")
    return next(iter(values.values())) if values else True


def _layer_types(data: Mapping[str, Any], layers: int) -> Tuple[str, ...]:
    """Block kinds from ``layer_types`` (one name per block) or ``full_attn_idxs``
    (indices of the attention blocks; every other block is a short convolution).
    The reference classifies a block by which tensors it carries and demands the
    KV-head array agree (native/src/v2_runtime.cpp:4203-4209); with both keys present
    the two must agree here as well."""
    names = data.get("layer_types")
    idxs = data.get("full_attn_idxs")
    if names is None and idxs is None:
        raise ConfigError("config.json is missing 'layer_types' (or 'full_attn_idxs')")
    from_names = None
    if names is not None:
        if not isinstance(names, list):
            raise ConfigError("'layer_types' must be a list of block kinds")
        resolved = []
        for index, name in enumerate(names):
            if name in _ATTENTION_NAMES:
                resolved.append("full_attention")
            elif name in _CONV_NAMES:
                resolved.append("conv")
            else:
                raise ConfigError(
                    f"layer_types[{index}] is {name!r}; known kinds are 'conv' and 'full_attention'")
        from_names = tuple(resolved)
        if len(from_names) != layers:
            raise ConfigError(
                f"layer_types names {len(from_names)} blocks but num_hidden_layers is {layers}")
    from_idxs = None
    if idxs is not None:
        if not isinstance(idxs, list) or any(isinstance(i, bool) or not isinstance(i, int) for i in idxs):
            raise ConfigError("'full_attn_idxs' must be a list of block indices")
        for i in idxs:
            if not 0 <= i < layers:
                raise ConfigError(f"full_attn_idxs holds {i}, outside 0..{layers - 1}")
        if len(set(idxs)) != len(idxs):
            raise ConfigError("'full_attn_idxs' names a block twice")
        chosen = set(idxs)
        from_idxs = tuple("full_attention" if i in chosen else "conv" for i in range(layers))
    if from_names is not None and from_idxs is not None and from_names != from_idxs:
        raise ConfigError("'layer_types' and 'full_attn_idxs' disagree about which blocks are attention")
    return from_names if from_names is not None else from_idxs
