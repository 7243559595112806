"""Architecture-independent description of a causal language model.

An architecture's config class (for example :class:`Lfm2Config`) reads its own
``config.json`` keys and lowers them to a :class:`ModelSpec`: a list of layers, each
assembled from parts (norm, mixer, feed-forward, position encoding) that carry every
size and constant as a parameter, and a *schedule*, the order in which layers run.
Nothing below this file looks at an architecture name.

The reference keeps the same information in one flat ``ModelConfig`` plus a per-layer
``QwenLayerPlan`` (native/include/flyweight_v2_config.hpp:6-167,
native/src/v2_runtime.cpp:395-560); here the per-layer plan *is* the description.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the offending key."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: ``kind`` selects the class from the parts registry,
    ``params`` are its sizes and constants, ``prefix`` is where its tensors live in
    the checkpoint (for example ``model.layers.3.self_attn.``)."""

    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)
    prefix: str = ""

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)

    def __getitem__(self, key: str) -> Any:
        try:
            return self.params[key]
        except KeyError:
            raise ConfigError(f"part '{self.kind}' at '{self.prefix}' needs parameter '{key}'") from None


@dataclass(frozen=True)
class LayerSpec:
    """A residual block: which arrangement, and the four parts it is made of."""

    arrangement: str            # key into the block registry, e.g. "pre_norm_residual"
    mixer_norm: PartSpec
    mixer: PartSpec
    ffn_norm: PartSpec
    ffn: PartSpec


@dataclass(frozen=True)
class ScheduleEntry:
    """One execution of a layer.

    ``layer`` indexes ``ModelSpec.layers``. ``cache`` names the cache entry the
    mixer uses during this execution; two entries with the same ``cache`` share
    keys/values or state, and only the one with ``writes_cache`` appends to it.
    A layer may be named by several entries (it then runs several times with the
    same weights)."""

    layer: int
    cache: Optional[int] = None
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    embedding_name: str
    lm_head_name: Optional[str]     # None: the head is the embedding table (tied)
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    # What some architectures put around the layers: a factor on the embedding rows, a factor on
    # the logits, a soft cap c on them (c * tanh(logits / c), after the factor; 0: none).
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0

    def validate(self) -> None:
        if self.hidden_size <= 0 or self.vocab_size <= 0:
            raise ConfigError("hidden_size and vocab_size must be positive")
        if self.logit_softcap < 0:
            raise ConfigError("logit_softcap must not be negative (0 switches it off)")
        if not self.layers or not self.schedule:
            raise ConfigError("a model needs at least one layer and one schedule entry")
        writers = {}
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ConfigError(f"schedule[{index}] names layer {entry.layer}, "
                                  f"but there are {len(self.layers)} layers")
            if entry.cache is not None and entry.writes_cache:
                if entry.cache in writers:
                    raise ConfigError(
                        f"cache entry {entry.cache} is written by schedule[{writers[entry.cache]}] "
                        f"and schedule[{index}]; only one may write it")
                writers[entry.cache] = index
        for index, entry in enumerate(self.schedule):
            if entry.cache is not None and not entry.writes_cache:
                if entry.cache not in writers or writers[entry.cache] > index:
                    raise ConfigError(
                        f"schedule[{index}] reads cache entry {entry.cache} before anything wrote it")


def default_schedule(num_layers: int) -> Tuple[ScheduleEntry, ...]:
    """Every layer once, in order, each with a cache entry of its own."""
    return tuple(ScheduleEntry(layer=i, cache=i) for i in range(num_layers))
