"""Interfaces of the parts a layer is made of, and the registries that map a part's
``kind`` to its class.

A part is built from a :class:`PartSpec` (its sizes and constants) and knows nothing of
the model it sits in. It declares the tensors it needs by full checkpoint name, is bound
to them once, and is then called by the step function with a :class:`StepContext` that
describes the batch. To add a part, subclass one of the four bases and register it:

* **Norm** - ``forward(x, ctx, row_index=None) -> h``: float32 rows in, activation dtype out.
* **PositionEncoding** - ``tables(ctx)``: whatever the mixer's kernels need for the rows of
  this step (computed once per step and shared by all layers with the same parameters).
* **Mixer** - ``cache_need()`` says what per-request memory it needs (paged keys/values, a
  fixed-size state, or nothing); ``forward(h, residual, ctx, cache)`` must ADD its output to
  ``residual`` (float32, in place).
* **FeedForward** - ``forward(h, residual, ctx)`` must ADD its output to ``residual``.

The reference keeps the same seams as per-layer flags and tensor slots of one plan
struct (native/src/v2_runtime.cpp:395-560,4177-4184).
"""

from __future__ import annotations

from typing import Callable, Dict, Mapping, Optional, Type

import torch

from ..config.spec import ConfigError, PartSpec
from ..weights.loader import TensorDecl


class Part:
    # True when ``forward`` only launches work on the current stream from device-side batch
    # data (no host reads of the batch, no synchronisation): a decode step made of such parts
    # may be captured in a HIP graph and replayed. Parts that look at ``ctx.host_*`` leave it False.
    graph_safe = False

    def __init__(self, spec: PartSpec):
        self.spec = spec
        self.prefix = spec.prefix

    def tensors(self) -> Dict[str, TensorDecl]:
        """Full checkpoint name -> declaration, for every tensor this part needs."""
        return {}

    def bind(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Take the loaded tensors (already on ``device``); ``dtype`` is the activation dtype."""
        self.dtype = dtype
        self.device = device

    # Index arrays of a part's own that its kernels need for every step (the tiles a kernel cuts
    # the rows into, the order it visits them in): built on the host from the batch, they travel
    # to the device in the step's one upload and are found again with ``ctx.step_arrays(part)``.
    def step_arrays_key(self):
        """None: the part needs none (the default). Parts with equal keys share one set."""
        return None

    def step_arrays(self, batch) -> Dict[str, "numpy.ndarray"]:
        """name -> int32 array, from ``batch.host_seg_row0`` (first row of each segment, and the
        end), ``batch.host_row_pos``, ``batch.host_seg_slot``, ``batch.decode_prefix``,
        ``batch.all_decode``, ``batch.num_rows``. For a recorded decode step this is asked once, for
        segments of one row each at position 0: it fixes the arrays' names and sizes, which may
        depend on the number of rows alone; what depends on positions or slots is then brought
        up to date by ``refresh_step_arrays`` before every replay."""
        return {}

    def refresh_step_arrays(self, batch, arrays: Dict[str, "numpy.ndarray"]) -> None:
        """For a recorded decode step, before each of its uploads: ``arrays`` are the host
        copies of what ``step_arrays`` returned (name -> int32 numpy array, to be changed in
        place), ``batch`` has this replay's ``host_row_pos`` and ``host_seg_slot``. When several
        steps run back to back on the device this is called before the first of them only.
        The default leaves the arrays as they were built."""


class Norm(Part):
    def forward(self, x: torch.Tensor, ctx, row_index: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def key(self):
        """Parts with equal keys share one set of per-step tables."""
        return (type(self).__name__, tuple(sorted((k, v) for k, v in self.spec.params.items())))

    def tables(self, ctx):
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        return None

    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx, cache):
        """Adds the mixer's output to ``residual`` in place. May return what its last product
        prepared for ``ctx.upcoming_norm`` (``Linear.accumulate(..., then=...)``); returning
        None is always right."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx):
        """Adds to ``residual`` in place; the return value is as for a mixer."""
        raise NotImplementedError


class Block:
    """The arrangement of parts in a layer. ``forward(x, ctx, cache, prepared, norm_after)``
    updates the float32 residual rows ``x`` in place. The model hands over what the layer before
    prepared for this block's ``first_norm()`` (``prepared``, may be None) and names the norm that
    reads the residual after this block (``norm_after``, may be None); the block returns what its
    last product prepared for that norm, or None. An arrangement that ignores both is right, only
    slower: the norms then run as kernels of their own."""

    graph_safe = False

    def parts(self):
        """Every part of the block (the model asks them for tensors and step arrays)."""
        return ()

    def first_norm(self):
        """The norm that reads the residual stream first in this block, if the block begins with
        one that a product before it may prepare; else None."""
        return None

    def tensors(self) -> Dict[str, TensorDecl]:
        declared: Dict[str, TensorDecl] = {}
        for part in self.parts():
            declared.update(part.tensors())
        return declared

    def bind(self, tensors, dtype, device) -> None:
        for part in self.parts():
            part.bind(tensors, dtype, device)

    def cache_need(self):
        return None

    def forward(self, x, ctx, cache, prepared=None, norm_after=None):
        raise NotImplementedError


_REGISTRIES: Dict[str, Dict[str, Type[Part]]] = {"norm": {}, "position": {}, "mixer": {}, "ffn": {}, "block": {}}


def _register(family: str, kind: str) -> Callable[[Type], Type]:
    def decorate(cls: Type) -> Type:
        _REGISTRIES[family][kind] = cls
        return cls
    return decorate


def register_norm(kind: str):
    return _register("norm", kind)


def register_position_encoding(kind: str):
    return _register("position", kind)


def register_mixer(kind: str):
    return _register("mixer", kind)


def register_feed_forward(kind: str):
    return _register("ffn", kind)


def register_block(kind: str):
    return _register("block", kind)


def build_part(family: str, spec: PartSpec):
    registry = _REGISTRIES[family]
    if spec.kind not in registry:
        raise ConfigError(f"unknown {family} kind '{spec.kind}'; registered: {', '.join(sorted(registry)) or 'none'}")
    return registry[spec.kind](spec)


def registered(family: str):
    return tuple(sorted(_REGISTRIES[family]))
