"""The generic causal language model: an embedding, layers run in the order the schedule
gives, a final norm and a head. It is built from a :class:`ModelSpec` alone; which classes
the layers are made of is decided by the parts registries."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..cache.needs import CacheView
from ..config import ModelSpec, load_config
from ..config.spec import ConfigError
from ..kernels import ops
from ..parts import Linear, build_part
from ..parts.norm import LazyNorm
from ..parts.base import _REGISTRIES
from ..weights.loader import TensorDecl, load_tensors

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine runs in float32 or bfloat16, not {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"unknown dtype '{name}'; choose bfloat16 or float32") from None


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.layers = []
        for layer in spec.layers:
            if layer.arrangement not in _REGISTRIES["block"]:
                raise ConfigError(f"unknown block arrangement '{layer.arrangement}'")
            self.layers.append(_REGISTRIES["block"][layer.arrangement](layer))
        self.final_norm = build_part("norm", spec.final_norm)
        self.bound = False

    # ----- tensors ----------------------------------------------------------------------
    def tensors(self) -> Dict[str, TensorDecl]:
        spec = self.spec
        declared: Dict[str, TensorDecl] = {spec.embedding_name: TensorDecl((spec.vocab_size, spec.hidden_size))}
        for block in self.layers:
            declared.update(block.tensors())
        declared.update(self.final_norm.tensors())
        if spec.lm_head_name is not None:
            declared[spec.lm_head_name] = TensorDecl((spec.vocab_size, spec.hidden_size))
        return declared

    def bind(self, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        self.dtype, self.device = dtype, device
        ops.prepare_device(device)
        self.embedding = tensors[self.spec.embedding_name]
        head = self.embedding if self.spec.lm_head_name is None else tensors[self.spec.lm_head_name]
        self.head = Linear(head)
        for block in self.layers:
            block.bind(tensors, dtype, device)
        self.final_norm.bind(tensors, dtype, device)
        self.bound = True

    # ----- cache ------------------------------------------------------------------------
    def cache_needs(self) -> Dict[int, object]:
        """Cache entry id -> what the mixer that writes it needs."""
        needs: Dict[int, object] = {}
        for entry in self.spec.schedule:
            need = self.layers[entry.layer].cache_need()
            if entry.cache is None:
                if need is not None:
                    raise ConfigError(f"layer {entry.layer} keeps state between steps but its schedule entry names no cache")
                continue
            if need is None:
                continue
            if entry.cache in needs and needs[entry.cache] != need:
                raise ConfigError(f"cache entry {entry.cache} is shared by layers with different needs")
            needs[entry.cache] = need
        return needs

    def step_array_providers(self) -> List:
        """The parts that ask for index arrays of their own in every step's upload
        (``Part.step_arrays``), one for each distinct key."""
        found: Dict = {}
        for block in self.layers:
            for part in block.parts():
                key = part.step_arrays_key()
                if key is not None:
                    found.setdefault(key, part)
        return list(found.values())

    # ----- forward ----------------------------------------------------------------------
    def forward(self, ctx, cache) -> Optional[torch.Tensor]:
        """Runs the rows of ``ctx`` through every scheduled layer; returns float32 logits
        [wanted, vocab] for ``ctx.want_rows`` (None when nothing is wanted)."""
        x = ops.embed_rows(self.embedding, ctx.token_ids, scale=self.spec.embedding_scale)
        schedule = self.spec.schedule
        # A step of single tokens: the final norm reads every row as it is, like a layer's first norm, so
        # the last layer's last product may prepare it; rows that nobody wants cost the head nothing
        # it would not read anyway, and are dropped behind it. (A recorded step computes every row too:
        # what it gives and what the launches give stay bit for bit the same.)
        every_row = bool(ctx.all_decode)
        prepared = None
        for at, entry in enumerate(schedule):
            # the norm that reads the residual after this layer, for the layer's last product
            if at + 1 < len(schedule):
                norm_after = self.layers[schedule[at + 1].layer].first_norm()
            else:
                norm_after = self.final_norm if every_row else None
            prepared = self.layers[entry.layer].forward(x, ctx, ctx.cache_view(cache, entry), prepared=prepared, norm_after=norm_after)
        if ctx.num_wanted == 0:
            return None
        final = LazyNorm(self.final_norm, x, ctx, prepared=prepared) if every_row else LazyNorm(self.final_norm, x, ctx, row_index=ctx.want_rows)
        logits = self.head.forward(final, out_dtype=torch.float32)
        if every_row and not getattr(ctx, "wants_every_row", False):
            logits = ops.gather_rows(logits, ctx.want_rows)
        if self.spec.logit_scale != 1.0 or self.spec.logit_softcap > 0.0:
            ops.scale_softcap_(logits, self.spec.logit_scale, self.spec.logit_softcap)
        return logits


def declared_tensors(spec: ModelSpec) -> Dict[str, TensorDecl]:
    return CausalLM(spec).tensors()


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """Model folder (config.json + safetensors) -> (config, bound CausalLM)."""
    dtype = parse_dtype(dtype)
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("flyweight_amd runs on a GPU only (no CPU path); no HIP device is available")
    ops.library()       # fail now, and loudly, if the kernel library cannot be had
    config = load_config(model_dir)
    model = CausalLM(config.model_spec())
    tensors = load_tensors(model_dir, model.tensors(), dtype, device)
    model.bind(tensors, dtype, device)
    return config, model
