"""Weights by tensor name.

Every part declares the tensors it needs (name, shape, role); the loader resolves them
in the checkpoint and reports everything that is wrong in ONE error: tensors that are
missing, tensors nobody asked for, and tensors of the wrong shape. The reference raises
on the first missing name (native/src/v2_runtime.cpp:3352-3357) and on the first
unmapped one (native/include/flyweight_v2_hf.hpp:1453-1456).

Storage rule: a matrix keeps the precision it is stored in (bfloat16 stays bfloat16, a
32-bit tensor stays 32-bit; float16 is rounded to the run's dtype); integer tables become
int32; small vectors (norm weights, biases, convolution taps) are widened to float32,
which is exact. A float32 run widens everything to float32.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFile, checkpoint_files


@dataclass(frozen=True)
class TensorDecl:
    """A tensor a part needs. ``role``: ``matrix`` (operand of a matrix product or an
    embedding table), ``vector`` (norm weight, bias, taps) or ``table`` (integers).
    ``init`` names the distribution the random-weights mode draws it from."""

    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "matrix"        # matrix | norm | conv | bias | zeros


class WeightError(ValueError):
    """Missing, unexpected and mis-shaped tensors of a checkpoint, all in one message."""

    def __init__(self, missing, unexpected, wrong_shape, where: str = ""):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        lines = [f"checkpoint {where} does not match the model:" if where
                 else "checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{name} expected {list(want)} found {list(found)}"
                for name, want, found in self.wrong_shape))
        super().__init__("\n".join(lines))


def storage_dtype(role: str, stored: torch.dtype, run_dtype: torch.dtype) -> torch.dtype:
    if role == "table":
        return torch.int32
    if role == "vector" or run_dtype == torch.float32:
        return torch.float32
    if stored == torch.float32:
        return torch.float32
    return run_dtype


def check_names(declared: Mapping[str, TensorDecl], found: Mapping[str, Tuple[int, ...]],
                where: str = "") -> None:
    missing = [name for name in declared if name not in found]
    unexpected = [name for name in found if name not in declared]
    wrong = [(name, declared[name].shape, found[name]) for name in declared
             if name in found and tuple(found[name]) != tuple(declared[name].shape)]
    if missing or unexpected or wrong:
        raise WeightError(missing, unexpected, wrong, where)


def load_tensors(model_dir: str, declared: Mapping[str, TensorDecl], run_dtype: torch.dtype,
                 device: torch.device) -> Dict[str, torch.Tensor]:
    files = [SafetensorsFile(path) for path in checkpoint_files(model_dir)]
    try:
        owner: Dict[str, SafetensorsFile] = {}
        shapes: Dict[str, Tuple[int, ...]] = {}
        for handle in files:
            for name, entry in handle.entries.items():
                owner[name] = handle
                shapes[name] = entry.shape
        check_names(declared, shapes, where=model_dir)
        tensors: Dict[str, torch.Tensor] = {}
        for name, decl in declared.items():
            host = owner[name].tensor(name)
            if decl.role == "table":
                if host.dtype not in (torch.int32, torch.int64):
                    raise WeightError([], [], [], where=f"{model_dir}: '{name}' must hold integers")
            elif not host.dtype.is_floating_point:
                raise ValueError(f"{model_dir}: tensor '{name}' holds integers where numbers are expected")
            target = storage_dtype(decl.role, host.dtype, run_dtype)
            tensors[name] = host.to(dtype=target).to(device=device).contiguous()
        return tensors
    finally:
        for handle in files:
            handle.close()
