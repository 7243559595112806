"""Random weights: write a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference's native code has no such mode; its tests write random *files*
(tests/lfm2_gguf_fixture.py:120-167). Distributions here: matrices N(0, 0.02), norm
weights 1 + U(-0.1, 0.1), convolution taps N(0, 0.1), biases N(0, 0.01). Values are drawn
in float32 from one seeded generator in the order of the declared names, then matrices
are rounded to the storage dtype, so a float32 run and a bfloat16 run of the same folder
see identical values.
"""

from __future__ import annotations

import math
import os
from typing import Dict, Mapping

import torch

from .loader import TensorDecl
from .safetensors_io import write_file

_STD = {"matrix": 0.02, "conv": 0.1, "bias": 0.01}


def _std(decl: TensorDecl, scale: str) -> float:
    """``scale`` "small": the fixed widths above. "fan_in": every linear map keeps the size
    of what passes through it (matrices 1/sqrt(columns), taps 0.5, biases 0.1), so that each
    part of a layer contributes visibly to the output; meant for tests."""
    if scale == "small":
        return _STD[decl.init]
    if scale != "fan_in":
        raise ValueError(f"unknown scale '{scale}'")
    if decl.init == "matrix":
        return 1.0 / math.sqrt(decl.shape[-1])
    return {"conv": 0.5, "bias": 0.1}[decl.init]


def random_tensors(declared: Mapping[str, TensorDecl], seed: int,
                   matrix_dtype: torch.dtype = torch.bfloat16, scale: str = "small") -> Dict[str, torch.Tensor]:
    generator = torch.Generator(device="cpu")
    generator.manual_seed(int(seed))
    tensors: Dict[str, torch.Tensor] = {}
    for name in declared:
        decl = declared[name]
        if decl.role == "table":
            tensors[name] = torch.zeros(decl.shape, dtype=torch.int32)
            continue
        if decl.init == "norm":
            value = 1.0 + (torch.rand(decl.shape, generator=generator, dtype=torch.float32) * 0.2 - 0.1)
        elif decl.init == "zeros":
            value = torch.zeros(decl.shape, dtype=torch.float32)
        else:
            value = torch.randn(decl.shape, generator=generator, dtype=torch.float32) * _std(decl, scale)
        tensors[name] = value.to(matrix_dtype) if decl.role == "matrix" else value
    return tensors


def write_random_model(folder: str, config, seed: int,
                       matrix_dtype: torch.dtype = torch.bfloat16, scale: str = "small") -> str:
    """``config`` is a registered architecture's configuration object."""
    from ..engine.model import declared_tensors      # parts decide which tensors exist
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    declared = declared_tensors(config.model_spec())
    tensors = random_tensors(declared, seed, matrix_dtype, scale)
    write_file(os.path.join(folder, "model.safetensors"), tensors,
               metadata={"format": "pt", "seed": str(int(seed))})
    return folder


def random_tensors_on_device(declared: Mapping[str, TensorDecl], seed: int, device: torch.device,
                             run_dtype: torch.dtype = torch.bfloat16, scale: str = "small") -> Dict[str, torch.Tensor]:
    """The same distributions drawn on the device, in the dtypes a loaded model would hold
    (for measurements on shapes too large to write to disk first; the values differ from
    ``random_tensors`` of the same seed)."""
    generator = torch.Generator(device=device)
    generator.manual_seed(int(seed))
    tensors: Dict[str, torch.Tensor] = {}
    for name, decl in declared.items():
        if decl.role == "table":
            tensors[name] = torch.zeros(decl.shape, dtype=torch.int32, device=device)
        elif decl.init == "norm":
            tensors[name] = 0.9 + 0.2 * torch.rand(decl.shape, generator=generator, dtype=torch.float32, device=device)
        elif decl.init == "zeros":
            tensors[name] = torch.zeros(decl.shape, dtype=torch.float32, device=device)
        else:
            value = torch.randn(decl.shape, generator=generator, dtype=torch.float32, device=device) * _std(decl, scale)
            tensors[name] = value.to(run_dtype) if decl.role == "matrix" else value
    return tensors
