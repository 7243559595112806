"""A small safetensors reader and writer.

File layout: an 8-byte little-endian header length, a JSON object that maps each
tensor name to ``{"dtype", "shape", "data_offsets": [begin, end]}`` (offsets relative
to the end of the header), then the payload. The checks are the ones the reference's
header parser makes (native/include/flyweight_v2_safetensors.hpp:50-135): the header
must lie inside the file, offsets must not be inverted or leave the payload, the byte
range must equal ``prod(shape) * sizeof(dtype)``, and a dtype outside the accepted set
is refused by name. ``__metadata__`` is skipped. Files are memory-mapped; nothing in
them is executed.
"""

from __future__ import annotations

import json
import mmap
import os
import struct
from dataclasses import dataclass
from typing import Dict, Iterable, List, Mapping, Tuple

import numpy as np
import torch

from ..config import json_reader


class SafetensorsError(ValueError):
    pass


# name -> (bytes per element, numpy carrier dtype, torch dtype)
_DTYPES = {
    "F32": (4, np.dtype("<f4"), torch.float32),
    "BF16": (2, np.dtype("<u2"), torch.bfloat16),
    "F16": (2, np.dtype("<f2"), torch.float16),
    "I32": (4, np.dtype("<i4"), torch.int32),
    "I64": (8, np.dtype("<i8"), torch.int64),
}
_TORCH_TO_NAME = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16",
                  torch.int32: "I32", torch.int64: "I64"}


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: str
    shape: Tuple[int, ...]
    begin: int          # absolute byte offset in the file
    end: int
    path: str


def _product(shape: Iterable[int]) -> int:
    count = 1
    for extent in shape:
        count *= int(extent)
    return count


def read_header(path: str) -> Dict[str, TensorEntry]:
    size = os.path.getsize(path)
    if size < 8:
        raise SafetensorsError(f"{path}: file is too short to hold a safetensors header")
    with open(path, "rb") as handle:
        (header_len,) = struct.unpack("<Q", handle.read(8))
        if header_len > size - 8:
            raise SafetensorsError(
                f"{path}: header length {header_len} exceeds the file ({size} bytes); truncated?")
        raw = handle.read(header_len)
    try:
        header = json_reader.parse(raw)
    except json_reader.JsonError as error:
        raise SafetensorsError(f"{path}: header is not valid JSON ({error})") from None
    if not isinstance(header, dict):
        raise SafetensorsError(f"{path}: header must be a JSON object")
    payload_begin = 8 + header_len
    payload_size = size - payload_begin
    entries: Dict[str, TensorEntry] = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        if not isinstance(info, dict):
            raise SafetensorsError(f"{path}: entry '{name}' is not an object")
        dtype = info.get("dtype")
        if dtype not in _DTYPES:
            raise SafetensorsError(
                f"{path}: tensor '{name}' has unsupported dtype {dtype!r} "
                f"(accepted: {', '.join(sorted(_DTYPES))})")
        shape = info.get("shape")
        offsets = info.get("data_offsets")
        if (not isinstance(shape, list)
                or any(isinstance(e, bool) or not isinstance(e, int) or e < 0 for e in shape)):
            raise SafetensorsError(f"{path}: tensor '{name}' has a malformed shape {shape!r}")
        if (not isinstance(offsets, list) or len(offsets) != 2
                or any(isinstance(e, bool) or not isinstance(e, int) or e < 0 for e in offsets)):
            raise SafetensorsError(f"{path}: tensor '{name}' has malformed data_offsets {offsets!r}")
        begin, end = offsets
        if end < begin:
            raise SafetensorsError(f"{path}: tensor '{name}' has inverted data_offsets {offsets}")
        if end > payload_size:
            raise SafetensorsError(
                f"{path}: tensor '{name}' ends at byte {end} of a {payload_size}-byte payload; truncated?")
        expected = _product(shape) * _DTYPES[dtype][0]
        if end - begin != expected:
            raise SafetensorsError(
                f"{path}: tensor '{name}' spans {end - begin} bytes but shape {shape} of {dtype} "
                f"needs {expected}")
        entries[name] = TensorEntry(name, dtype, tuple(shape), payload_begin + begin,
                                    payload_begin + end, path)
    return entries


class SafetensorsFile:
    """A memory-mapped safetensors file; tensors come out as CPU torch tensors that
    own their memory (a copy of the mapped bytes)."""

    def __init__(self, path: str):
        self.path = path
        self.entries = read_header(path)
        self._handle = open(path, "rb")
        self._map = mmap.mmap(self._handle.fileno(), 0, access=mmap.ACCESS_READ) \
            if os.path.getsize(path) else None

    def names(self) -> List[str]:
        return list(self.entries)

    def tensor(self, name: str) -> torch.Tensor:
        entry = self.entries[name]
        width, carrier, torch_dtype = _DTYPES[entry.dtype]
        count = _product(entry.shape)
        if count == 0:
            return torch.empty(entry.shape, dtype=torch_dtype)
        array = np.frombuffer(self._map, dtype=carrier, count=count, offset=entry.begin)
        tensor = torch.from_numpy(array.copy())
        if entry.dtype == "BF16":
            tensor = tensor.view(torch.int16).view(torch.bfloat16)
        return tensor.reshape(entry.shape)

    def close(self) -> None:
        if self._map is not None:
            self._map.close()
            self._map = None
        self._handle.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def write_file(path: str, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] = None) -> None:
    header: Dict[str, object] = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    blobs: List[bytes] = []
    for name, tensor in tensors.items():
        tensor = tensor.detach().cpu().contiguous()
        if tensor.dtype not in _TORCH_TO_NAME:
            raise SafetensorsError(f"cannot write tensor '{name}' of dtype {tensor.dtype}")
        if tensor.dtype == torch.bfloat16:
            blob = tensor.view(torch.int16).numpy().tobytes()
        else:
            blob = tensor.numpy().tobytes()
        header[name] = {"dtype": _TORCH_TO_NAME[tensor.dtype], "shape": list(tensor.shape),
                        "data_offsets": [offset, offset + len(blob)]}
        offset += len(blob)
        blobs.append(blob)
    raw = json.dumps(header, separators=(",", ":")).encode("utf-8")
    raw += b" " * ((-len(raw)) % 8)
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(raw)))
        handle.write(raw)
        for blob in blobs:
            handle.write(blob)


def checkpoint_files(model_dir: str) -> List[str]:
    """The shards of a model folder: those ``model.safetensors.index.json`` lists, else
    every ``*.safetensors`` in the folder, sorted (the reference globs and sorts,
    native/src/v2_runtime.cpp:9961-9993)."""
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        try:
            weight_map = json_reader.parse_file(index)["weight_map"]
        except (json_reader.JsonError, KeyError, TypeError) as error:
            raise SafetensorsError(f"{index}: malformed index ({error})") from None
        files = sorted(set(weight_map.values()))
    else:
        files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    if not files:
        raise SafetensorsError(f"{model_dir}: no .safetensors files")
    paths = [os.path.join(model_dir, f) for f in files]
    for path in paths:
        if not os.path.isfile(path):
            raise SafetensorsError(f"{path}: listed in the index but not present")
    return paths
