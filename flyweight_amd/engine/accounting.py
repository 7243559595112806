"""What a step has to read and to compute, counted from the bound model and its cache alone,
whatever parts the model is made of: the bytes of every weight a decode step uses once, the
cache bytes per token and per request, the flops of the matrix products per token. A roofline is
priced against these (what must be read, not what the kernels happened to read)."""

from __future__ import annotations

from typing import Dict, Iterator, List

import torch

from ..parts.linear import Linear


def _walk(obj, seen: set) -> Iterator:
    """Every Linear and tensor reachable from a part, a block or a container of them."""
    if id(obj) in seen:
        return
    seen.add(id(obj))
    if isinstance(obj, (torch.Tensor, Linear)):
        yield obj
        return
    if isinstance(obj, dict):
        children = list(obj.values())
    elif isinstance(obj, (list, tuple)):
        children = list(obj)
    elif hasattr(obj, "__dict__") and type(obj).__module__.split(".")[0] not in ("torch", "numpy", "builtins"):
        children = list(vars(obj).values())
    else:
        return
    for child in children:
        yield from _walk(child, seen)


def _tensors(obj) -> List[torch.Tensor]:
    found: Dict[int, torch.Tensor] = {}
    for item in _walk(obj, set()):
        for tensor in ((item.weight, item.bias) if isinstance(item, Linear) else (item,)):
            if tensor is not None and tensor.is_cuda:
                found.setdefault(tensor.data_ptr(), tensor)
    return list(found.values())


def _bytes(tensors) -> int:
    return sum(t.numel() * t.element_size() for t in tensors)


def step_weight_bytes(model) -> int:
    """Bytes of every weight a decode step reads once: the layers, the final norm and the head
    (a tied embedding table is read as the head; an untied one only by the row, which is not
    counted). ``model``: a bound CausalLM."""
    return _bytes(_tensors([model.layers, model.final_norm, model.head]))


def product_flops_per_token(model) -> int:
    """Flops of the layers' matrix products for one token (the head is not among them: it runs
    for wanted rows only)."""
    linears = {id(item): item for item in _walk(model.layers, set()) if isinstance(item, Linear)}
    return 2 * sum(linear.weight.numel() for linear in linears.values())


def head_flops_per_row(model) -> int:
    return 2 * model.head.weight.numel()


def attention_flops(model, rows: int, keys_before: int = 0) -> int:
    """Flops of scores and weighted sums for ``rows`` new tokens of one sequence behind
    ``keys_before`` cached ones, causal, summed over the scheduled mixers that attend over a
    paged cache (2 products x 2 flops x heads x head size per visible query-key pair; a window
    bounds the pairs)."""
    total = 0
    for entry in model.spec.schedule:
        mixer = getattr(model.layers[entry.layer], "mixer", None)
        need = mixer.cache_need() if mixer is not None else None
        if need is None or not need.paged or not hasattr(mixer, "num_heads"):
            continue
        pairs = 0
        for row in range(rows):
            visible = keys_before + row + 1
            pairs += min(visible, need.window) if need.window else visible
        total += 4 * mixer.num_heads * mixer.head_dim * pairs
    return total


def cache_bytes_per_token(cache) -> int:
    """Bytes one token of one request holds in the paged entries of the cache."""
    total = 0
    for entry, need in cache.needs.items():
        if need.paged:
            total += _bytes(_tensors([cache.storage[entry]])) // ((cache.group_pages[cache.entry_group[entry]] + 1) * cache.page_size)
    return total


def state_bytes_per_request(cache) -> int:
    """Bytes of fixed-size state one request holds."""
    total = 0
    for entry, need in cache.needs.items():
        if not need.paged:
            total += _bytes(_tensors([cache.storage[entry]])) // (cache.max_requests + 1)
    return total
