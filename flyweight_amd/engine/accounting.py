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
    if hasattr(obj, "gathered_tensors"):        # tables a part reads by the row: not weights that a step streams
        for table in obj.gathered_tensors():
            seen.add(id(table))
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


def _chosen_parts(model) -> List:
    """The parts that read only the weights a step's tokens choose (a mixture of experts): they keep those
    weights out of the walk (``gathered_tensors``) and say themselves what a step reads and a token computes."""
    found = []

    def visit(part) -> None:
        if hasattr(part, "chosen_weight_bytes"):
            found.append(part)
        for below in (part.sub_parts() if hasattr(part, "sub_parts") else ()):
            visit(below)

    for block in model.layers:
        for part in block.parts():
            visit(part)
    return found


def step_weight_bytes(model, rows: int = 1) -> int:
    """Bytes of every weight a decode step of ``rows`` tokens reads once: the layers, the final norm and
    the head (a tied embedding table is read as the head; an untied one only by the row, which is not
    counted); of weights that tokens choose among, those that ``rows`` tokens are expected to choose.
    ``model``: a bound CausalLM."""
    return _bytes(_tensors([model.layers, model.final_norm, model.head])) + sum(
        int(part.chosen_weight_bytes(rows)) for part in _chosen_parts(model))


def product_flops_per_token(model) -> int:
    """Flops of the layers' matrix products for one token (the head is not among them: it runs
    for wanted rows only)."""
    linears = {id(item): item for item in _walk(model.layers, set()) if isinstance(item, Linear)}
    return 2 * sum(linear.weight.numel() for linear in linears.values()) + sum(
        int(part.chosen_flops_per_token()) for part in _chosen_parts(model))


def head_flops_per_row(model) -> int:
    return 2 * model.head.weight.numel()


def attention_flops(model, rows: int, keys_before: int = 0) -> int:
    """Flops of scores and weighted sums for ``rows`` new tokens of one sequence behind
    ``keys_before`` cached ones, causal, summed over the scheduled mixers that attend over a
    paged cache (2 products x 2 flops x heads x head size per visible query-key pair; a window
    bounds the pairs)."""
    total = 0

    def mixers_of(part):
        """A mixer, or the mixers it is made of."""
        below = part.sub_parts() if hasattr(part, "sub_parts") else ()
        if not below:
            yield part
        for inner in below:
            yield from mixers_of(inner)

    for entry in model.spec.schedule:
        top = getattr(model.layers[entry.layer], "mixer", None)
        for mixer in (mixers_of(top) if top is not None else ()):
            if hasattr(mixer, "mixing_flops"):      # a mixer that is no attention says what its rows cost
                total += mixer.mixing_flops(rows, keys_before)
                continue
            need = mixer.cache_need()
            if need is None or isinstance(need, dict) or not need.paged or not hasattr(mixer, "num_heads"):
                continue
            if getattr(mixer, "chunk", 0):      # a row sees the keys of its own chunk: its place in the chunk, and itself
                pairs = sum((keys_before + row) % mixer.chunk + 1 for row in range(rows))
            elif need.window:     # visible keys of row r: min(keys_before + r + 1, window)
                full = max(0, min(rows, need.window - keys_before - 1))     # rows that still see fewer than a window
                pairs = full * keys_before + full * (full + 1) // 2 + (rows - full) * need.window
            else:
                pairs = rows * keys_before + rows * (rows + 1) // 2
            total += 2 * mixer.num_heads * (mixer.head_dim + getattr(mixer, "v_head_dim", mixer.head_dim)) * pairs
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
