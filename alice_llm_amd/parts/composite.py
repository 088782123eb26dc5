"""A mixer made of several mixers that read the same input side by side.

Each side is any registered mixer with its own constants and tensors (under `<side name>.`); each side's
output is RMS-normed over the model width with a plain weight of its own (`<side name>.<norm_tensor>`) and
the normed outputs are averaged.  The average is folded into the norm weights (w / sides), so every side
reaches the residual stream as one more branch with its post norm, through the stream's fused add + norm.

With `side_norms=False` the sides' outputs are added as they are (a side that takes a constant factor of its
output has it among its own constructor arguments), and no norm tensors are declared.

At most one side may keep keys and values in pages; state tensors of the sides are kept apart by the side's
name.  A part that returns several branches returns a list of (branch, post norm) pairs; blocks push them
one after the other.
"""
from __future__ import annotations

from typing import Dict, Sequence

import torch

from .base import MIXERS, NORMS, CacheNeed, ParamSpec, Part, Precision


class _SideCache:
    """What one side sees of the layer's cache: the pages as they are, and its own state tensors."""

    def __init__(self, cache, prefix: str):
        self.k, self.v, self.block_table, self.writable, self.group = cache.k, cache.v, cache.block_table, cache.writable, cache.group
        self.state = {name[len(prefix):]: t for name, t in cache.state.items() if name.startswith(prefix)}


@MIXERS.register("side_by_side")
class SideBySide(Part):
    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, sides: Sequence, norm_eps: float,
                 norm_tensor: str = "out", side_norms: bool = True):
        if not sides:
            raise ValueError("side_by_side needs at least one side")
        self.precision = precision
        self.names = [s.name for s in sides]
        if len(set(self.names)) != len(self.names) or not all(self.names):
            raise ValueError(f"side_by_side: the sides need distinct names, found {self.names}")
        self.sides = [MIXERS.get(s.kind)(precision, positions, **s.args) for s in sides]
        self.norm_tensor = norm_tensor
        # the plain-weight RMS norm of each side's output; its weight is kept divided by the number of sides
        self.norms = [NORMS.get("rmsnorm")(precision, dim=hidden_size, eps=norm_eps, weight_offset=0.0,
                                           tensor_name=norm_tensor) if side_norms else None for _ in sides]
        needs = [m.cache_need() if hasattr(m, "cache_need") else None for m in self.sides]
        if sum(1 for n in needs if n is not None and n.kv is not None) > 1:
            raise ValueError("side_by_side: only one side may keep keys and values in pages")
        self._needs = needs

    @property
    def graph_safe(self) -> bool:
        return all(getattr(m, "graph_safe", False) for m in self.sides)

    @property
    def graph_safe_prompts(self) -> bool:
        return all(getattr(m, "graph_safe_prompts", False) or not (n is not None and n.state)
                   for m, n in zip(self.sides, self._needs))

    @property
    def accepts_fragment_activations(self) -> bool:
        return all(getattr(m, "accepts_fragment_activations", False) for m in self.sides)

    def param_specs(self) -> Dict[str, ParamSpec]:
        specs: Dict[str, ParamSpec] = {}
        for name, m, n in zip(self.names, self.sides, self.norms):
            for local, spec in m.param_specs().items():
                specs[f"{name}.{local}"] = spec
        for name, n in zip(self.names, self.norms):
            for local, spec in (n.param_specs().items() if n is not None else ()):
                specs[f"{name}.{local}"] = spec
        return specs

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        for side, m, n in zip(self.names, self.sides, self.norms):
            if name.startswith(side + "."):
                local = name[len(side) + 1:]
                if n is not None and local == self.norm_tensor:
                    # x / rms * w / sides: a division by a power of two is exact in every dtype here; otherwise the
                    # weight is kept in 32-bit
                    k = len(self.sides)
                    w = tensor / k if (k & (k - 1)) == 0 else tensor.float() / k
                    n.assign(local, w)
                else:
                    m.assign(local, tensor)
                return
        raise KeyError(name)

    def finalize(self) -> None:
        for m in self.sides:
            m.finalize()
        if len({n.weight.dtype for n in self.norms if n is not None}) > 1:
            for n in self.norms:
                n.weight = n.weight.float()

    def weight_bytes(self) -> int:
        return sum(m.weight_bytes() for m in self.sides if hasattr(m, "weight_bytes"))

    def cache_need(self) -> CacheNeed:
        kv = next((n.kv for n in self._needs if n is not None and n.kv is not None), None)
        state = []
        for name, n in zip(self.names, self._needs):
            if n is not None:
                state += [type(s)(f"{name}.{s.name}", s.shape, s.dtype) for s in n.state]
        return CacheNeed(kv=kv, state=tuple(state))

    def forward(self, x, ctx, cache):
        """Returns [(branch, post norm)] for the block to push: the stream adds norm(branch) for each."""
        return [(m.forward(x, ctx, _SideCache(cache, name + ".")), n)
                for name, m, n in zip(self.names, self.sides, self.norms)]
