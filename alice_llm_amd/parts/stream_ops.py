"""Operations on the residual stream between layers: shared parts of the model with an `apply(stream, ctx)`.

`reinject`: x <- W [x ; x_0], with x_0 the embedding output of the step's tokens (the stream keeps it as
`stream.start`) and W [width, 2 width] applied to the two side by side, x first.  The product's operands are
in the activation dtype, its sum and the new stream 32-bit.

`pass_offset`: before pass r of a repeated run of layers, x <- x + x_0 (from the second pass on) and
x <- x + P[r], with P [passes, width] a learned row per pass; all 32-bit.  The schedule entry that starts a pass
carries r (`before_arg`).
"""
from __future__ import annotations

from typing import Dict

import torch

from ..hip import ops
from .base import SHARED, ParamSpec, Part, Precision
from .linear import Linear


@SHARED.register("reinject")
class Reinject(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, tensor_name: str = "weight"):
        self.precision = precision
        self.W, self.tensor_name = hidden_size, tensor_name
        self.proj = Linear(2 * hidden_size, hidden_size, precision)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor_name: ParamSpec((self.W, 2 * self.W))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != self.tensor_name:
            raise KeyError(name)
        self.proj.load(tensor)

    def weight_bytes(self) -> int:
        return self.proj.nbytes()

    def apply(self, stream, ctx) -> None:
        stream.flush()
        both = torch.cat([stream.x, stream.start], dim=1).to(self.precision.act)
        stream.x = self.proj(both, torch.float32)


@SHARED.register("pass_offset")
class PassOffset(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, hidden_size: int, passes: int, tensor_name: str = "step",
                 reinject_start: bool = True):
        self.precision = precision
        self.W, self.passes, self.tensor_name, self.reinject_start = hidden_size, int(passes), tensor_name, reinject_start
        self.rows = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor_name: ParamSpec((self.passes, self.W))}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != self.tensor_name:
            raise KeyError(name)
        self.rows = tensor.float().contiguous()

    def weight_bytes(self) -> int:
        return self.rows.numel() * 4

    def apply(self, stream, ctx, number: int = 0) -> None:
        if not 0 <= number < self.passes:
            raise ValueError(f"pass {number} is outside the {self.passes} passes of this model")
        stream.flush()
        ops.add_rows(stream.x, stream.start if (number > 0 and self.reinject_start) else None, self.rows[number])
