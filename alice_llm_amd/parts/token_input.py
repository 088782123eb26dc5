"""A second token table and the per-layer input that reads it.

`token_table` (a shared part of the model): a [vocab, dim] table that several layers read columns of.
`token_gate` (a layer extra): with the layer's columns e = table[token][column : column + dim] and the
residual stream x after the layer's other parts,
    g = gelu_tanh(W_gate x) * e,   y = W_proj g,   x <- x + y / sqrt(mean(y^2) + eps) * w_norm.
The last step is the stream's fused add with a plain-weight RMS norm.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import EXTRAS, NORMS, SHARED, ParamSpec, Part, Precision
from .linear import Linear


@SHARED.register("token_table")
class TokenTable(Part):
    graph_safe = True

    def __init__(self, precision: Precision, *, vocab_size: int, dim: int, tensor_name: str = "weight"):
        self.V, self.dim, self.tensor_name = vocab_size, dim, tensor_name
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.tensor_name: ParamSpec((self.V, self.dim), init_std=1.0)}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        if name != self.tensor_name:
            raise KeyError(name)
        self.weight = tensor.contiguous()          # row-major, as stored: rows are gathered, never multiplied


@EXTRAS.register("token_gate")
class TokenGate(Part):
    graph_safe = True

    def __init__(self, precision: Precision, shared: dict, *, hidden_size: int, dim: int, column: int, table: str,
                 norm_eps: float, tensor_names: Optional[Dict[str, str]] = None):
        if table not in shared or not isinstance(shared[table], TokenTable):
            raise ValueError(f"token_gate: the model shares no token table named '{table}'")
        self.precision = precision
        self.table = shared[table]
        if column < 0 or column + dim > self.table.dim:
            raise ValueError(f"token_gate: columns {column}..{column + dim} are outside the table's {self.table.dim}")
        self.W, self.dim, self.column = hidden_size, dim, column
        self.names = dict({"gate": "gate", "proj": "proj", "norm": "norm"}, **(tensor_names or {}))
        self.gate = Linear(hidden_size, dim, precision)
        self.proj = Linear(dim, hidden_size, precision)
        self.norm = NORMS.get("rmsnorm")(precision, dim=hidden_size, eps=norm_eps, weight_offset=0.0,
                                         tensor_name=self.names["norm"])

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["gate"]: ParamSpec((self.dim, self.W)), n["proj"]: ParamSpec((self.W, self.dim)),
                n["norm"]: ParamSpec((self.W,), init_std=0.1)}

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["gate"]:
            self.gate.load(tensor)
        elif name == n["proj"]:
            self.proj.load(tensor)
        elif name == n["norm"]:
            self.norm.assign(name, tensor)
        else:
            raise KeyError(name)

    def weight_bytes(self) -> int:
        return self.gate.nbytes() + self.proj.nbytes()

    def forward(self, stream, ctx) -> None:
        """Reads the stream as it stands (pending branches added first) and pushes its own branch."""
        x = stream.normed(None)                               # the stream itself in the activation dtype
        z = self.gate(x, self.precision.act)
        g = torch.empty_like(z)
        ops.gelu_mul_rows(z, self.table.weight, self.column, ctx.tokens, g, full_precision=self.precision.full)
        stream.push(self.proj(g, torch.float32), self.norm)
