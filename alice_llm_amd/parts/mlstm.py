"""The matrix-memory mixer (mLSTM): a recurrent layer whose state per head is a matrix.

With the mixer's input h, per head: q = W_q h * d^(-1/2), k = W_k h, v = W_v h, the log input gate
i = cap * tanh((W_i h + b_i) / cap) and the log forget gate f = logsigmoid(cap * tanh((W_f h + b_f) / cap));
then, with a stabiliser m that starts at 0,
    m' = max(f + m, i),  S' = exp(f + m - m') S + exp(i - m') k v^T,  n' = exp(f + m - m') n + exp(i - m') k,
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).
Each head's o is divided by its root mean square, the heads are concatenated, multiplied by a weight and by
sigmoid(W_g h), and go through the output matrix.  S, n and m live in 32-bit in the cache's state tensors, one
row per slot, and are carried from step to step; all the gate arithmetic is 32-bit on both paths.

Head count, head sizes, the gates' cap and the norm's eps are constructor arguments.  One fused projection
gives [q | k | v | g | a | b] (a, b: the raw gate numbers) in 32-bit, so that nothing that enters the
recurrence is rounded on the way.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, Precision, StateNeed
from .linear import Linear

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "i_bias": "i.b",
                  "f": "f", "f_bias": "f.b"}


@MIXERS.register("mlstm")
class MatrixMemory(Part):
    graph_safe = True
    graph_safe_prompts = True        # the kernels find each sequence's rows and state row on the device

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int, head_dim: int,
                 value_head_dim: Optional[int] = None, gate_cap: float = 0.0, norm_eps: float = 1e-6,
                 tensor_names: Optional[Dict[str, str]] = None):
        self.precision = precision
        self.W, self.nH, self.d = hidden_size, num_heads, head_dim
        self.dv = head_dim if value_head_dim is None else int(value_head_dim)
        if min(self.nH, self.d, self.dv) < 1 or self.dv > ops.MLSTM_MAX_VALUE_DIM:
            raise ValueError(f"mlstm: heads {self.nH}, head sizes {self.d} and {self.dv}: at least 1, values at most "
                             f"{ops.MLSTM_MAX_VALUE_DIM}")
        self.cap = float(gate_cap or 0.0)
        self.eps = float(norm_eps)
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        self.qk, self.vw = self.nH * self.d, self.nH * self.dv
        self.row = -(-(2 * self.qk + 2 * self.vw + 2 * self.nH) // 4) * 4      # rows of whole 16-byte units
        self.proj = Linear(hidden_size, self.row, precision)
        self.o = Linear(self.vw, hidden_size, precision)
        self.norm_w: Optional[torch.Tensor] = None
        self.bias_i: Optional[torch.Tensor] = None
        self.bias_f: Optional[torch.Tensor] = None
        self._parts: Dict[str, torch.Tensor] = {}

    def _order(self):
        return ["q", "k", "v", "g", "i", "f"]

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["q"]: ParamSpec((self.qk, self.W)), n["k"]: ParamSpec((self.qk, self.W)),
                n["v"]: ParamSpec((self.vw, self.W)), n["g"]: ParamSpec((self.vw, self.W)),
                n["o"]: ParamSpec((self.W, self.vw)), n["norm"]: ParamSpec((self.vw,), init_std=0.1),
                n["i"]: ParamSpec((self.nH, self.W)), n["i_bias"]: ParamSpec((self.nH,), init_std=0.5),
                n["f"]: ParamSpec((self.nH, self.W)), n["f_bias"]: ParamSpec((self.nH,), init_std=0.5)}

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=(StateNeed("S", (self.nH, self.d, self.dv)), StateNeed("n", (self.nH, self.d)),
                                StateNeed("m", (self.nH,))))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["o"]:
            self.o.load(tensor)
        elif name == n["norm"]:
            self.norm_w = tensor.contiguous()
        elif name == n["i_bias"]:
            self.bias_i = tensor.float().contiguous()
        elif name == n["f_bias"]:
            self.bias_f = tensor.float().contiguous()
        elif name in [n[c] for c in self._order()]:
            self._parts[name] = tensor
        else:
            raise KeyError(name)

    def finalize(self) -> None:
        mats = [self.precision.matrix(self._parts.pop(self.names[c])) for c in self._order()]
        if len({m.dtype for m in mats}) > 1:
            mats = [m.float() for m in mats]
        w = torch.cat(mats, dim=0)
        if w.shape[0] < self.row:                             # the padding rows: zeros that nobody reads
            w = torch.cat([w, w.new_zeros(self.row - w.shape[0], w.shape[1])], dim=0)
        self.proj.load(w)

    def weight_bytes(self) -> int:
        return self.proj.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.proj.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        T = x.shape[0]
        rows = self.proj(x, torch.float32)                   # [T, q | k | v | g | a | b], nothing rounded
        out = torch.empty((T, self.vw), dtype=self.precision.act, device=rows.device)
        st = cache.state
        ops.mlstm(rows, self.bias_i, self.bias_f, self.norm_w, out, ctx, st["S"], st["n"], st["m"],
                  heads=self.nH, head_dim=self.d, value_head_dim=self.dv, cap=self.cap, eps=self.eps)
        return self.o(out, torch.float32, allow_partials=True)
