"""The gated-linear-attention mixer: a recurrent layer whose state per head is a matrix with a decay per key channel.

With the mixer's input h, per head: q = W_q h * d^(-1/2), k = W_k h, v = W_v h, and a decay per key channel
alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau) (a projection through a narrow middle); then
    S' = diag(alpha) S + k v^T,   o = S'^T q.
Each head's o is divided by its root mean square over the value size (times a weight of that size which the
heads share), the heads are concatenated, multiplied by silu(W_g h) and by a constant, and go through the
output matrix.  S starts at zero, lives in 32-bit in the cache's state rows, one per slot, and is carried from
step to step; the decay, its logarithm and exponential, the recurrence and the norm are 32-bit on both paths.

Head count, head sizes, tau, the norm's eps and the output factor are constructor arguments.  One fused
projection gives [q | k | v | g | W_a1 h] in 32-bit, so that nothing that enters the recurrence is rounded on the
way; the decay's second matrix is a projection of its own.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..hip import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, Precision, StateNeed
from .linear import Linear

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}


@MIXERS.register("gla")
class GatedLinearAttention(Part):
    graph_safe = True
    graph_safe_prompts = True        # the kernel finds each sequence's rows and state row on the device

    def __init__(self, precision: Precision, positions: dict, *, hidden_size: int, num_heads: int, head_dim: int,
                 decay_rank: int, tau: float, value_head_dim: Optional[int] = None, norm_eps: float = 1e-6,
                 output_scale: float = 1.0, tensor_names: Optional[Dict[str, str]] = None):
        self.precision = precision
        self.W, self.nH, self.d, self.rank = hidden_size, num_heads, head_dim, int(decay_rank)
        self.dv = head_dim if value_head_dim is None else int(value_head_dim)
        if min(self.nH, self.d, self.dv, self.rank) < 1 or self.d > ops.GLA_MAX_KEY_DIM:
            raise ValueError(f"gla: heads {self.nH}, head sizes {self.d} and {self.dv}, decay rank {self.rank}: at least 1, "
                             f"keys at most {ops.GLA_MAX_KEY_DIM}")
        if not tau > 0:
            raise ValueError(f"gla: tau must be positive, found {tau}")
        self.tau, self.eps, self.output_scale = float(tau), float(norm_eps), float(output_scale)
        self.names = dict(_DEFAULT_NAMES, **(tensor_names or {}))
        self.qk, self.vw = self.nH * self.d, self.nH * self.dv
        self.cols = (0, self.qk, 2 * self.qk, 2 * self.qk + self.vw)          # q, k, v, g
        self.a_col = 2 * self.qk + 2 * self.vw
        self.row = -(-(self.a_col + self.rank) // 4) * 4                       # rows of whole 16-byte units
        self.proj = Linear(hidden_size, self.row, precision)
        self.decay = Linear(self.rank, self.qk, precision)
        self.o = Linear(self.vw, hidden_size, precision)
        self.norm_w: Optional[torch.Tensor] = None
        self.decay_bias: Optional[torch.Tensor] = None
        self._parts: Dict[str, torch.Tensor] = {}

    def _order(self):
        return ["q", "k", "v", "g", "a1"]

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["q"]: ParamSpec((self.qk, self.W)), n["k"]: ParamSpec((self.qk, self.W)),
                n["v"]: ParamSpec((self.vw, self.W)), n["g"]: ParamSpec((self.vw, self.W)),
                n["o"]: ParamSpec((self.W, self.vw)), n["norm"]: ParamSpec((self.dv,), init_std=0.1),
                n["a1"]: ParamSpec((self.rank, self.W)), n["a2"]: ParamSpec((self.qk, self.rank), init_std=0.3),
                n["a2_bias"]: ParamSpec((self.qk,), init_std=1.0)}

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=(StateNeed("S", (self.nH, self.d, self.dv)),))

    def assign(self, name: str, tensor: torch.Tensor) -> None:
        n = self.names
        if name == n["o"]:
            self.o.load(tensor)
        elif name == n["a2"]:
            self.decay.load(tensor)
        elif name == n["norm"]:
            self.norm_w = tensor.contiguous()
        elif name == n["a2_bias"]:
            self.decay_bias = tensor.float().contiguous()
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
        return self.proj.nbytes() + self.decay.nbytes() + self.o.nbytes()

    @property
    def accepts_fragment_activations(self) -> bool:
        return self.proj.accepts_fragment_input

    def forward(self, x, ctx, cache) -> torch.Tensor:
        T = x.shape[0]
        rows = self.proj(x, torch.float32)                   # [T, q | k | v | g | a], nothing rounded
        narrow = rows[:, self.a_col:self.a_col + self.rank].to(self.precision.act).contiguous()      # the second matrix's operand
        z = self.decay(narrow, torch.float32)
        out = torch.empty((T, self.vw), dtype=self.precision.act, device=rows.device)
        ops.gla(rows, z, self.decay_bias, self.norm_w, out, ctx, cache.state["S"], heads=self.nH, head_dim=self.d,
                value_head_dim=self.dv, tau=self.tau, q_scale=self.d ** -0.5, eps=self.eps, columns=self.cols,
                out_scale=self.output_scale)
        return self.o(out, torch.float32, allow_partials=True)
