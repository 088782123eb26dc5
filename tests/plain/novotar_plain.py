"""Plain, slow Novotar for whole sequences: the oracle of the tests.

One function per mechanism, written from the design's equations; whole sequences, dense masks,
token-by-token recurrences, no cache, float64 by default, and no code shared with the package
under test: it reads config.json keys and safetensors tensor names itself.

The design in this file's notation (T tokens, width W, weights stored [out, in], y = x A^T):

  x_0      = E[token] * s_e                                       embedding output
  order    = layers 0..a-1, then (a..b-1) repeated n times, then b..L-1     (loop a, b, n)
  pass     : before the first layer of each repetition  x <- [x, x_0] J^T   (J: [W, 2W])
  layer    : h = N(x);  x <- x + mix(h) + ff(h);  x <- x + side(x, token)
  N(x)     = x / sqrt(mean(x^2) + eps) * w
  mix(h)   = ( N_l(left(h)) + N_r(right(h)) ) / 2                 N_l, N_r: RMS norms over W
  left     : windowed grouped-query softmax attention without positions, each head's output
             times sigmoid of one gate number, then the output matrix
  right    : the mLSTM matrix memory with a stabiliser that starts at 0
  ff(h)    : g = min(G h, c); u = clip(U h, -c, c); D (g sigmoid(1.702 g) (u + 1))
  side     : e = Tab[token][i d:(i+1) d];  y = P (gelu_tanh(S x) * e);  y / rms(y) * w_s
  logits   = H N_f(x)
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

DT = torch.float64


# --------------------------------------------------------------------------- small formulas

def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """Plain weight: no one-plus."""
    return unit_rms(x, eps) * w


def logsigmoid(z: torch.Tensor) -> torch.Tensor:
    return -torch.nn.functional.softplus(-z)


# --------------------------------------------------------------------------- left: windowed attention with a gate

def windowed_attention(q, k, v, scale: float, window: int) -> torch.Tensor:
    """q: [T, H, d], k: [T, G, d], v: [T, G, dv]; query head h reads kv head h // (H / G); position i sees
    j with 0 <= i - j < window.  Returns [T, H, dv].  No position enters the scores."""
    T, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (i - j >= 0) & (i - j < window)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def gated_attention(h, w, *, heads, kv_heads, dim, vdim, scale, window) -> torch.Tensor:
    """w: dict with q, k, v, g, o.  Head a's output is multiplied by sigmoid((g h)_a) before o."""
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, heads, dim)
    k = (h @ w["k"].T).view(T, kv_heads, dim)
    v = (h @ w["v"].T).view(T, kv_heads, vdim)
    o = windowed_attention(q, k, v, scale, window)
    o = o * torch.sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, heads * vdim) @ w["o"].T


# --------------------------------------------------------------------------- right: matrix memory

def mlstm_gates(h, w, cap: float):
    """Log input gate and log forget gate, [T, heads] each."""
    i = cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap)
    f = logsigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    return i, f


def mlstm_scan(q, k, v, i, f, state=None):
    """Token by token.  q, k: [T, H, d] (q already scaled), v: [T, H, dv], i, f: [T, H] logs.
    state: (S [H, d, dv], n [H, d], m [H]) or None for zeros (m starts at 0, not at minus infinity).
    Returns the read-outs [T, H, dv] and the state after the last token."""
    T, H, d = q.shape
    dv = v.shape[-1]
    if state is None:
        S, n, m = torch.zeros(H, d, dv, dtype=q.dtype), torch.zeros(H, d, dtype=q.dtype), torch.zeros(H, dtype=q.dtype)
    else:
        S, n, m = (t.clone() for t in state)
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        m_new = torch.maximum(f[t] + m, i[t])
        keep = torch.exp(f[t] + m - m_new)
        put = torch.exp(i[t] - m_new)
        S = keep[:, None, None] * S + put[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = keep[:, None] * n + put[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out[t] = num / den[:, None]
    return out, (S, n, m)


def matrix_memory(h, w, *, heads, dim, vdim, cap, eps, state=None, return_state=False):
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, heads, dim) * dim ** -0.5
    k = (h @ w["k"].T).view(T, heads, dim)
    v = (h @ w["v"].T).view(T, heads, vdim)
    i, f = mlstm_gates(h, w, cap)
    o, state = mlstm_scan(q, k, v, i, f, state)
    o = unit_rms(o, eps).reshape(T, heads * vdim) * w["norm"]
    o = o * torch.sigmoid(h @ w["g"].T)
    y = o @ w["o"].T
    return (y, state) if return_state else y


# --------------------------------------------------------------------------- the rest of a layer

def parallel_mixer(h, w_left, w_right, left, right, eps):
    """Half the sum of the two sides, each RMS-normed over the width with its own plain weight."""
    a = gated_attention(h, w_left, heads=left["heads"], kv_heads=left.get("kv_heads", left["heads"]), dim=left["dim"],
                        vdim=left.get("vdim", left["dim"]), scale=left["scale"],
                        window=left["mask"]["size"] if left.get("mask") else h.shape[0])
    b = matrix_memory(h, w_right, heads=right["heads"], dim=right["dim"], vdim=right.get("vdim", right["dim"]),
                      cap=right["gate_cap"], eps=eps)
    return 0.5 * (rms_norm(a, w_left["out"], eps) + rms_norm(b, w_right["out"], eps))


def dense_ff(h, gate, up, down, limit: float):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def token_side(x, e, gate, proj, w, eps):
    """e: the layer's part of the side table's rows of the tokens, [T, d]."""
    y = (gelu_tanh(x @ gate.T) * e) @ proj.T
    return unit_rms(y, eps) * w


def layer_order(n_layers: int, loop) -> list:
    """[(layer, starts_a_pass)] in the order in which the layers run."""
    if not loop:
        return [(i, False) for i in range(n_layers)]
    a, b, n = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(n):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n_layers)]


# --------------------------------------------------------------------------- reading a folder

def read_safetensors(path: str) -> dict:
    """name -> float64 (or int64) tensor; bfloat16, float32 and int32 only."""
    with open(path, "rb") as fh:
        n = struct.unpack("<Q", fh.read(8))[0]
        head = json.loads(fh.read(n))
        data = fh.read()
    out = {}
    for name, info in head.items():
        if name == "__metadata__":
            continue
        lo, hi = info["data_offsets"]
        raw = bytearray(data[lo:hi])
        kind = info["dtype"]
        if kind == "BF16":
            t = torch.frombuffer(raw, dtype=torch.bfloat16).to(DT)
        elif kind == "F32":
            t = torch.frombuffer(raw, dtype=torch.float32).to(DT)
        elif kind == "I32":
            t = torch.frombuffer(raw, dtype=torch.int32).to(torch.int64)
        else:
            raise ValueError(f"{name}: dtype {kind}")
        out[name] = t.reshape(info["shape"]).clone()
    return out


class PlainNovotar:
    def __init__(self, config: dict, tensors: dict):
        self.c = config
        self.t = tensors
        self.eps = config["norm"]["eps"]

    @classmethod
    def from_folder(cls, folder: str) -> "PlainNovotar":
        with open(os.path.join(folder, "config.json")) as fh:
            config = json.load(fh)
        return cls(config, read_safetensors(os.path.join(folder, "model.safetensors")))

    def _sub(self, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def layer(self, i: int, x, tokens):
        c, t, eps = self.c, self.t, self.eps
        spec = c["layers"][i]
        p = f"l{i}."
        h = rms_norm(x, t[p + "norm1"], eps)
        if spec["type"] != "parallel":
            raise ValueError(spec["type"])
        y = parallel_mixer(h, self._sub(p + "mix.left."), self._sub(p + "mix.right."),
                           spec["mixer"]["left"], spec["mixer"]["right"], eps)
        if spec.get("mlp"):
            y = y + dense_ff(h, t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"], spec["mlp"]["limit"])
        x = x + y
        side = c.get("token_side")
        if side:
            d = side["dim"]
            e = t["side.embed"][tokens][:, i * d:(i + 1) * d]
            x = x + token_side(x, e, t[p + "side.gate"], t[p + "side.proj"], t[p + "side.norm"], eps)
        return x

    def forward(self, tokens, return_layers: bool = False):
        """Logits [T, vocab] in float64 (and the residual stream after every layer run)."""
        c, t = self.c, self.t
        tokens = torch.as_tensor(tokens, dtype=torch.int64)
        x0 = t["embed"][tokens] * c["embedding"]["scale"]
        x = x0
        runs = []
        for i, first in layer_order(len(c["layers"]), c.get("loop")):
            if first:
                x = torch.cat([x, x0], dim=-1) @ t["loop.in"].T
            x = self.layer(i, x, tokens)
            runs.append(x)
        logits = rms_norm(x, t["final.norm"], self.eps) @ t["head"].T
        return (logits, torch.stack(runs)) if return_layers else logits

    def greedy(self, prompt, n: int) -> list:
        seq, out = list(prompt), []
        for _ in range(n):
            tok = int(torch.argmax(self.forward(seq)[-1]))
            out.append(tok)
            seq.append(tok)
        return out
