"""Plain, slow Telulorn for whole sequences: the oracle of the tests.

One function per mechanism, written from the design's equations; whole sequences, dense masks,
token-by-token recurrences, no cache, float64 by default, and no code shared with the package
under test: it reads config.json keys and safetensors tensor names itself.

The design in this file's notation (T tokens, width W, weights stored [out, in], y = x A^T):

  x_0      = E[token]                                             embedding output
  order    = layers 0..a-1, then (a..b-1) repeated n times, then b..L-1     (loop a, b, n)
  pass r   : before the first layer of repetition r:  x <- x + x_0 (r > 0);  x <- x + P[r]   (P: [n, W])
  layer    : x <- x + mix(N_1(x));  x <- x + ff(N_2(x))  (ff may be absent)
  N(x)     = x / sqrt(mean(x^2) + eps) * w
  ff(h)    = D relu(U h)^2
  logits   = E N_f(x)

  mixer "attention": q, k, v with biases; the first R dimensions of q and k heads rotated in pairs (2i, 2i+1) by
             p * base^(-2i/R); values rotated over all their dimensions by their own position and the head's
             output rotated back by the query's; keys j <= i with i - j < w or j < keep; softmax whose
             denominator also holds exp(sink_h); output times sigmoid(G h); output matrix.
  mixer "parallel": c_l * left(h) + c_r * right(h);
    left   : no rotation; score - slope_h (i - j), slope_h = 2^(-8 (h+1) / H); keys of the query's own chunk
             floor(i / c) = floor(j / c); softmax; the heads' weights mixed by M [H, H]; output times
             sigmoid(G h); output matrix.
    right  : S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with q scaled by d^(-1/2),
             a = sigmoid(A_2 A_1 h + b)^(1/tau); o normed per head over its values with a weight shared by
             the heads, times silu(G h); output matrix.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

DT = torch.float64


# --------------------------------------------------------------------------- small formulas

def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * w


def relu_squared_ff(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    z = torch.relu(h @ up.T)
    return (z * z) @ down.T


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int, sign: float = 1.0) -> torch.Tensor:
    """x: [T, heads, d]; the first `dims` dimensions of every head turn in pairs (2i, 2i + 1) by the angle
    sign * position * base^(-2i / dims); the rest pass."""
    T = x.shape[0]
    i = torch.arange(dims // 2, dtype=DT)
    ang = sign * positions.to(DT)[:, None] * base ** (-2.0 * i / dims)[None, :]       # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# --------------------------------------------------------------------------- masks

def window_mask(T: int, size, keep_first: int) -> torch.Tensor:
    """[T, T] bool: i sees j if j <= i and (i - j < size or j < keep_first); size None: every j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m = m & ((i - j < size) | (j < keep_first))
    return m


def chunk_mask(T: int, size) -> torch.Tensor:
    """[T, T] bool: i sees j <= i of its own chunk, chunks counted from position 0; size None: every j <= i."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m = m & (i // size == j // size)
    return m


# --------------------------------------------------------------------------- softmax attention in its two forms

def sink_attention(q, k, v, mask, scale: float, sink) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv], mask [T, T], sink [H] or None.  The softmax's denominator also
    holds exp(sink_h), which has no value.  Returns [T, H, dv]."""
    T, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=DT)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        m = s.max(dim=1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].reshape(1, 1))
        e = torch.exp(s - m)
        den = e.sum(dim=1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def talking_attention(q, k, v, mask, scale: float, slopes, talk) -> torch.Tensor:
    """Scores minus slope_h (i - j); softmax over the visible keys; the heads' weights mixed by talk [H, H]
    (new weight of head h = sum_g talk[h, g] weight_g); head h applies them to its own kv head's values."""
    T, H, d = q.shape
    G = k.shape[1]
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(DT)
    w = torch.zeros(H, T, T, dtype=DT)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale - slopes[h] * dist
        s = s.masked_fill(~mask, -math.inf)
        w[h] = torch.softmax(s, dim=1)
    if talk is not None:
        w = torch.einsum("hg,gij->hij", talk, w)
    out = torch.zeros(T, H, v.shape[2], dtype=DT)
    for h in range(H):
        out[:, h] = w[h] @ v[:, h // (H // G)]
    return out


def distance_slopes(H: int) -> torch.Tensor:
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=DT)


# --------------------------------------------------------------------------- the recurrence

def gated_linear_recurrence(q, k, v, alpha, S0=None):
    """q, k, alpha: [T, H, d], v: [T, H, dv].  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by
    token from S0 (zero if None).  Returns (o [T, H, dv], the last S [H, d, dv])."""
    T, H, d = q.shape
    dv = v.shape[2]
    S = torch.zeros(H, d, dv, dtype=DT) if S0 is None else S0.clone()
    o = torch.zeros(T, H, dv, dtype=DT)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    return o, S


# --------------------------------------------------------------------------- mixers

def attention_mixer(h, p, cfg, eps, positions=None) -> torch.Tensor:
    """The mixer "attention" on the normed input h [T, W]; p: the mixer's tensors by local name."""
    T = h.shape[0]
    H, G, d = cfg["heads"], cfg.get("kv_heads", cfg["heads"]), cfg["dim"]
    dv = cfg.get("vdim", d)
    pos = torch.arange(T) if positions is None else positions
    q = (h @ p["q"].T + p["q.b"]).reshape(T, H, d)
    k = (h @ p["k"].T + p["k.b"]).reshape(T, G, d)
    v = (h @ p["v"].T + p["v.b"]).reshape(T, G, dv)
    rot = cfg.get("rot")
    if rot is not None:
        q = rotate_pairs(q, pos, rot["base"], rot["dims"])
        k = rotate_pairs(k, pos, rot["base"], rot["dims"])
        v = rotate_pairs(v, pos, rot["base"], dv)
    mask = cfg.get("mask") or {}
    o = sink_attention(q, k, v, window_mask(T, mask.get("size"), mask.get("keep_first", 0)), cfg["scale"], p.get("sink"))
    if rot is not None:
        o = rotate_pairs(o, pos, rot["base"], dv, sign=-1.0)
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T


def left_mixer(h, p, cfg) -> torch.Tensor:
    T = h.shape[0]
    H, G, d = cfg["heads"], cfg.get("kv_heads", cfg["heads"]), cfg["dim"]
    dv = cfg.get("vdim", d)
    q = (h @ p["q"].T).reshape(T, H, d)
    k = (h @ p["k"].T).reshape(T, G, d)
    v = (h @ p["v"].T).reshape(T, G, dv)
    mask = cfg.get("mask") or {}
    o = talking_attention(q, k, v, chunk_mask(T, mask.get("size")), cfg["scale"], distance_slopes(H), p.get("talk"))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ p["g"].T)
    return o @ p["o"].T


def decay(h, p, cfg) -> torch.Tensor:
    """alpha [T, H, d] = sigmoid(A_2 A_1 h + b)^(1 / tau)."""
    z = (h @ p["a1"].T) @ p["a2"].T + p["a2.b"]
    return torch.exp(torch.nn.functional.logsigmoid(z) / cfg["tau"]).reshape(h.shape[0], cfg["heads"], cfg["dim"])


def right_mixer(h, p, cfg, eps, S0=None, return_state=False):
    T = h.shape[0]
    H, d = cfg["heads"], cfg["dim"]
    dv = cfg.get("vdim", d)
    q = (h @ p["q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ p["k"].T).reshape(T, H, d)
    v = (h @ p["v"].T).reshape(T, H, dv)
    o, S = gated_linear_recurrence(q, k, v, decay(h, p, cfg), S0)
    o = rms_norm(o, p["norm"], eps).reshape(T, H * dv)
    z = h @ p["g"].T
    y = (o * z * torch.sigmoid(z)) @ p["o"].T
    return (y, S) if return_state else y


def sub(p: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v for k, v in p.items() if k.startswith(prefix)}


def parallel_mixer(h, p, cfg, eps) -> torch.Tensor:
    return (cfg["left_scale"] * left_mixer(h, sub(p, "left."), cfg["left"])
            + cfg["right_scale"] * right_mixer(h, sub(p, "right."), cfg["right"], eps))


# --------------------------------------------------------------------------- the model

def layer_runs(config: dict):
    """[(layer, number of the pass that starts here or None)]"""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None) for i in range(L)]
    a, b, n = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(a)]
    for r in range(n):
        runs += [(i, r if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, L)]


def forward(config: dict, tensors: dict, tokens, return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer run)."""
    w = {k: (v.to(DT) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps = config["norm"]["eps"]
    x0 = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    streams = []
    for i, start_of_pass in layer_runs(config):
        if start_of_pass is not None:
            if start_of_pass > 0:
                x = x + x0
            x = x + w["loop.step"][start_of_pass]
        layer = config["layers"][i]
        p = sub(w, f"l{i}.mix.")
        h = rms_norm(x, w[f"l{i}.norm1"], eps)
        if layer["type"] == "parallel":
            x = x + parallel_mixer(h, p, layer["mixer"], eps)
        elif layer["type"] == "attention":
            x = x + attention_mixer(h, p, layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            x = x + relu_squared_ff(rms_norm(x, w[f"l{i}.norm2"], eps), w[f"l{i}.mlp.up"], w[f"l{i}.mlp.down"])
        streams.append(x.clone())
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T
    return (logits, torch.stack(streams)) if return_layers else logits


# --------------------------------------------------------------------------- files

_DTYPES = {"BF16": (torch.bfloat16, 2), "F32": (torch.float32, 4), "I32": (torch.int32, 4), "F16": (torch.float16, 2)}


def read_safetensors(path: str) -> dict:
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        meta = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, m in meta.items():
        if name == "__metadata__":
            continue
        dt, _ = _DTYPES[m["dtype"]]
        a, b = m["data_offsets"]
        out[name] = torch.frombuffer(bytearray(data[a:b]), dtype=dt).reshape(m["shape"]).clone()
    return out


def read_model(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    return config, read_safetensors(os.path.join(folder, "model.safetensors"))


class PlainTelulorn:
    """The plain model on given tensors (64-bit)."""

    def __init__(self, config: dict, tensors: dict):
        self.c = config
        self.w = {k: (v.to(DT) if v.is_floating_point() else v) for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder: str) -> "PlainTelulorn":
        return cls(*read_model(folder))

    def forward(self, tokens, return_layers: bool = False):
        return forward(self.c, self.w, tokens, return_layers)

    def greedy(self, prompt, n: int):
        seq, out = list(prompt), []
        for _ in range(n):
            tok = int(self.forward(seq)[-1].argmax())
            out.append(tok)
            seq.append(tok)
        return out
