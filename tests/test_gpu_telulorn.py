"""Telulorn on the GPU against the plain implementation, in 32-bit and in bfloat16: every mechanism alone, then the
model through the engine: whole prompts, the stream after every layer run, a prefix and then single tokens,
prompts in pieces down to two tokens, unequal batches against each request alone on slots and pages that are used
again, long decoding from the first token, captured against eager steps, and greedy generation, the command line
and trace replay through the package's own entry points."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.hip import ops
from alice_llm_amd.parts import FEED_FORWARDS, SHARED, Precision
from helpers import TELULORN, max_err, random_tokens, telulorn_folder, telulorn_pair
from plain import telulorn_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
CASES = [(n, d) for n in TELULORN for d in DTYPES]
_PAIRS = {}


def pair(name, dtype):
    if (name, dtype) not in _PAIRS:
        _PAIRS[(name, dtype)] = telulorn_pair(name, dtype, seed=len(name) + 3)
    return _PAIRS[(name, dtype)]


def row_errors(got, ref):
    """Per row of logits: the root mean square of the difference (means taken off) over that of the row itself."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean(-1, keepdim=True)
    r = ref.double().cpu() - ref.double().cpu().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def assert_close(got, ref, dtype, what=""):
    """The test models' weights make softmaxes sharp, gates open and close and decays range from fast to almost
    none, so a rounding ahead of such a place is amplified.  32-bit: every logit within 1e-3 of the plain model's
    (relative to the largest logit) and the median row within 2e-5.  bfloat16: a row's error is measured as a whole
    (root mean square against the row's own): the rows' mean within 0.06 and nine rows in ten within 0.1 (of twenty
    rows and more; every row within 0.3 of fewer).  A wrong key, state or position moves most rows by 0.3 and more."""
    assert got.shape == ref.shape, what
    if dtype == "float32":
        scale = max(1.0, float(ref.abs().max()))
        e = (got.double().cpu() - ref.double().cpu()).abs().max(-1).values
        assert float(e.max()) < 1e-3 * scale and float(e.median()) < 2e-5 * scale, (what, float(e.max()), float(e.median()))
    else:
        e = row_errors(got, ref)
        many = e.numel() >= 20
        assert float(e.mean()) < 0.06 and float(e.quantile(0.9) if many else e.max()) < (0.1 if many else 0.3) and float(e.max()) < 1.0, \
            (what, float(e.max()), float(e.mean()))


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def tables(T, width, base):
    i = torch.arange(width // 2, dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * base ** (-2.0 * i / width)[None, :]
    return torch.cos(ang).float().to(DEV), torch.sin(ang).float().to(DEV)


# ------------------------------------------------------------------ mechanisms alone

def _paged(k, v, page, scatter_seed):
    """Keys [T, G, d] and values [T, G, dv] of one sequence put into scattered pages; returns pools and the table."""
    T, G, d = k.shape
    n = -(-T // page)
    order = torch.randperm(n + 3, generator=torch.Generator().manual_seed(scatter_seed))[:n] + 1
    kp = torch.full((n + 5, G, page, d), 7.0, dtype=k.dtype)
    vp = torch.full((n + 5, G, page, v.shape[-1]), -7.0, dtype=v.dtype)
    for t in range(T):
        kp[order[t // page], :, t % page] = k[t]
        vp[order[t // page], :, t % page] = v[t]
    return kp.to(DEV), vp.to(DEV), order.to(torch.int32)[None].to(DEV)


class _Pieces:
    """What the matrix-core prompt kernel reads of a step: pieces of one sequence as if they were sequences of a step."""

    def __init__(self, pieces, T):
        cu = [0]
        for a, b in pieces:
            cu.append(cu[-1] + b - a)
        self.positions = torch.cat([torch.arange(a, b) for a, b in pieces]).to(torch.int32).to(DEV)
        self.cu_seqlens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.n_seqs, self.max_position, self.rows = len(pieces), T - 1, torch.cat([torch.arange(a, b) for a, b in pieces])


def _pieces_of(T, edges):
    """The whole prompt as one piece; then pieces that start and end around every edge, as sequences of one step."""
    cuts = sorted({0, T} | {p for e in edges for p in (e - 1, e, e + 2) if 0 < p < T})
    return [[(0, T)], list(zip(cuts[:-1], cuts[1:]))]


def _rows_of(T, edges):
    """A whole prompt, its last token alone, and the single tokens around every edge."""
    out = [slice(0, T), slice(T - 1, T)]
    for e in edges:
        out += [slice(p, p + 1) for p in (e - 1, e, e + 1) if 0 <= p < T]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,keep,T", [(5, 3, 40), (64, 2, 200), (65, 70, 200), (1, 1, 9), (300, 4, 130), (9, 0, 50)])
def test_window_with_kept_first_positions_sink_and_turned_values(dtype, window, keep, T):
    """Marker keys that every query scores far above the others: one sits just inside the window of one query and just
    outside that of the next; one is the last kept first position and one the first that is not kept.  Scattered
    pages; value heads of another size than the keys; a sink of the scores' order; the values cached turned by their
    position and the output turned back; the gate one number an output element."""
    H, G, d, dv, page, base = 4, 2, 24, 40, 64, 30.0
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    gate = rnd(T, H * dv + 3, seed=4, scale=2.0)
    sink = torch.tensor([0.5, 3.0, -2.0, 8.0])
    mark = max(keep + 1, T - 20 - window)       # seen by queries up to mark + window - 1, not by mark + window
    q[:, :, 0] = 3.0
    k[:, :, 0] = 0.0
    k[mark, :, 0] = 6.0
    v[mark] += 5.0
    if keep:
        k[keep - 1, :, 0] = 5.0                 # the last kept position: seen by every later query
        v[keep - 1] -= 4.0
        k[keep, :, 0] = 5.5                     # the next one: seen only while it is inside the window
        v[keep] += 3.0
    q, k, v = (x.to(dt) for x in (q, k, v))
    pos = torch.arange(T)
    vt = P.rotate_pairs(v.double(), pos, base, dv)
    ref = P.sink_attention(q.double(), k.double(), vt, P.window_mask(T, window, keep), 0.5, sink.double())
    ref = P.rotate_pairs(ref, pos, base, dv, sign=-1.0) * torch.sigmoid(gate.double()[:, :H * dv]).view(T, H, dv) * 1.25
    kp, vp, bt = _paged(k, vt.to(dt), page, 5)
    vc, vs = tables(T, dv, base)
    posd = pos.to(torch.int32).to(DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    for rows in _rows_of(T, [mark + window, keep + window]):
        n = rows.stop - rows.start
        out = torch.empty(n, H * dv, dtype=dt, device=DEV)
        ops.attention_masked(q[rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, out, posd[rows].contiguous(),
                             seq[rows].contiguous(), bt, num_heads=H, scale=0.5, window=window, keep_first=keep,
                             max_position=T - 1, full_precision=dtype == "float32", sink=sink.to(DEV),
                             gate=gate.to(DEV)[rows][:, :H * dv], gate_per_element=True, out_scale=1.25,
                             value_cos=vc, value_sin=vs)
        err = max_err(out.view(n, H, dv), ref[rows])
        assert err < (3e-5 if dtype == "float32" else 8e-2), (rows, err)
        out2 = torch.empty_like(out)            # the same rows by the kernel that splits the keys over blocks
        ops.attention_split(q[rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, out2, posd[rows].contiguous(),
                            seq[rows].contiguous(), bt, num_heads=H, scale=0.5, window=window, keep_first=keep,
                            max_position=T - 1, max_keys=min(T, window + keep), sink=sink.to(DEV),
                            gate=gate.to(DEV)[rows][:, :H * dv], gate_per_element=True, out_scale=1.25,
                            value_cos=vc, value_sin=vs)
        err = max_err(out2.view(n, H, dv), ref[rows])
        assert err < (3e-5 if dtype == "float32" else 8e-2), ("split", rows, err)
    if dtype == "bfloat16":                     # the matrix-core kernel of prompts: whole, and in pieces around the edges
        for hpw, pieces in [(w, p) for w in (1, 2) for p in _pieces_of(T, [mark + window, keep + window, 64])]:
            ctx = _Pieces(pieces, T)
            n = ctx.rows.numel()
            out = torch.empty(n, H * dv, dtype=dt, device=DEV)
            ops.attention_tiled(q[ctx.rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, out, ctx, bt.expand(ctx.n_seqs, -1).contiguous(),
                                num_heads=H, scale=0.5, window=window, keep_first=keep, sink=sink.to(DEV),
                                gate=gate.to(DEV)[ctx.rows][:, :H * dv], gate_per_element=True, out_scale=1.25,
                                value_cos=vc, value_sin=vs, heads_per_wave=hpw)
            err = max_err(out.view(n, H, dv), ref[ctx.rows])
            assert err < 8e-2, (hpw, len(pieces), err)
    if mark + window < T:
        assert (ref[mark + window - 1] - ref[mark + window]).abs().max() > 0.3          # the markers do show
    if keep and keep + window < T:
        assert (ref[keep + window - 1] - ref[keep + window]).abs().max() > 0.1


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chunk,T", [(7, 40), (64, 200), (65, 200), (1, 9), (300, 130), (100, 330)])
def test_chunks_distance_term_and_mixed_heads(dtype, chunk, T):
    """A marker key at the last position of a chunk: seen by that position alone, not by the first query of the next
    chunk; another at a chunk's first position, seen to the chunk's end.  The distance term is taken off the scores,
    the heads' weights are mixed by a matrix far from the identity, and every head keeps its own kv head's values.  The
    prompt kernel is run with one, two and four heads of a group a wave."""
    H, G, d, dv, page = 8, 2, 16, 24, 64
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    gate = rnd(T, H * dv, seed=4, scale=2.0)
    talk = (torch.eye(H) * 0.5 + rnd(H, H, seed=5, scale=0.5))
    n_chunks = -(-T // chunk)
    c = max(0, n_chunks - 2)                    # a chunk that is followed by another where there are two
    first, last = c * chunk, min(T, (c + 1) * chunk) - 1
    q[:, :, 0] = 3.0
    k[:, :, 0] = 0.0
    k[last, :, 0] = 6.0
    v[last] += 5.0
    k[first, :, 0] = 4.0
    v[first] -= 3.0
    q, k, v = (x.to(dt) for x in (q, k, v))
    slopes = P.distance_slopes(H)
    ref = P.talking_attention(q.double(), k.double(), v.double(), P.chunk_mask(T, chunk), 0.5, slopes, talk.double())
    ref = ref * torch.sigmoid(gate.double()).view(T, H, dv) * 0.75
    kp, vp, bt = _paged(k, v, page, 6)
    posd = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    for rows in _rows_of(T, [last + 1, first]):
        n = rows.stop - rows.start
        per = torch.empty(n, H, G, dv, dtype=torch.float32, device=DEV)
        out = torch.empty(n, H * dv, dtype=dt, device=DEV)
        ops.attention_masked(q[rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, None, posd[rows].contiguous(),
                             seq[rows].contiguous(), bt, num_heads=H, scale=0.5, chunk=chunk, max_position=T - 1,
                             full_precision=dtype == "float32", bias_slopes=slopes.float().to(DEV), per_value_head=per)
        ops.mix_heads(per, talk.to(DEV), gate.to(DEV)[rows].contiguous(), out, full_precision=dtype == "float32", out_scale=0.75)
        err = max_err(out.view(n, H, dv), ref[rows])
        assert err < (3e-5 if dtype == "float32" else 8e-2), (rows, err)
        per.fill_(9.0)                          # the same rows by the kernel that splits the keys over blocks
        ops.attention_split(q[rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, None, posd[rows].contiguous(),
                            seq[rows].contiguous(), bt, num_heads=H, scale=0.5, chunk=chunk, max_position=T - 1,
                            max_keys=min(T, chunk), bias_slopes=slopes.float().to(DEV), per_value_head=per)
        ops.mix_heads(per, talk.to(DEV), gate.to(DEV)[rows].contiguous(), out, full_precision=dtype == "float32", out_scale=0.75)
        err = max_err(out.view(n, H, dv), ref[rows])
        assert err < (3e-5 if dtype == "float32" else 8e-2), ("split", rows, err)
    if dtype == "bfloat16":
        for hpw, pieces in [(w, p) for w in (1, 2, 4) for p in _pieces_of(T, [last + 1, first, 64])]:
            ctx = _Pieces(pieces, T)
            n = ctx.rows.numel()
            per = torch.empty(n, H, G, dv, dtype=torch.float32, device=DEV)
            out = torch.empty(n, H * dv, dtype=dt, device=DEV)
            ops.attention_tiled(q[ctx.rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, None, ctx, bt.expand(ctx.n_seqs, -1).contiguous(),
                                num_heads=H, scale=0.5, chunk=chunk, bias_slopes=slopes.float().to(DEV), per_value_head=per,
                                heads_per_wave=hpw)
            ops.mix_heads(per, talk.to(DEV), gate.to(DEV)[ctx.rows].contiguous(), out, full_precision=False, out_scale=0.75)
            err = max_err(out.view(n, H, dv), ref[ctx.rows])
            assert err < 8e-2, (hpw, len(pieces), err)
    if last + 1 < T:
        assert (ref[last] - ref[last + 1]).abs().max() > 0.3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,dv,R,interleaved", [(24, 40, 8, True), (32, 32, 32, True), (20, 12, 0, True), (16, 8, 16, False)])
def test_projection_rows_to_query_and_cache(dtype, d, dv, R, interleaved):
    """Bias, rotation of neighbouring pairs over a part of the head, values turned over all their dimensions, and the
    write into scattered pages, for two sequences in one step that start at other positions than 0."""
    H, G, page, base = 3, 2, 64, 100.0
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    starts, lens = [60, 3], [10, 70]
    T = sum(lens)
    width = H * d + G * (d + dv)
    rows = rnd(T, width + 5, seed=1)
    bias = rnd(width, seed=2)
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)])
    seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)])
    bt = torch.tensor([[3, 1, 0], [4, 2, 0]], dtype=torch.int32)
    kp = torch.zeros(6, G, page, d, dtype=dt, device=DEV)
    vp = torch.zeros(6, G, page, dv, dtype=dt, device=DEV)
    q = torch.empty(T, H * d, dtype=dt, device=DEV)
    c, s = tables(80, R, base) if R else (None, None)
    vc, vs = tables(80, dv, base)
    ops.qkv_prepare(rows.to(DEV), bias.to(DEV), q, kp, vp, pos.to(torch.int32).to(DEV), seq.to(torch.int32).to(DEV), bt.to(DEV),
                    num_heads=H, num_kv_heads=G, head_dim=d, value_head_dim=dv, max_position=79, cos=c, sin=s,
                    rotary_dim=R, interleaved=interleaved, value_cos=vc, value_sin=vs)
    x = rows.double()[:, :width] + bias.double()
    qr, kr, vr = x[:, :H * d].view(T, H, d), x[:, H * d:(H + G) * d].view(T, G, d), x[:, (H + G) * d:].view(T, G, dv)

    def turn(x, width):
        if not width:
            return x
        if interleaved:
            return P.rotate_pairs(x, pos, base, width)
        half = width // 2                        # halves: i with i + width / 2, the same angles
        perm = torch.stack([torch.arange(half), torch.arange(half) + half], 1).flatten()
        y = x.clone()
        y[..., perm] = P.rotate_pairs(x[..., perm].contiguous(), pos, base, width)
        return y
    tol = 2e-6 if dtype == "float32" else 4e-2
    assert max_err(q.view(T, H, d), turn(qr, R)) < tol * 4
    kt, vt = turn(kr, R), turn(vr, dv)
    for t in range(T):
        page_id = int(bt[seq[t], pos[t] // page])
        assert max_err(kp[page_id, :, pos[t] % page], kt[t]) < tol * 4, t
        assert max_err(vp[page_id, :, pos[t] % page], vt[t]) < tol * 4, t
    assert float(kp[5].abs().max()) == 0.0 and float(kp[0].abs().max()) == 0.0       # nothing beside its own places


def _gla_plain(rows, z, bias, w, H, d, dv, tau, eps, cols, S0=None):
    T = rows.shape[0]
    x = rows.double()
    q = x[:, cols[0]:cols[0] + H * d].view(T, H, d) * d ** -0.5
    k = x[:, cols[1]:cols[1] + H * d].view(T, H, d)
    v = x[:, cols[2]:cols[2] + H * dv].view(T, H, dv)
    g = x[:, cols[3]:cols[3] + H * dv]
    a = torch.exp(torch.nn.functional.logsigmoid(z.double() + bias.double()) / tau).view(T, H, d)
    o, S = P.gated_linear_recurrence(q, k, v, a, S0)
    return (P.rms_norm(o, w.double(), eps).reshape(T, H * dv) * g * torch.sigmoid(g)), S


class _Ctx:
    def __init__(self, lens, slots):
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        self.cu_seqlens = torch.tensor(cu, dtype=torch.int32, device=DEV)
        self.slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
        self.n_seqs = len(lens)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cb", [0, 8, 16, 64])
@pytest.mark.parametrize("H,d,dv", [(2, 16, 32), (3, 12, 20), (1, 136, 24), (2, 64, 128), (1, 256, 70)])
def test_gated_linear_attention_over_two_steps_on_shuffled_state_rows(dtype, H, d, dv, cb):
    """Three unequal sequences (one of a single token) on state rows in another order, then a second step of single
    tokens and a piece from the state the first step left; decays from fast to none; the state rows of other
    slots untouched.  With every number of value columns a block that is built, and the launcher's own choice."""
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    tau, eps = 4.0, 1e-5
    cols = (3, 3 + H * d, 5 + 2 * H * d, 5 + 2 * H * d + H * dv)          # a layout with gaps
    width = cols[3] + H * dv + 2
    w = (1.0 + 0.2 * rnd(dv, seed=9)).to(dt)
    bias = 2.0 + 3.0 * rnd(H * d, seed=8)
    S = torch.zeros(6, H, d, dv, device=DEV)
    S[4] = 3.0
    slots = [5, 0, 2]
    states = [None, None, None]
    for step, lens in enumerate(([17, 1, 70], [1, 1, 9])):
        T = sum(lens)
        rows, z = rnd(T, width, seed=10 + step), rnd(T, H * d, seed=20 + step, scale=2.0)
        out = torch.empty(T, H * dv, dtype=dt, device=DEV)
        ops.gla(rows.to(DEV), z.to(DEV), bias.to(DEV), w.to(DEV), out, _Ctx(lens, slots), S, heads=H, head_dim=d,
                value_head_dim=dv, tau=tau, q_scale=d ** -0.5, eps=eps, columns=cols, out_scale=1.5, columns_per_block=cb)
        at = 0
        for i, n in enumerate(lens):
            ref, states[i] = _gla_plain(rows[at:at + n], z[at:at + n], bias, w, H, d, dv, tau, eps, cols, states[i])
            err = max_err(out[at:at + n], 1.5 * ref)
            assert err < (1e-4 if dtype == "float32" else 5e-2) * max(1.0, float(ref.abs().max())), (step, i, err)
            assert max_err(S[slots[i]], states[i]) < 1e-4 * max(1.0, float(states[i].abs().max())), (step, i)
            at += n
    assert float((S[4] - 3.0).abs().max()) == 0.0 and float(S[1].abs().max()) == 0.0 and float(S[3].abs().max()) == 0.0


def test_a_far_token_is_kept_by_a_decay_of_almost_one_and_lost_by_a_fast_one():
    """One key channel that does not decay carries the first token's value over 700 single-token steps; the channel
    beside it decays and has lost it."""
    H, d, dv, T = 1, 4, 8, 700
    cols = (0, d, 2 * d, 2 * d + dv)
    rows = torch.zeros(T, 2 * d + 2 * dv)
    z = torch.zeros(T, d)
    z[:, 0] = 30.0                                        # sigmoid = 1 in 32-bit: no decay
    z[:, 1] = 0.0                                         # sigmoid(0)^(1/2) = 0.707 a step
    rows[0, d + 0] = rows[0, d + 1] = 1.0                 # k of the first token on both channels
    rows[0, 2 * d:2 * d + dv] = torch.arange(1, dv + 1).float()      # its value
    rows[:, cols[3]:] = 10.0                              # gate open: silu(10) = 10
    rows[-1, 0] = 2.0                                     # the last query reads channel 0 (q scale 0.5: 1)
    S = torch.zeros(2, H, d, dv, device=DEV)
    w, bias = torch.ones(dv, device=DEV), torch.zeros(d, device=DEV)
    outs = []
    for t in range(T):
        out = torch.empty(1, dv, dtype=torch.float32, device=DEV)
        ops.gla(rows[t:t + 1].to(DEV), z[t:t + 1].to(DEV), bias, w, out, _Ctx([1], [1]), S, heads=H, head_dim=d,
                value_head_dim=dv, tau=2.0, q_scale=0.5, eps=0.0, columns=cols)
        outs.append(out)
    v = torch.arange(1, dv + 1).double()
    want = v / v.pow(2).mean().sqrt() * 10.0 / (1 + math.exp(-10.0))
    assert max_err(outs[-1][0], want) < 1e-4
    assert max_err(S[1, 0, 0], v) < 1e-5 and float(S[1, 0, 1].abs().max()) < 1e-30


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,I", [(5, 64, 96), (70, 72, 100), (300, 128, 256), (33, 50, 17)])
def test_squared_relu_feed_forward(dtype, T, W, I):
    p = Precision.of(dtype)
    ff = FEED_FORWARDS.get("dense_mlp")(p, hidden_size=W, intermediate_size=I, activation="relu_squared",
                                        tensor_names={"up": "up", "down": "down"})
    ws = {n: rnd(*s.shape, seed=i, scale=0.15).to(torch.bfloat16).to(DEV) for i, (n, s) in enumerate(ff.param_specs().items())}
    assert set(ws) == {"up", "down"}
    for n, t in ws.items():
        ff.assign(n, t)
    ff.finalize()
    x = rnd(T, W, seed=9).to(p.act).to(DEV)
    out = ff.forward(x, None)
    out = out.sum(0) if out.dim() == 3 else out
    ref = P.relu_squared_ff(x.double().cpu(), ws["up"].double().cpu(), ws["down"].double().cpu())
    assert max_err(out, ref) < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))
    with pytest.raises(ValueError, match="activation"):
        FEED_FORWARDS.get("dense_mlp")(p, hidden_size=W, intermediate_size=I, activation="swish")


def test_pass_offset_adds_the_start_from_the_second_pass_on():
    class Stream:
        def flush(self):
            pass
    op = SHARED.get("pass_offset")(Precision.of("float32"), hidden_size=24, passes=3)
    rows = rnd(3, 24, seed=1).to(torch.bfloat16)
    op.assign("step", rows.to(DEV))
    s = Stream()
    x, s.start = rnd(11, 24, seed=2), rnd(11, 24, seed=3).to(DEV)
    for number in range(3):
        s.x = x.clone().to(DEV)
        op.apply(s, None, number)
        want = x + rows[number].float() + (s.start.cpu() if number else 0.0)
        assert max_err(s.x, want) < 1e-6, number
    with pytest.raises(ValueError, match="pass"):
        op.apply(s, None, 3)


# ------------------------------------------------------------------ the model through the engine

@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=512)
    V = plain.c["vocab"]
    for n, seed in ((1, 1), (2, 2), (9, 3), (64, 4), (65, 5), (200, 6)):
        toks = random_tokens(V, n, seed)
        ref = plain.forward(toks)
        s = eng.open(1)
        got = eng.step(s, [toks], "all")
        eng.close(s)
        assert_close(got, ref, dtype, n)
    eng.cache.check_consistent()


@pytest.mark.parametrize("dtype", DTYPES)
def test_residual_stream_after_every_layer_run(dtype):
    """The stream after each run of a layer (a looped layer counts each time), against the plain one."""
    model, plain = pair("tl-a", dtype)
    toks = random_tokens(97, 21, 8)
    _, runs = plain.forward(toks, return_layers=True)
    seen = []
    blocks = [l.block for l in model.lm.layers]
    olds = [b.forward for b in blocks]
    try:
        for b, old in zip(blocks, olds):
            def fwd(stream, ctx, cache, old=old):
                old(stream, ctx, cache)
                stream.flush()
                seen.append(stream.x.clone())
            b.forward = fwd
        eng = model.engine(max_tokens=64, use_graphs=False)
        s = eng.open(1)
        eng.step(s, [toks], "none")
        eng.close(s)
    finally:
        for b, old in zip(blocks, olds):
            b.forward = old
    assert len(seen) == runs.shape[0] == 5
    for i, x in enumerate(seen):
        assert max_err(x, runs[i]) < (2e-5 if dtype == "float32" else 5e-2) * float(runs[i].abs().max()), i


@pytest.mark.parametrize("name,dtype", CASES)
def test_prefix_then_single_tokens_past_windows_chunks_and_pages(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.c["vocab"], 190, 7)
    ref = plain.forward(toks)
    s = eng.open(1)
    got = [eng.step(s, [toks[:50]], "all")]                     # decoding crosses positions 64 and 128, every window and chunk
    for t in toks[50:]:
        got.append(eng.step(s, [[t]], "last"))
    eng.close(s)
    assert_close(torch.cat(got), ref, dtype)


@pytest.mark.parametrize("name,dtype", CASES)
def test_prompt_in_pieces(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.c["vocab"], 180, 9)
    ref = plain.forward(toks)
    for cuts in ([2, 3, 7, 64, 1, 73, 30], [63, 2, 2, 113], [128, 52]):
        assert sum(cuts) == 180
        s = eng.open(1)
        got, at = [], 0
        for c in cuts:
            got.append(eng.step(s, [toks[at:at + c]], "all"))
            at += c
        eng.close(s)
        assert_close(torch.cat(got), ref, dtype, cuts)
    eng.cache.check_consistent()


@pytest.mark.parametrize("name,dtype", CASES)
def test_unequal_batch_against_each_alone_on_reused_slots(name, dtype):
    model, plain = pair(name, dtype)
    V = plain.c["vocab"]
    eng = model.engine(max_tokens=640, max_seqs=4)
    for rnd_ in range(2):                                       # the second round runs on slots and pages used before
        lens = [1, 66, 23, 130] if rnd_ == 0 else [70, 2, 129, 5]
        n_dec = [12, 30, 5, 20]
        seqs = [random_tokens(V, L + d, 20 + 10 * rnd_ + i) for i, (L, d) in enumerate(zip(lens, n_dec))]
        refs = [plain.forward(t) for t in seqs]
        slots = eng.open(4)
        if rnd_ == 1:
            slots = slots[::-1]
        got = [[] for _ in seqs]
        out = eng.step(slots, [t[:L] for t, L in zip(seqs, lens)], "last")
        for b in range(4):
            got[b].append(out[b])
        live = list(range(4))
        for step in range(max(n_dec)):
            live = [b for b in live if step < n_dec[b]]
            out = eng.step([slots[b] for b in live], [[seqs[b][lens[b] + step]] for b in live], "last")
            for r, b in enumerate(live):
                got[b].append(out[r])
            for b in list(live):
                if step + 1 == n_dec[b]:
                    eng.close([slots[b]])                       # shorter requests end earlier and give their slot back
        for b in range(4):
            ref = refs[b][lens[b] - 1:]
            assert_close(torch.stack(got[b]), ref, dtype, (rnd_, b))
        eng.cache.check_consistent()
    assert eng.cache.slots.n_free() == 4


@pytest.mark.parametrize("name,dtype", [("tl-a", "float32"), ("tl-b", "bfloat16"), ("tl-c", "float32"), ("tl-d", "bfloat16")])
def test_long_decoding_from_the_first_token(name, dtype):
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.c["vocab"], 330, 11)
    ref = plain.forward(toks)
    eng = model.engine(max_tokens=384)
    s = eng.open(1)
    got = torch.cat([eng.step(s, [[t]], "last") for t in toks])
    eng.close(s)
    assert_close(got, ref, dtype)


@pytest.mark.parametrize("name", list(TELULORN))
def test_captured_steps_equal_eager_ones(name):
    model, plain = pair(name, "bfloat16")
    toks = [random_tokens(plain.c["vocab"], 40 + 9 * i, 30 + i) for i in range(3)]
    outs = []
    for graphs in (False, True):
        eng = model.engine(max_tokens=512, use_graphs=graphs)
        slots = eng.open(3)
        rows = [eng.step(slots, [t[:20] for t in toks], "last")]
        for j in range(20, 40):
            rows.append(eng.step(slots, [[t[j]] for t in toks], "last"))
        # short pieces of several tokens: recorded at their second sighting
        for rep in range(3):
            eng.close(slots)
            slots = eng.open(3)
            rows.append(eng.step(slots, [t[:7] for t in toks], "last"))
        eng.close(slots)
        outs.append(torch.cat(rows))
    assert max_err(outs[0], outs[1]) < 1e-5


@pytest.mark.parametrize("name,dtype", CASES)
def test_greedy_generation_through_the_entry_point(name, dtype):
    model, plain = pair(name, dtype)
    V = plain.c["vocab"]
    prompts = [random_tokens(V, n, 40 + n) for n in (3, 17, 70)]
    res = model.generate(prompts, max_new_tokens=[10, 6, 12], stop_token_ids=[])
    for p, r, cap in zip(prompts, res, (10, 6, 12)):
        assert len(r.tokens) == cap
        seq = list(p)
        for tok in r.tokens:
            lg = plain.forward(seq)[-1]
            if dtype == "float32":
                assert float(lg.max() - lg[tok]) < 1e-4, "the chosen token is not the plain model's maximum"
            else:
                assert float(lg.max() - lg[tok]) < 0.15 * float(lg.std()) + 0.05
            seq.append(tok)
    model.release_engine()


# ------------------------------------------------------------------ a folder on disk: loader, command line, trace replay
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_of_a_folder(dtype, tmp_path):
    """bin/trace_run on a model folder whose config.json leaves the decay projection's middle to the tensors: prompts of
    unequal lengths as one batch, single tokens together, a request that ends early, one that starts later on the
    slot given back; rows asked for by index."""
    folder = telulorn_folder("tl-d", 5)
    plain = P.PlainTelulorn.from_folder(folder)
    a, b, c = (random_tokens(61, n, 60 + n) for n in (70, 9, 40))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 64, 65]}, {"id": "b", "tokens": b[:7], "want": [6]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]}, {"id": "b", "tokens": b[7:8], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[67:68], "want": []}, {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:69], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "c", "tokens": c[:38], "want": [37]}], "end": []},
             {"step": 5, "entries": [{"id": "c", "tokens": c[38:], "want": [0, 1]}], "end": ["c"]},
             {"step": 6, "entries": [{"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "140"], input="".join(json.dumps(s) + "\n" for s in steps),
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == [f"done {i}" for i in range(7)]
    ra, rb, rc = plain.forward(a), plain.forward(b), plain.forward(c)
    want = {0: torch.stack([ra[0], ra[64], ra[65], rb[6]]), 1: torch.stack([ra[66], rb[7]]), 2: rb[8][None], 3: ra[68][None],
            4: rc[37][None], 5: torch.stack([rc[38], rc[39]]), 6: ra[69][None]}
    got_all, want_all = [], []
    for i, w in want.items():
        got = torch.frombuffer(bytearray((out / f"{i}.f32").read_bytes()), dtype=torch.float32).view(-1, 61)
        assert got.shape == w.shape, i
        got_all.append(got)
        want_all.append(w)
    assert_close(torch.cat(got_all), torch.cat(want_all), dtype)


def test_command_line_generates_from_a_folder():
    folder = telulorn_folder("tl-a", 6)
    plain = P.PlainTelulorn.from_folder(folder)
    proc = subprocess.run([sys.executable, "-m", "alice_llm_amd.generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", "5,9,11,60", "--prompt-ids", "3", "--max-tokens", "5"],
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    for prompt in ([5, 9, 11, 60], [3]):
        ids = plain.greedy(prompt, 5)
        assert ",".join(str(i) for i in ids) in proc.stdout, (ids, proc.stdout[-500:])
