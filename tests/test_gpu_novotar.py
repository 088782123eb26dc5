"""Novotar on the GPU against the plain implementation, in 32-bit and in bfloat16: every mechanism alone, then the
model through the engine: whole prompts, a prefix and then single tokens, prompts in pieces down to two tokens,
unequal batches against each request alone on slots and pages that are used again, long decoding from the first
token, and greedy generation through the package's own entry point."""
import json
import os
import subprocess
import sys

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.cache import Cache
from alice_llm_amd.hip import ops
from alice_llm_amd.parts import FEED_FORWARDS, MIXERS, Precision
from alice_llm_amd.engine.step import StepContext
from helpers import NOVOTAR, max_err, novotar_folder, novotar_pair, random_tokens
from plain import novotar_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = ["float32", "bfloat16"]
CASES = [(n, d) for n in NOVOTAR for d in DTYPES]
# logits here are of order 1 to 10; see helpers.TOL for the two numbers' derivation
TOL = {"float32": 5e-5, "bfloat16": 6e-2}
_PAIRS = {}


def pair(name, dtype):
    if (name, dtype) not in _PAIRS:
        _PAIRS[(name, dtype)] = novotar_pair(name, dtype, seed=len(name) + 7)
    return _PAIRS[(name, dtype)]


def tol(dtype, ref):
    return TOL[dtype] * max(1.0, float(ref.abs().max()))


def row_errors(got, ref):
    """Per row of logits: the root mean square of the difference (means taken off) over that of the row itself."""
    d = got.double().cpu() - ref.double().cpu()
    d = d - d.mean(-1, keepdim=True)
    r = ref.double().cpu() - ref.double().cpu().mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt().clamp_min(1e-9)


def assert_close(got, ref, dtype, what=""):
    """These models' weights are made so that gates close, limits bind and softmaxes are sharp; a rounding ahead of
    such a place is amplified.  The plain implementation itself, run in 32-bit, is within 3e-6 of its 64-bit self
    at the median row and 3e-4 off at the worst rows of these configurations.  32-bit: every logit within 1e-3
    (relative to the largest logit) and the median row within 2e-5.  bfloat16: a row's error is measured as a
    whole (root mean square against the row's own): the rows' mean within 0.06 and nine rows in ten within 0.1
    (of twenty rows and more; every row within 0.3 of fewer).
    A wrong key, state or position moves most rows by 0.3 and more."""
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


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,T", [(5, 40), (64, 200), (65, 200), (1, 9), (300, 130)])
def test_windowed_attention_with_value_size_and_gate(dtype, window, T):
    """A marker key that every query scores far above the others sits just inside the window of one query and just
    outside that of the next; scattered pages; value heads wider than key heads; one gate number a head."""
    H, G, d, dv, page = 4, 2, 24, 40, 64
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    gate = rnd(T, H + 3, seed=4, scale=2.0)
    mark = max(0, T - 20 - window)              # seen by queries up to mark + window - 1, not by mark + window
    q[:, :, 0] = 3.0
    k[:, :, 0] = 0.0
    k[mark, :, 0] = 6.0
    v[mark] += 5.0
    q, k, v, gate = (x.to(dt) for x in (q, k, v, gate))
    ref = P.windowed_attention(q.double(), k.double(), v.double(), 0.5, window) * torch.sigmoid(gate.double()[:, :H, None])
    kp, vp, bt = _paged(k, v, page, 5)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    seq = torch.zeros(T, dtype=torch.int32, device=DEV)
    for rows in (slice(0, T), slice(T - 1, T), slice(mark + window - 1, mark + window + 1)):     # prompt, single token, the edge
        if rows.start < 0 or rows.stop > T:
            continue
        n = rows.stop - rows.start
        out = torch.empty(n, H * dv, dtype=dt, device=DEV)
        ops.attention_generic(q[rows].reshape(n, H * d).contiguous().to(DEV), kp, vp, out, pos[rows].contiguous(),
                              seq[rows].contiguous(), bt, num_heads=H, scale=0.5, softcap=None, window=window,
                              max_position=T - 1, full_precision=dtype == "float32", gate=gate.to(DEV)[rows][:, :H])
        err = max_err(out.view(n, H, dv), ref[rows])
        assert err < (2e-5 if dtype == "float32" else 6e-2), (rows, err)
    if mark + window < T:
        inside, outside = ref[mark + window - 1], ref[mark + window]
        assert (inside - outside).abs().max() > 0.5          # the marker does show


def _mlstm_inputs(T, H, d, dv, seed, hot=3.0):
    row = 2 * H * d + 2 * H * dv + 2 * H
    x = rnd(T, row + 2, seed=seed)
    x[:, -2 - 2 * H:-2] *= hot                                   # raw gate numbers that open and close
    return x


def _mlstm_plain(x, bi, bf, w, H, d, dv, cap, eps, state=None):
    T = x.shape[0]
    x = x.double()
    o = 0
    q = x[:, o:o + H * d].view(T, H, d) * d ** -0.5; o += H * d
    k = x[:, o:o + H * d].view(T, H, d); o += H * d
    v = x[:, o:o + H * dv].view(T, H, dv); o += H * dv
    g = x[:, o:o + H * dv]; o += H * dv
    i = cap * torch.tanh((x[:, o:o + H] + bi.double()) / cap); o += H
    f = P.logsigmoid(cap * torch.tanh((x[:, o:o + H] + bf.double()) / cap))
    out, state = P.mlstm_scan(q, k, v, i, f, state)
    return P.unit_rms(out, eps).reshape(T, H * dv) * w.double() * torch.sigmoid(g), state


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,d,dv", [(2, 16, 32), (3, 8, 40), (1, 64, 128), (2, 32, 16), (1, 128, 64)])
def test_matrix_memory_kernels(dtype, H, d, dv):
    """Three sequences of unequal lengths in one step, on state rows in another order; then a second step (two
    tokens, one token, 70 tokens) from the state the first left; then a state row given back and used again."""
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    cap, eps = 9.0, 1e-5
    lens1, lens2 = [150, 1, 67], [2, 1, 70]
    bi, bf, w = rnd(H, seed=1), rnd(H, seed=2) + 2.0, (1 + 0.2 * rnd(H * dv, seed=3)).to(dt)
    n_slots = 5
    S = torch.zeros(n_slots, H, d, dv, device=DEV); n = torch.zeros(n_slots, H, d, device=DEV); m = torch.zeros(n_slots, H, device=DEV)
    S[4] = 3.0                                                   # a row nobody owns: stays as it is
    slots = torch.tensor([3, 0, 1], dtype=torch.int32, device=DEV)
    states = [None, None, None]
    for step, lens in enumerate((lens1, lens2)):
        T = sum(lens)
        x = _mlstm_inputs(T, H, d, dv, seed=10 + step)
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
        out = torch.empty(T, H * dv, dtype=dt, device=DEV)
        ops.mlstm_rows(x.to(DEV), bi.to(DEV), bf.to(DEV), w.to(DEV), out, cu, slots, S, n, m, n_seqs=3, max_new=max(lens),
                       heads=H, head_dim=d, value_head_dim=dv, cap=cap, eps=eps)
        at = 0
        for b, L in enumerate(lens):
            ref, states[b] = _mlstm_plain(x[at:at + L], bi, bf, w, H, d, dv, cap, eps, states[b])
            err = max_err(out[at:at + L], ref)
            assert err < (3e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max())), (step, b, err)
            at += L
    for b, s in enumerate([3, 0, 1]):
        assert max_err(S[s], states[b][0]) < 1e-4 * max(1.0, float(states[b][0].abs().max()))
        assert max_err(n[s], states[b][1]) < 1e-4 * max(1.0, float(states[b][1].abs().max()))
        assert max_err(m[s], states[b][2]) < 1e-4
    assert torch.all(S[4] == 3.0) and torch.all(S[2] == 0)


def test_matrix_memory_chunks_side_by_side_and_one_after_the_other():
    """A step that leaves the chip unfilled runs its chunks side by side (every chunk's own sums, a walk over the
    chunks' states, then the read-outs); with max_new below a chunk's length the same rows go through the single
    pass.  Both against the plain recurrence, and the states they leave against each other."""
    H, d, dv, cap, eps = 2, 32, 64, 9.0, 1e-5
    lens = [300, 64, 65, 1]
    T = sum(lens)
    x = _mlstm_inputs(T, H, d, dv, seed=21)[:, :2 * H * d + 2 * H * dv + 2 * H].contiguous()   # rows of whole 16-byte units
    bi, bf, w = rnd(H, seed=1), rnd(H, seed=2) + 2.0, 1 + 0.2 * rnd(H * dv, seed=3)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
    slots = torch.tensor([2, 0, 3, 1], dtype=torch.int32, device=DEV)
    ends = []
    for max_new in (max(lens), 64):                             # 64: not above a chunk's length, so the single pass
        S = torch.zeros(4, H, d, dv, device=DEV); n = torch.zeros(4, H, d, device=DEV); m = torch.zeros(4, H, device=DEV)
        out = torch.empty(T, H * dv, device=DEV)
        ops.mlstm_chunks(x.to(DEV), bi.to(DEV), bf.to(DEV), w.to(DEV), out, cu, slots, S, n, m, n_seqs=4, heads=H, head_dim=d,
                         value_head_dim=dv, cap=cap, eps=eps, max_new=max_new)
        at = 0
        for b, L in enumerate(lens):
            ref, st = _mlstm_plain(x[at:at + L], bi, bf, w, H, d, dv, cap, eps)
            assert max_err(out[at:at + L], ref) < 3e-5 * max(1.0, float(ref.abs().max())), (max_new, b)
            assert max_err(S[int(slots[b])], st[0]) < 1e-4 * max(1.0, float(st[0].abs().max()))
            assert max_err(m[int(slots[b])], st[2]) < 1e-4
            at += L
        ends.append((S.clone(), n.clone(), m.clone()))
    for a, b in zip(*ends):
        assert max_err(a, b) < 1e-4 * max(1.0, float(a.abs().max()))


@pytest.mark.parametrize("dtype", DTYPES)
def test_matrix_memory_keeps_a_far_token(dtype):
    """One early token is written with a wide-open input gate while every later forget gate stays open: hundreds of
    tokens on, a query along its key still reads its value."""
    H, d, dv, T = 1, 16, 32, 700
    x = _mlstm_inputs(T, H, d, dv, seed=5, hot=0.0) * 0.1
    o_k, o_v, o_a = H * d, 2 * H * d, 2 * H * d + 2 * H * dv
    x[:, o_a] = -6.0                    # input gates nearly shut,
    x[:, o_a + 1] = 12.0                # forget gates open,
    x[3, o_a] = 6.0                     # but for token 3,
    x[3, o_k:o_k + d] = 0.0; x[3, o_k] = 4.0
    x[3, o_v:o_v + dv] = torch.linspace(-2, 2, dv)
    x[-1, :d] = 0.0; x[-1, 0] = 4.0     # and the last query asks for it
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    w = torch.ones(dv, dtype=dt)
    z = torch.zeros(H)
    out = torch.empty(T, dv, dtype=dt, device=DEV)
    S = torch.zeros(1, H, d, dv, device=DEV); n = torch.zeros(1, H, d, device=DEV); m = torch.zeros(1, H, device=DEV)
    ops.mlstm_rows(x.to(DEV), z.to(DEV), z.to(DEV), w.to(DEV), out, torch.tensor([0, T], dtype=torch.int32, device=DEV),
                   torch.zeros(1, dtype=torch.int32, device=DEV), S, n, m, n_seqs=1, max_new=T, heads=H, head_dim=d,
                   value_head_dim=dv, cap=20.0, eps=1e-6)
    ref, _ = _mlstm_plain(x, z, z, w, H, d, dv, 20.0, 1e-6)
    assert max_err(out, ref) < (1e-4 if dtype == "float32" else 3e-2)
    gated = ref[-1] / torch.sigmoid(x[-1, 2 * H * d + H * dv:2 * H * d + 2 * H * dv].double())
    want = torch.linspace(-2, 2, dv, dtype=torch.float64)
    assert torch.corrcoef(torch.stack([gated, want]))[0, 1] > 0.99


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T", [1, 5, 70, 300])
def test_limited_gated_feed_forward(dtype, T):
    p = Precision.of(dtype)
    W, I, limit = 96, 160, 0.8
    ff = FEED_FORWARDS.get("gated_mlp")(p, hidden_size=W, intermediate_size=I, activation="swish_limited", limit=limit,
                                        tensor_names={"gate": "gate", "up": "up", "down": "down"})
    ws = {n: rnd(*s.shape, seed=i, scale=0.15).to(torch.bfloat16).to(DEV) for i, (n, s) in enumerate(ff.param_specs().items())}
    assert set(ws) == {"gate", "up", "down"}
    for n, t in ws.items():
        ff.assign(n, t)
    ff.finalize()
    x = rnd(T, W, seed=9).to(p.act).to(DEV)
    out = ff.forward(x, None)
    out = out.sum(0) if out.dim() == 3 else out
    ref = P.dense_ff(x.double().cpu(), ws["gate"].double().cpu(), ws["up"].double().cpu(), ws["down"].double().cpu(), limit)
    g = x.double().cpu() @ ws["gate"].double().cpu().T
    assert (g > limit).any() and (g < -limit).any()              # the limits bind, and only from above for the gate
    assert max_err(out, ref) < (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(ref.abs().max()))
    with pytest.raises(ValueError, match="limit"):
        FEED_FORWARDS.get("gated_mlp")(p, hidden_size=W, intermediate_size=I, activation="gelu_tanh", limit=1.0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_token_table_gate_rows(dtype):
    dt = torch.float32 if dtype == "float32" else torch.bfloat16
    T, n, V, width = 37, 24, 50, 72
    z = rnd(T, n, seed=1).to(dt).to(DEV)
    table = rnd(V, width, seed=2).to(torch.bfloat16).to(DEV)
    tokens = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(3)).to(torch.int32).to(DEV)
    out = torch.empty_like(z)
    ops.gelu_mul_rows(z, table, 48, tokens, out, full_precision=dtype == "float32")
    ref = P.gelu_tanh(z.double()) * table.double()[tokens.long()][:, 48:72]
    assert max_err(out, ref) < (1e-6 if dtype == "float32" else 2e-2)
    with pytest.raises(ops.HipLibraryError, match="columns"):
        ops.gelu_mul_rows(z, table, 49, tokens, out, full_precision=True)


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
    model, plain = pair("nv-a", dtype)
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
def test_prefix_then_single_tokens_past_window_and_page(name, dtype):
    model, plain = pair(name, dtype)
    eng = model.engine(max_tokens=256)
    toks = random_tokens(plain.c["vocab"], 190, 7)
    ref = plain.forward(toks)
    s = eng.open(1)
    got = [eng.step(s, [toks[:50]], "all")]                     # decoding crosses positions 64 and 128 and every window
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


@pytest.mark.parametrize("name,dtype", [("nv-a", "float32"), ("nv-b", "bfloat16"), ("nv-c", "float32"), ("nv-c", "bfloat16")])
def test_long_decoding_from_the_first_token(name, dtype):
    model, plain = pair(name, dtype)
    toks = random_tokens(plain.c["vocab"], 330, 11)
    ref = plain.forward(toks)
    eng = model.engine(max_tokens=384)
    s = eng.open(1)
    got = torch.cat([eng.step(s, [[t]], "last") for t in toks])
    eng.close(s)
    assert_close(got, ref, dtype)


@pytest.mark.parametrize("name", list(NOVOTAR))
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
    """bin/trace_run on a model folder: prompts of unequal lengths as one batch, single tokens together, a request
    that ends early, one that starts later on the slot given back; rows asked for by index."""
    from plain.novotar_plain import PlainNovotar
    folder = novotar_folder("nv-d", 5)
    plain = PlainNovotar.from_folder(folder)
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
    from plain.novotar_plain import PlainNovotar
    folder = novotar_folder("nv-a", 6)
    plain = PlainNovotar.from_folder(folder)
    proc = subprocess.run([sys.executable, "-m", "alice_llm_amd.generate", "--model", folder, "--dtype", "float32",
                           "--prompt-ids", "5,9,11,60", "--prompt-ids", "3", "--max-tokens", "5"],
                          capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    for prompt in ([5, 9, 11, 60], [3]):
        ids = plain.greedy(prompt, 5)
        assert ",".join(str(i) for i in ids) in proc.stdout, (ids, proc.stdout[-500:])
