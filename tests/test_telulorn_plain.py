"""Telulorn on the CPU: the configuration reader and its refusals, the plan's order of layer runs, tensor names and
shapes, the cache's bookkeeping for kept first positions and chunks, and the plain implementation's own invariants
(a recurrence cut in two, the edges of a window and of a chunk, the first positions, the sink, values that are
turned and turned back, the mix of the heads, the loop)."""
import json
import math

import pytest
import torch

import alice_llm_amd as alice
from alice_llm_amd.cache import Cache
from alice_llm_amd.engine.model import CausalLM
from alice_llm_amd.parts import CacheNeed, KVNeed, Precision
from helpers import TELULORN, telulorn_tensors
from plain import telulorn_plain as P


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# ------------------------------------------------------------------ configuration and plan

def test_architecture_is_found_by_its_key_and_round_trips():
    raw = TELULORN["tl-a"]()
    cfg = alice.config_from_dict(raw)
    assert type(cfg).__name__ == "TelulornConfig" and "Telulorn" in alice.registered_architectures()
    assert alice.config_from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    assert cfg.layer_runs() == [(0, None), (1, 0), (2, None), (1, 1), (2, None)] == P.layer_runs(raw)
    plan = cfg.plan()
    assert [(e.layer, e.before, e.before_arg) for e in plan.schedule] == \
        [(0, None, None), (1, "loop", 0), (2, None, None), (1, "loop", 1), (2, None, None)]
    assert plan.layers[2].feed_forward is None and "pre_ff" not in plan.layers[2].norms
    left, right = plan.layers[0].mixer.args["sides"]
    assert left.args["chunk"] == 7 and left.args["window"] is None and left.args["output_scale"] == 0.8
    assert right.args["tau"] == 4.0 and right.args["decay_rank"] == 8 and right.args["output_scale"] == 1.3
    assert plan.layers[1].mixer.args["window"] == 9 and plan.layers[1].mixer.args["keep_first"] == 3
    assert left.args["score_bias_slopes"] == pytest.approx(P.distance_slopes(4).tolist())
    assert plan.head.args["tied_to"] == "embed"


def test_defaults_and_absent_keys():
    raw = TELULORN["tl-d"]()
    plan = alice.config_from_dict(raw).plan()
    assert plan.layers[2].mixer.args["window"] is None and plan.layers[2].mixer.args["keep_first"] == 0
    assert plan.layers[2].mixer.args["position"] is None and len(plan.positions) == 1
    assert plan.layers[0].mixer.args["keep_first"] == 0 and plan.layers[0].mixer.args["window"] == 33
    assert plan.layers[1].mixer.args["sides"][0].args["chunk"] is None
    no_loop = alice.config_from_dict(TELULORN["tl-b"]()).plan()
    assert not no_loop.shared and all(e.before is None for e in no_loop.schedule)
    names = set(CausalLM(no_loop, Precision.of("float32"), "cpu").param_specs())
    assert "loop.step" not in names and "head" not in names and "l1.mix.sink" in names


def test_tensor_names_and_shapes():
    cfg = alice.config_from_dict(TELULORN["tl-a"]())
    specs = {k: tuple(v.shape) for k, v in CausalLM(cfg.plan(), Precision.of("float32"), "cpu").param_specs().items()}
    want = {"embed": (97, 64), "loop.step": (2, 64), "l0.norm1": (64,), "l0.norm2": (64,), "l0.mix.left.q": (64, 64),
            "l0.mix.left.k": (32, 64), "l0.mix.left.v": (64, 64), "l0.mix.left.talk": (4, 4), "l0.mix.left.g": (128, 64),
            "l0.mix.left.o": (64, 128), "l0.mix.right.q": (32, 64), "l0.mix.right.v": (64, 64), "l0.mix.right.g": (64, 64),
            "l0.mix.right.o": (64, 64), "l0.mix.right.norm": (32,), "l0.mix.right.a1": (8, 64), "l0.mix.right.a2": (32, 8),
            "l0.mix.right.a2.b": (32,), "l0.mlp.up": (96, 64), "l0.mlp.down": (64, 96), "l1.mix.q": (128, 64),
            "l1.mix.q.b": (128,), "l1.mix.k": (32, 64), "l1.mix.k.b": (32,), "l1.mix.v": (16, 64), "l1.mix.v.b": (16,),
            "l1.mix.sink": (4,), "l1.mix.g": (64, 64), "l1.mix.o": (64, 64), "final.norm": (64,)}
    for name, shape in want.items():
        assert specs.get(name) == shape, (name, specs.get(name))
    assert "l2.norm2" not in specs and "l2.mlp.up" not in specs


def test_the_decay_projections_middle_comes_from_the_tensor_shapes():
    raw = TELULORN["tl-b"]()
    del raw["layers"][0]["mixer"]["right"]["rank"]
    cfg = alice.config_from_dict(raw)
    with pytest.raises(alice.ConfigError, match="middle"):
        cfg.plan()
    full = cfg.with_tensor_shapes({"l0.mix.right.a1": (5, 72), "embed": (130, 72)})
    assert full.plan().layers[0].mixer.args["sides"][1].args["decay_rank"] == 5


@pytest.mark.parametrize("change,match", [
    (lambda r: r["layers"][1].update(type="conv"), "no mixer"),
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda r: r["layers"][1]["mixer"]["rot"].update(dims=17), "rot"),
    (lambda r: r["layers"][1]["mixer"]["mask"].update(size=0), "mask"),
    (lambda r: r["layers"][0]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda r: r["loop"].update(stop=9), "loop"),
    (lambda r: r["layers"][0]["mlp"].update(kind="routed"), "feed-forward"),
    (lambda r: r.pop("width"), "width"),
])
def test_refusals(change, match):
    raw = TELULORN["tl-a"]()
    change(raw)
    with pytest.raises(alice.ConfigError, match=match):
        alice.config_from_dict(raw)


# ------------------------------------------------------------------ cache bookkeeping

def test_kept_first_pages_stay_and_the_rest_of_the_window_moves():
    need = CacheNeed(kv=KVNeed(1, 8, window=10, keep_first=20))            # pages of 8: the first three stay
    c = Cache([need], max_tokens=200, dtype=torch.float32, device="cpu", page_size=8, allocate=False)
    s = c.open()
    c.reserve([s], [70])
    c.commit([s], [70])
    tab = c.groups[0].table(s)
    assert [p >= 0 for p in tab] == [True, True, True, False, False, False, False, True, True]
    for _ in range(30):
        c.reserve([s], [1])
        c.commit([s], [1])
    tab = c.groups[0].table(s)
    assert all(p >= 0 for p in tab[:3]) and all(p < 0 for p in tab[3:11]) and all(p >= 0 for p in tab[11:])
    c.check_consistent()
    c.close(s)
    c.check_consistent()
    assert c.groups[0].n_free() == c.groups[0].n_pages


# ------------------------------------------------------------------ the plain implementation's own invariants

def test_recurrence_cut_in_two_and_from_a_state():
    T, H, d, dv = 23, 2, 5, 7
    q, k, v = rnd(T, H, d, seed=1), rnd(T, H, d, seed=2), rnd(T, H, dv, seed=3)
    a = torch.sigmoid(rnd(T, H, d, seed=4, scale=3.0))
    o, S = P.gated_linear_recurrence(q, k, v, a)
    o1, S1 = P.gated_linear_recurrence(q[:9], k[:9], v[:9], a[:9])
    o2, S2 = P.gated_linear_recurrence(q[9:], k[9:], v[9:], a[9:], S1)
    assert torch.allclose(torch.cat([o1, o2]), o, atol=1e-12) and torch.allclose(S2, S, atol=1e-12)
    # the closed form: o_t = sum_j (prod_{j < r <= t} a_r . k_j . q_t) v_j, the decay on the key channels
    t = 6
    want = sum(((a[j + 1:t + 1].prod(0) * k[j] * q[t]).sum(-1, keepdim=True) * v[j]) for j in range(t + 1))
    assert torch.allclose(o[t], want, atol=1e-10)


def test_decay_is_sigmoid_to_the_power_one_over_tau():
    h = rnd(4, 6, seed=1)
    p = {"a1": rnd(3, 6, seed=2), "a2": rnd(10, 3, seed=3), "a2.b": rnd(10, seed=4)}
    a = P.decay(h, p, {"heads": 2, "dim": 5, "tau": 4.0})
    z = (h @ p["a1"].T) @ p["a2"].T + p["a2.b"]
    assert torch.allclose(a.reshape(4, 10), torch.sigmoid(z) ** 0.25, atol=1e-12)


def test_masks_at_their_edges():
    m = P.window_mask(40, 5, 3)
    assert m[10, 6] and not m[10, 5] and m[10, 2] and not m[10, 3] and m[10, 10] and not m[10, 11]
    assert P.window_mask(9, None, 0).sum() == 45
    c = P.chunk_mask(40, 7)
    assert c[13, 7] and not c[13, 6] and not c[14, 13] and c[14, 14] and c[20, 14] and not c[6, 7]
    assert P.chunk_mask(9, None).sum() == 45


def test_sink_takes_weight_and_has_no_value():
    T, H, d = 6, 2, 4
    q, k, v = rnd(T, H, d, seed=1), rnd(T, H, d, seed=2), torch.ones(T, H, 3, dtype=torch.float64)
    mask = P.window_mask(T, None, 0)
    plain = P.sink_attention(q, k, v, mask, 0.5, None)
    assert torch.allclose(plain, torch.ones_like(plain))              # weights sum to one
    sink = torch.tensor([0.0, 50.0], dtype=torch.float64)
    out = P.sink_attention(q, k, v, mask, 0.5, sink)
    assert (out[:, 0] < 1).all() and (out[:, 0] > 0).all() and float(out[:, 1].abs().max()) < 1e-15
    s0 = (q[0, 0] @ k[0, 0]) * 0.5                                    # one key and the sink, which counts once, unscaled
    assert math.isclose(float(out[0, 0, 0]), math.exp(s0) / (math.exp(s0) + 1.0), rel_tol=1e-12)


def test_values_turned_and_turned_back_enter_by_the_distance():
    T, dv, base = 9, 6, 50.0
    v = rnd(T, 1, dv, seed=1)
    pos = torch.arange(T)
    w = torch.softmax(rnd(T, T, seed=2).masked_fill(~P.window_mask(T, None, 0), -math.inf), dim=1)
    out = P.rotate_pairs((w @ P.rotate_pairs(v, pos, base, dv)[:, 0])[:, None], pos, base, dv, sign=-1.0)[:, 0]
    i = 7
    want = sum(w[i, j] * P.rotate_pairs(v[j:j + 1], torch.tensor([j - i]), base, dv)[0, 0] for j in range(i + 1))
    assert torch.allclose(out[i], want, atol=1e-12)
    # pairs are neighbours, and only the first `dims` dimensions turn
    x = torch.zeros(1, 1, 6, dtype=torch.float64)
    x[0, 0, 0] = 1.0
    x[0, 0, 5] = 2.0
    y = P.rotate_pairs(x, torch.tensor([1]), 10.0, 4)
    assert math.isclose(float(y[0, 0, 0]), math.cos(1.0)) and math.isclose(float(y[0, 0, 1]), math.sin(1.0)) and float(y[0, 0, 5]) == 2.0


def test_mixed_heads_keep_their_own_values_and_the_distance_term_is_taken_off():
    T, H, G, d, dv = 7, 4, 2, 3, 2
    q, k, v = rnd(T, H, d, seed=1), rnd(T, G, d, seed=2), rnd(T, G, dv, seed=3)
    mask = P.chunk_mask(T, None)
    eye = P.talking_attention(q, k, v, mask, 1.0, P.distance_slopes(H), torch.eye(H, dtype=torch.float64))
    none = P.talking_attention(q, k, v, mask, 1.0, P.distance_slopes(H), None)
    assert torch.allclose(eye, none)
    swap = torch.zeros(H, H, dtype=torch.float64)
    swap[0, 3] = 1.0                                                   # head 0 takes head 3's weights, and its own kv head's values
    out = P.talking_attention(q, k, v, mask, 1.0, P.distance_slopes(H), swap)
    s = q[:, 3] @ k[:, 1].T - P.distance_slopes(H)[3] * (torch.arange(T)[:, None] - torch.arange(T)[None, :])
    want = torch.softmax(s.masked_fill(~mask, -math.inf), dim=1) @ v[:, 0]
    assert torch.allclose(out[:, 0], want, atol=1e-12) and float(out[:, 1:].abs().max()) == 0.0
    assert P.distance_slopes(8)[7] == 2.0 ** -8 and P.distance_slopes(8)[0] == 0.5


def test_the_loop_and_causality():
    raw = TELULORN["tl-a"]()
    _, tensors = telulorn_tensors(raw, 3)
    plain = P.PlainTelulorn(raw, tensors)
    toks = [5, 9, 11, 60, 3, 3, 70, 1, 8, 8, 2, 90]
    full, runs = plain.forward(toks, return_layers=True)
    assert runs.shape == (5, 12, 64)
    assert torch.allclose(plain.forward(toks[:7]), full[:7], atol=1e-9)       # nothing looks ahead
    once = dict(raw, loop={"start": 1, "stop": 3, "times": 1})
    w1 = dict(tensors)
    w1["loop.step"] = tensors["loop.step"][:1]
    assert not torch.allclose(P.PlainTelulorn(once, w1).forward(toks), full, atol=1e-3)
    moved = dict(tensors)
    moved["loop.step"] = tensors["loop.step"].clone()
    moved["loop.step"][1] += 1.0
    _, runs2 = P.PlainTelulorn(raw, moved).forward(toks, return_layers=True)
    assert torch.allclose(runs2[:3], runs[:3]) and not torch.allclose(runs2[3], runs[3], atol=1e-3)
