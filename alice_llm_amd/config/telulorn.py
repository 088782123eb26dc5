"""Telulorn: typed configuration from config.json, and its plan.

A pre-norm decoder whose layers are written out one by one in config.json (`layers`: per layer its `type`, the
sizes of its `mixer` and its `mlp`, which may be null), with a run of layers that is repeated with the same
weights (`loop`: start, stop, times; before every pass but the first the embedding output is added to the
stream, and before every pass a learned row of that pass).  The feed-forward is up, squared ReLU, down; the
output head is the embedding matrix.  Two mixer types:

  "attention"  grouped-query attention with biases on q, k and v; rotation of neighbouring pairs over the first
               `rot.dims` dimensions of q and k; values turned by their position over all their dimensions and
               the head's output turned back by the query's; a sliding window (`mask.size`) that keeps the
               first `mask.keep_first` positions visible; a learned sink a head in the softmax's denominator;
               an elementwise sigmoid gate before the output matrix.
  "parallel"   two mixers on the same input, their outputs added with the constant factors `left_scale` and
               `right_scale`: "left" is attention without rotation, with a distance term slope_h * (i - j)
               taken off the scores (slope_h = 2^(-8 (h + 1) / heads)), keys of the query's own chunk of
               `mask.size` positions only, the heads' softmax weights mixed by a learned matrix, and the
               elementwise gate; "right" is gated linear attention (a matrix state a head with a decay per key
               channel, sigmoid(.)^(1 / tau), from a projection through a narrow middle), normed per head
               and gated by silu.

Everything here is data for the builder: which registered part, with which constants, under which tensor
names.  Sizes and constants come from config.json, and the one size that only the tensors give (the width of
the decay projection's middle) from their shapes (`with_tensor_shapes`); what the design fixes is in the parts
and kernels.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .novotar import _obj
from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry, read_key, require

DEFAULT_MAX_POSITIONS = 65536        # the design has no position limit of its own; tables are sized by this
SLOPE_EXPONENT = 8.0                 # slope_h = 2^(-SLOPE_EXPONENT (h + 1) / heads)


def distance_slopes(heads: int):
    return [2.0 ** (-SLOPE_EXPONENT * (h + 1) / heads) for h in range(heads)]


def _read_heads(m: Mapping[str, Any], where: str, kv: bool) -> Dict[str, Any]:
    heads, dim = read_key(m, "heads", int), read_key(m, "dim", int)
    out = {"heads": heads, "dim": dim, "vdim": read_key(m, "vdim", int, dim)}
    if kv:
        out["kv_heads"] = read_key(m, "kv_heads", int, heads)
        out["scale"] = read_key(m, "scale", float)
        require(heads % out["kv_heads"] == 0, f"{where}kv_heads must divide heads")
    for k, v in out.items():
        require(k == "scale" or v >= 1, f"{where}{k} must be at least 1")
    return out


@dataclass(frozen=True)
class TelulornConfig:
    vocab: int
    width: int
    layers: Tuple[Mapping[str, Any], ...]          # as config.json gives them, validated
    norm_eps: float = 1e-6
    loop: Optional[Tuple[int, int, int]] = None    # (start, stop, times)
    max_positions: int = DEFAULT_MAX_POSITIONS
    torch_dtype: str = "bfloat16"

    architecture = "Telulorn"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "TelulornConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        norm = _obj(d, "norm", "", optional=True) or {}
        loop = _obj(d, "loop", "", optional=True)
        if loop is not None:
            loop = (read_key(loop, "start", int), read_key(loop, "stop", int), read_key(loop, "times", int))
        cfg = cls(vocab=read_key(d, "vocab", int), width=read_key(d, "width", int),
                  layers=tuple(cls._read_layer(i, l) for i, l in enumerate(raw_layers)),
                  norm_eps=read_key(norm, "eps", float, 1e-6), loop=loop,
                  max_positions=read_key(d, "max_positions", int, DEFAULT_MAX_POSITIONS),
                  torch_dtype=read_key(d, "torch_dtype", str, "bfloat16"))
        cfg.validate()
        return cfg

    @staticmethod
    def _read_layer(i: int, l: Any) -> Dict[str, Any]:
        where = f"layers[{i}]: "
        if not isinstance(l, Mapping):
            raise ConfigError(f"config.json: {where}must be an object")
        kind = read_key(l, "type", str)
        require(kind in ("parallel", "attention"), f"{where}type '{kind}' has no mixer here (known: 'attention', 'parallel')")
        mixer = _obj(l, "mixer", where)
        if kind == "attention":
            out = _read_heads(mixer, where + "mixer.", kv=True)
            mask = _obj(mixer, "mask", where + "mixer: ", optional=True)
            out["mask"] = None if mask is None else {"size": read_key(mask, "size", int),
                                                     "keep_first": read_key(mask, "keep_first", int, 0)}
            rot = _obj(mixer, "rot", where + "mixer: ", optional=True)
            out["rot"] = None if rot is None else {"base": read_key(rot, "base", float),
                                                   "dims": read_key(rot, "dims", int, out["dim"])}
        else:
            left, right = _obj(mixer, "left", where + "mixer: "), _obj(mixer, "right", where + "mixer: ")
            out_left = _read_heads(left, where + "mixer.left.", kv=True)
            mask = _obj(left, "mask", where + "mixer.left: ", optional=True)
            out_left["mask"] = None if mask is None else {"size": read_key(mask, "size", int)}
            out_right = _read_heads(right, where + "mixer.right.", kv=False)
            out_right["tau"] = read_key(right, "tau", float)
            rank = read_key(right, "rank", int, 0)        # not a key of the files: the tensors' shapes give it
            if rank:
                out_right["rank"] = rank
            out = {"left": out_left, "right": out_right, "left_scale": read_key(mixer, "left_scale", float, 1.0),
                   "right_scale": read_key(mixer, "right_scale", float, 1.0)}
        mlp = _obj(l, "mlp", where, optional=True)
        out_mlp = None
        if mlp is not None:
            mk = read_key(mlp, "kind", str, "dense")
            require(mk == "dense", f"{where}mlp kind '{mk}' has no feed-forward here (known: 'dense')")
            out_mlp = {"kind": mk, "ff": read_key(mlp, "ff", int)}
        return {"type": kind, "mixer": out, "mlp": out_mlp}

    def validate(self) -> None:
        require(self.vocab >= 1 and self.width >= 1, "vocab and width must be at least 1")
        require(self.norm_eps > 0, "norm.eps must be positive")
        require(self.max_positions >= 1, "max_positions must be at least 1")
        L = len(self.layers)
        if self.loop is not None:
            a, b, n = self.loop
            require(0 <= a < b <= L, f"loop start {a} and stop {b} must satisfy 0 <= start < stop <= {L}")
            require(n >= 1, f"loop times must be at least 1, found {n}")
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "attention":
                require(m["mask"] is None or (m["mask"]["size"] >= 1 and m["mask"]["keep_first"] >= 0),
                        f"layers[{i}].mixer.mask: size must be at least 1 and keep_first not negative")
                if m["rot"] is not None:
                    require(m["rot"]["base"] > 0 and 0 <= m["rot"]["dims"] <= m["dim"] and m["rot"]["dims"] % 2 == 0,
                            f"layers[{i}].mixer.rot: base must be positive, dims even and at most dim")
                    require(m["vdim"] % 2 == 0, f"layers[{i}].mixer.vdim must be even (the values are turned in pairs)")
            else:
                require(m["left"]["mask"] is None or m["left"]["mask"]["size"] >= 1,
                        f"layers[{i}].mixer.left.mask.size must be at least 1")
                require(m["right"]["tau"] > 0, f"layers[{i}].mixer.right.tau must be positive")
            require(l["mlp"] is None or l["mlp"]["ff"] >= 1, f"layers[{i}].mlp.ff must be at least 1")
        require(self.torch_dtype in ("bfloat16", "float32"), f"torch_dtype must be 'bfloat16' or 'float32', found '{self.torch_dtype}'")

    def to_dict(self) -> dict:
        d: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "norm": {"eps": self.norm_eps}, "layers": [_plain(l) for l in self.layers],
                             "max_positions": self.max_positions, "torch_dtype": self.torch_dtype}
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return d

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "TelulornConfig":
        """The configuration with the sizes that only a folder's tensors give: the width of the middle of each
        "right" mixer's decay projection is the number of rows of `l<i>.mix.right.a1`."""
        layers = []
        for i, l in enumerate(self.layers):
            name = f"l{i}.mix.right.a1"
            if l["type"] == "parallel" and "rank" not in l["mixer"]["right"] and name in shapes and len(shapes[name]) == 2:
                l = dict(l, mixer=dict(l["mixer"], right=dict(l["mixer"]["right"], rank=int(shapes[name][0]))))
            layers.append(l)
        return replace(self, layers=tuple(layers))

    # ------------------------------------------------------------------ derived
    def layer_runs(self):
        """[(layer, the number of the pass that starts with this run, or None)] in the order in which the layers run."""
        L = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(L)]
        a, b, n = self.loop
        runs = [(i, None) for i in range(a)]
        for r in range(n):
            runs += [(i, r if i == a else None) for i in range(a, b)]
        return runs + [(i, None) for i in range(b, L)]

    # ------------------------------------------------------------------ the plan
    def _attention(self, m) -> PartSpec:
        mask, rot = m["mask"], m["rot"]
        return PartSpec("attention", {
            "hidden_size": self.width, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_head_dim": m["vdim"], "scale": m["scale"], "softcap": None,
            "window": None if mask is None else mask["size"], "keep_first": 0 if mask is None else mask["keep_first"],
            "position": None if rot is None else _rot_name(m), "bias": True, "sink": True, "output_gate": "elementwise",
            "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "sink": "sink"}}, "mix")

    def _parallel(self, i: int, m) -> PartSpec:
        le, ri = m["left"], m["right"]
        if "rank" not in ri:
            raise ConfigError(f"config.json: layers[{i}].mixer.right: the width of the decay projection's middle is not "
                              f"known (the tensors' shapes give it when a folder is loaded; 'rank' names it otherwise)")
        left = PartSpec("attention", {
            "hidden_size": self.width, "num_heads": le["heads"], "num_kv_heads": le["kv_heads"], "head_dim": le["dim"],
            "value_head_dim": le["vdim"], "scale": le["scale"], "softcap": None, "window": None,
            "chunk": None if le["mask"] is None else le["mask"]["size"], "position": None,
            # the term taken off the scores: the kernel adds slope * (key position - query position)
            "score_bias_slopes": distance_slopes(le["heads"]), "talk": True, "output_gate": "elementwise",
            "output_scale": m["left_scale"],
            "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "talk": "talk"}}, "left")
        right = PartSpec("gla", {
            "hidden_size": self.width, "num_heads": ri["heads"], "head_dim": ri["dim"], "value_head_dim": ri["vdim"],
            "decay_rank": ri["rank"], "tau": ri["tau"], "norm_eps": self.norm_eps, "output_scale": m["right_scale"]}, "right")
        return PartSpec("side_by_side", {"hidden_size": self.width, "sides": (left, right), "norm_eps": self.norm_eps,
                                         "side_norms": False}, "mix")

    def plan(self) -> ModelPlan:
        W, eps = self.width, self.norm_eps
        norm = lambda name: PartSpec("rmsnorm", {"dim": W, "eps": eps, "weight_offset": 0.0, "tensor_name": ""}, name)
        layers, positions = [], {}
        for i, l in enumerate(self.layers):
            m = l["mixer"]
            if l["type"] == "attention":
                mixer = self._attention(m)
                if m["rot"] is not None:
                    positions[_rot_name(m)] = PartSpec("rope_pairs", {
                        "dim": m["dim"], "theta": m["rot"]["base"], "rotary_dim": m["rot"]["dims"], "value_dim": m["vdim"],
                        "max_positions": self.max_positions, "interleaved": True})
            else:
                mixer = self._parallel(i, m)
            ff, norms = None, {"pre_mixer": norm("norm1")}
            if l["mlp"] is not None:
                ff = PartSpec("dense_mlp", {"hidden_size": W, "intermediate_size": l["mlp"]["ff"], "activation": "relu_squared",
                                            "tensor_names": {"up": "up", "down": "down"}}, "mlp")
                norms["pre_ff"] = norm("norm2")
            layers.append(LayerPlan(block="prenorm", mixer=mixer, feed_forward=ff, norms=norms, prefix=f"l{i}."))
        shared = {}
        if self.loop is not None:
            shared["loop"] = PartSpec("pass_offset", {"hidden_size": W, "passes": self.loop[2], "tensor_name": "step"})
        schedule = tuple(ScheduleEntry(i, before=None if r is None else "loop", before_arg=r) for i, r in self.layer_runs())
        return ModelPlan(
            vocab_size=self.vocab, hidden_size=W, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "dim": W, "scale": 1.0, "tensor_name": ""}, "embed"),
            positions=positions, layers=tuple(layers), schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "dim": W, "softcap": None, "tied_to": "embed"}, "head"),
            stop_token_ids=(), shared=shared)


def _rot_name(m) -> str:
    """One table set per distinct (head size, rotated width, base, value size)."""
    return f"pairs_{m['dim']}_{m['rot']['dims']}_{m['rot']['base']!r}_{m['vdim']}"


def _plain(x):
    if isinstance(x, Mapping):
        return {k: _plain(v) for k, v in x.items()}
    return x
