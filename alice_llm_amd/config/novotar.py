"""Novotar: typed configuration from config.json, and its plan.

A decoder whose layers are written out one by one in config.json (`layers`: per layer its `type`, the sizes
of its `mixer` and its `mlp`, which may be null), with a run of layers that is repeated with the same weights
(`loop`: start, stop, times; before each repetition the stream and the embedding output go through one
matrix), one norm per layer whose output feeds the mixer and the feed-forward side by side, and a gated
per-layer input from a second token table (`token_side`).  The mixer type "parallel" is two mixers on the
same input: windowed grouped-query attention without positions and with a gate per head ("left"), and the
mLSTM matrix memory ("right"); each side's output is RMS-normed over the width and the two are averaged.

Everything here is data for the builder: which registered part, with which constants, under which tensor
names.  Sizes and constants come from config.json; what the design fixes is in the parts and kernels.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .plan import ConfigError, LayerPlan, ModelPlan, PartSpec, ScheduleEntry, read_key, require

DEFAULT_MAX_POSITIONS = 65536        # the design has no position limit of its own; tables are sized by this


def _obj(d: Mapping[str, Any], key: str, where: str, optional: bool = False) -> Optional[Mapping[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"config.json: {where}'{key}' is missing")
    if not isinstance(v, Mapping):
        raise ConfigError(f"config.json: {where}'{key}' must be an object, found {v!r}")
    return v


@dataclass(frozen=True)
class NovotarConfig:
    vocab: int
    width: int
    layers: Tuple[Mapping[str, Any], ...]          # as config.json gives them, validated
    embedding_scale: float = 1.0
    norm_eps: float = 1e-6
    loop: Optional[Tuple[int, int, int]] = None    # (start, stop, times)
    token_side_dim: Optional[int] = None
    max_positions: int = DEFAULT_MAX_POSITIONS
    torch_dtype: str = "bfloat16"

    architecture = "Novotar"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "NovotarConfig":
        V = read_key(d, "vocab", int)
        W = read_key(d, "width", int)
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = tuple(cls._read_layer(i, l) for i, l in enumerate(raw_layers))
        emb = _obj(d, "embedding", "", optional=True) or {}
        norm = _obj(d, "norm", "", optional=True) or {}
        loop = _obj(d, "loop", "", optional=True)
        if loop is not None:
            loop = (read_key(loop, "start", int), read_key(loop, "stop", int), read_key(loop, "times", int))
        side = _obj(d, "token_side", "", optional=True)
        cfg = cls(vocab=V, width=W, layers=layers,
                  embedding_scale=read_key(emb, "scale", float, 1.0),
                  norm_eps=read_key(norm, "eps", float, 1e-6),
                  loop=loop,
                  token_side_dim=None if side is None else read_key(side, "dim", int),
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
        require(kind == "parallel", f"{where}type '{kind}' has no mixer here (known: 'parallel')")
        mixer = _obj(l, "mixer", where)
        left, right = _obj(mixer, "left", where + "mixer: "), _obj(mixer, "right", where + "mixer: ")
        mask = _obj(left, "mask", where + "mixer.left: ", optional=True)
        heads = read_key(left, "heads", int)
        dim = read_key(left, "dim", int)
        out_left = {"heads": heads, "kv_heads": read_key(left, "kv_heads", int, heads), "dim": dim,
                    "vdim": read_key(left, "vdim", int, dim), "scale": read_key(left, "scale", float),
                    "mask": None if mask is None else {"size": read_key(mask, "size", int)}}
        rdim = read_key(right, "dim", int)
        out_right = {"heads": read_key(right, "heads", int), "dim": rdim, "vdim": read_key(right, "vdim", int, rdim),
                     "gate_cap": read_key(right, "gate_cap", float)}
        mlp = _obj(l, "mlp", where, optional=True)
        out_mlp = None
        if mlp is not None:
            mk = read_key(mlp, "kind", str, "dense")
            require(mk == "dense", f"{where}mlp kind '{mk}' has no feed-forward here (known: 'dense')")
            out_mlp = {"kind": mk, "ff": read_key(mlp, "ff", int), "limit": read_key(mlp, "limit", float)}
        return {"type": kind, "mixer": {"left": out_left, "right": out_right}, "mlp": out_mlp}

    def validate(self) -> None:
        require(self.vocab >= 1 and self.width >= 1, "vocab and width must be at least 1")
        require(self.norm_eps > 0, "norm.eps must be positive")
        require(self.max_positions >= 1, "max_positions must be at least 1")
        L = len(self.layers)
        if self.loop is not None:
            a, b, n = self.loop
            require(0 <= a < b <= L, f"loop start {a} and stop {b} must satisfy 0 <= start < stop <= {L}")
            require(n >= 1, f"loop times must be at least 1, found {n}")
        require(self.token_side_dim is None or self.token_side_dim >= 1, "token_side.dim must be at least 1")
        for i, l in enumerate(self.layers):
            le, ri = l["mixer"]["left"], l["mixer"]["right"]
            for k in ("heads", "kv_heads", "dim", "vdim"):
                require(le[k] >= 1, f"layers[{i}].mixer.left.{k} must be at least 1")
            require(le["heads"] % le["kv_heads"] == 0, f"layers[{i}].mixer.left: kv_heads must divide heads")
            require(le["mask"] is None or le["mask"]["size"] >= 1, f"layers[{i}].mixer.left.mask.size must be at least 1")
            for k in ("heads", "dim", "vdim"):
                require(ri[k] >= 1, f"layers[{i}].mixer.right.{k} must be at least 1")
            require(ri["gate_cap"] > 0, f"layers[{i}].mixer.right.gate_cap must be positive")
            if l["mlp"] is not None:
                require(l["mlp"]["ff"] >= 1 and l["mlp"]["limit"] > 0, f"layers[{i}].mlp: ff and limit must be positive")
        require(self.torch_dtype in ("bfloat16", "float32"), f"torch_dtype must be 'bfloat16' or 'float32', found '{self.torch_dtype}'")

    def to_dict(self) -> dict:
        d: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                             "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                             "layers": [dict(l) for l in self.layers], "max_positions": self.max_positions,
                             "torch_dtype": self.torch_dtype}
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        if self.token_side_dim is not None:
            d["token_side"] = {"dim": self.token_side_dim}
        return d

    # ------------------------------------------------------------------ derived
    def layer_runs(self):
        """[(layer, starts a repetition of the loop)] in the order in which the layers run."""
        L = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(L)]
        a, b, n = self.loop
        runs = [(i, False) for i in range(a)]
        for _ in range(n):
            runs += [(i, i == a) for i in range(a, b)]
        return runs + [(i, False) for i in range(b, L)]

    # ------------------------------------------------------------------ the plan
    def plan(self) -> ModelPlan:
        W, eps = self.width, self.norm_eps
        norm = lambda name: PartSpec("rmsnorm", {"dim": W, "eps": eps, "weight_offset": 0.0, "tensor_name": ""}, name)
        layers = []
        for i, l in enumerate(self.layers):
            le, ri = l["mixer"]["left"], l["mixer"]["right"]
            left = PartSpec("attention", {
                "hidden_size": W, "num_heads": le["heads"], "num_kv_heads": le["kv_heads"], "head_dim": le["dim"],
                "value_head_dim": le["vdim"], "scale": le["scale"], "softcap": None,
                "window": None if le["mask"] is None else le["mask"]["size"], "position": None,
                "output_gate": "head",
                "tensor_names": {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g"},
            }, "left")
            right = PartSpec("mlstm", {
                "hidden_size": W, "num_heads": ri["heads"], "head_dim": ri["dim"], "value_head_dim": ri["vdim"],
                "gate_cap": ri["gate_cap"], "norm_eps": eps,
            }, "right")
            mixer = PartSpec("side_by_side", {"hidden_size": W, "sides": (left, right), "norm_eps": eps,
                                              "norm_tensor": "out"}, "mix")
            ff = None
            if l["mlp"] is not None:
                ff = PartSpec("gated_mlp", {"hidden_size": W, "intermediate_size": l["mlp"]["ff"],
                                            "activation": "swish_limited", "limit": l["mlp"]["limit"],
                                            "tensor_names": {"gate": "gate", "up": "up", "down": "down"}}, "mlp")
            extras = {}
            if self.token_side_dim is not None:
                d = self.token_side_dim
                extras["token_input"] = PartSpec("token_gate", {"hidden_size": W, "dim": d, "column": i * d,
                                                                "table": "side", "norm_eps": eps}, "side")
            layers.append(LayerPlan(block="parallel", mixer=mixer, feed_forward=ff, norms={"pre": norm("norm1")},
                                    prefix=f"l{i}.", extras=extras))
        shared = {}
        if self.token_side_dim is not None:
            shared["side"] = PartSpec("token_table", {"vocab_size": self.vocab, "dim": len(self.layers) * self.token_side_dim,
                                                      "tensor_name": "embed"})
        if self.loop is not None:
            shared["loop"] = PartSpec("reinject", {"hidden_size": W, "tensor_name": "in"})
        schedule = tuple(ScheduleEntry(i, before="loop" if first else None) for i, first in self.layer_runs())
        return ModelPlan(
            vocab_size=self.vocab, hidden_size=W, max_positions=self.max_positions,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab, "dim": W, "scale": self.embedding_scale,
                                             "tensor_name": ""}, "embed"),
            positions={}, layers=tuple(layers), schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("lm_head", {"vocab_size": self.vocab, "dim": W, "softcap": None, "tied_to": None,
                                      "tensor_name": ""}, "head"),
            stop_token_ids=(), shared=shared)
