"""Configuration of the Fikevik decoder, read from its config.json.

Keys: `vocab`, `width`, `embedding.scale`, `norm.eps`, `postln_alpha` and `layers`, a list with one entry per layer:
`type` ("gla" or "parallel"), `mixer` (the mixer's sizes and constants), `mlp` ({"kind": "dense", "ff": n} or null
for a layer without a feed-forward) and optionally `weights_of`: j, which makes the layer run with layer j's tensors
and a cache or state of its own. One size is in no key: the rank of a "gla" mixer's decay projection is the first
dimension of its `mix.a1` tensor, so `with_tensor_shapes` completes the configuration from the weight file's header
(a config.json may also give it as `rank` in the mixer's entry).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Tuple

from .model_config import ConfigError

MIXER_TYPES = ("gla", "parallel")


def _need(cond, msg):
    if not cond:
        raise ConfigError(msg)


def _number(d, key, where, kind=float, minimum=None):
    _need(isinstance(d, Mapping) and key in d, f"config.json lacks {where}.{key}")
    v = d[key]
    _need(not isinstance(v, bool) and isinstance(v, (int, float)), f"{where}.{key} must be a number, got {v!r}")
    if kind is int:
        _need(float(v) == int(v), f"{where}.{key} must be an integer, got {v!r}")
        v = int(v)
    else:
        v = float(v)
    if minimum is not None:
        _need(v >= minimum, f"{where}.{key} must be at least {minimum}, got {v}")
    return v


def _check_recurrent(m, where):
    for k in ("heads", "dim", "vdim"):
        _number(m, k, where, int, 1)


def _check_layer(i, entry, n_layers):
    where = f"layers[{i}]"
    _need(isinstance(entry, Mapping), f"{where} must be an object")
    _need(entry.get("type") in MIXER_TYPES, f"{where}.type {entry.get('type')!r}: known are {', '.join(MIXER_TYPES)}")
    m = entry.get("mixer")
    _need(isinstance(m, Mapping), f"{where}.mixer must be an object")
    if entry["type"] == "gla":
        _check_recurrent(m, where + ".mixer")
        _number(m, "tau", where + ".mixer", float)
        _need(m["tau"] > 0, f"{where}.mixer.tau must be positive")
        if "rank" in m:
            _number(m, "rank", where + ".mixer", int, 1)
    else:
        left, right = m.get("left"), m.get("right")
        _need(isinstance(left, Mapping) and isinstance(right, Mapping), f"{where}.mixer needs 'left' and 'right'")
        lw = where + ".mixer.left"
        for k in ("heads", "kv_heads", "dim", "vdim"):
            _number(left, k, lw, int, 1)
        _need(left["heads"] % left["kv_heads"] == 0, f"{lw}: {left['heads']} heads over {left['kv_heads']} kv_heads")
        _number(left, "scale", lw, float)
        _number(left.get("mask"), "size", lw + ".mask", int, 1)
        dims = _number(left.get("rot"), "dims", lw + ".rot", int, 0)
        if dims:
            _need(_number(left.get("rot"), "base", lw + ".rot", float) > 0, f"{lw}.rot.base must be positive")
        _need(dims % 2 == 0 and dims <= left["dim"], f"{lw}.rot.dims {dims}: an even number, at most dim {left['dim']}")
        _check_recurrent(right, where + ".mixer.right")
        _number(right, "gate_cap", where + ".mixer.right", float)
        _need(right["gate_cap"] > 0, f"{where}.mixer.right.gate_cap must be positive")
        _number(m, "left_scale", where + ".mixer", float)
        _number(m, "right_scale", where + ".mixer", float)
    mlp = entry.get("mlp")
    if mlp is not None:
        _need(isinstance(mlp, Mapping) and mlp.get("kind") == "dense", f"{where}.mlp.kind {mlp!r}: known is 'dense'")
        _number(mlp, "ff", where + ".mlp", int, 1)
    if "weights_of" in entry:
        j = _number(entry, "weights_of", where, int, 0)
        _need(j < n_layers and j != i, f"{where}.weights_of {j} names no other layer")


@dataclass(frozen=True)
class FikevikConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    postln_alpha: float
    layers: Tuple[Dict[str, Any], ...]
    architecture: str = "Fikevik"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    def __post_init__(self):
        _need(self.vocab >= 1 and self.width >= 1, f"vocab {self.vocab} and width {self.width} must be at least 1")
        _need(self.norm_eps >= 0, f"norm.eps must not be negative, got {self.norm_eps}")
        _need(len(self.layers) >= 1, "layers must not be empty")
        for i, entry in enumerate(self.layers):
            _check_layer(i, entry, len(self.layers))
        for i in range(len(self.layers)):
            j = self.owner_of(i)
            if j != i:
                _need(self.layers[j]["type"] == self.layers[i]["type"],
                      f"layers[{i}] is {self.layers[i]['type']!r} but takes the weights of layers[{j}], a {self.layers[j]['type']!r}")

    def owner_of(self, i: int) -> int:
        """The layer whose tensors layer i runs with."""
        seen = set()
        while "weights_of" in self.layers[i]:
            _need(i not in seen, f"layers[{i}].weights_of goes in a circle")
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FikevikConfig":
        _need(isinstance(raw.get("layers"), list), "config.json lacks 'layers' (a list)")
        used = {"architecture", "vocab", "width", "embedding", "norm", "postln_alpha", "layers"}
        return cls(vocab=_number(raw, "vocab", "config", int, 1), width=_number(raw, "width", "config", int, 1),
                   embedding_scale=_number(raw.get("embedding"), "scale", "embedding", float),
                   norm_eps=_number(raw.get("norm"), "eps", "norm", float),
                   postln_alpha=_number(raw, "postln_alpha", "config", float),
                   layers=tuple(copy.deepcopy(dict(e)) if isinstance(e, Mapping) else e for e in raw["layers"]),
                   architecture=str(raw.get("architecture", "Fikevik")),
                   extra={k: v for k, v in raw.items() if k not in used})

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "postln_alpha": self.postln_alpha, "layers": copy.deepcopy(list(self.layers))}

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "FikevikConfig":
        """The same configuration with every size that only a tensor's shape gives filled in."""
        layers = copy.deepcopy(list(self.layers))
        for i, entry in enumerate(layers):
            if entry["type"] == "gla" and "rank" not in entry["mixer"]:
                name = f"l{self.owner_of(i)}.mix.a1"
                if name in shapes and len(shapes[name]) == 2:
                    entry["mixer"]["rank"] = int(shapes[name][0])
        return FikevikConfig(self.vocab, self.width, self.embedding_scale, self.norm_eps, self.postln_alpha, tuple(layers),
                             self.architecture, dict(self.extra))
