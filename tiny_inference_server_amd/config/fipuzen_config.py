"""Configuration of the Fipuzen decoder, read from its config.json.

Keys: `vocab`, `width`, `norm.eps`, optionally `token_side.dim` (the width of a layer's slice of the per-token side
table; absent: no layer has a token input) and `layers`, a list with one entry per layer: `type` ("attention",
"lightning" or "latent_attention"), `mixer` (the mixer's sizes and constants) and `mlp` ({"kind": "moe", "expert":
{"ff": n}, "router": {"experts", "identity", "top", "scale"}} or null for a layer without a feed-forward).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Tuple

from .fikevik_config import _need, _number

MIXER_TYPES = ("attention", "lightning", "latent_attention")


def _check_mixer(kind, m, where):
    for k in ("heads", "dim", "vdim"):
        _number(m, k, where, int, 1)
    if kind == "attention":
        _number(m, "kv_heads", where, int, 1)
        _need(m["heads"] % m["kv_heads"] == 0, f"{where}: {m['heads']} heads over {m['kv_heads']} kv_heads")
        _number(m, "scale", where, float)
        if m.get("q_temp") is not None:
            _number(m["q_temp"], "coef", where + ".q_temp", float)
            _number(m["q_temp"], "every", where + ".q_temp", int, 1)
    elif kind == "lightning":
        decay = m.get("decay")
        _need(isinstance(decay, (list, tuple)) and len(decay) == m["heads"]
              and all(isinstance(a, (int, float)) and not isinstance(a, bool) for a in decay),
              f"{where}.decay must list one number per head ({m['heads']})")
    else:
        _number(m, "kv_rank", where, int, 1)
        _number(m, "scale", where, float)
        rot_dim = _number(m, "rot_dim", where, int, 0)
        dims = _number(m.get("rot"), "dims", where + ".rot", int, 0) if rot_dim else 0
        if dims:
            _need(_number(m.get("rot"), "base", where + ".rot", float) > 0, f"{where}.rot.base must be positive")
        _need(dims % 2 == 0 and dims <= rot_dim, f"{where}.rot.dims {dims}: an even number, at most rot_dim {rot_dim}")


def _check_layer(i, entry):
    where = f"layers[{i}]"
    _need(isinstance(entry, Mapping), f"{where} must be an object")
    _need(entry.get("type") in MIXER_TYPES, f"{where}.type {entry.get('type')!r}: known are {', '.join(MIXER_TYPES)}")
    _need(isinstance(entry.get("mixer"), Mapping), f"{where}.mixer must be an object")
    _check_mixer(entry["type"], entry["mixer"], where + ".mixer")
    mlp = entry.get("mlp")
    if mlp is not None:
        _need(isinstance(mlp, Mapping) and mlp.get("kind") == "moe", f"{where}.mlp.kind {mlp!r}: known is 'moe'")
        r = mlp.get("router")
        n = _number(r, "experts", where + ".mlp.router", int, 0)
        ident = _number(r, "identity", where + ".mlp.router", int, 0) if "identity" in r else 0
        top = _number(r, "top", where + ".mlp.router", int, 1)
        _need(top <= n + ident, f"{where}.mlp.router.top {top} of {n} + {ident} experts")
        if "scale" in r:
            _number(r, "scale", where + ".mlp.router", float)
        if n:
            _number(mlp.get("expert"), "ff", where + ".mlp.expert", int, 1)


@dataclass(frozen=True)
class FipuzenConfig:
    vocab: int
    width: int
    norm_eps: float
    side_dim: int                      # 0: no per-layer token input
    layers: Tuple[Dict[str, Any], ...]
    architecture: str = "Fipuzen"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)
    side_table_width: int = 0          # columns of the side table; 0: side_dim * layers (a file's table may be wider)

    def __post_init__(self):
        _need(self.vocab >= 1 and self.width >= 1, f"vocab {self.vocab} and width {self.width} must be at least 1")
        _need(self.norm_eps >= 0, f"norm.eps must not be negative, got {self.norm_eps}")
        _need(self.side_dim >= 0, f"token_side.dim must not be negative, got {self.side_dim}")
        _need(len(self.layers) >= 1, "layers must not be empty")
        for i, entry in enumerate(self.layers):
            _check_layer(i, entry)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FipuzenConfig":
        _need(isinstance(raw.get("layers"), list), "config.json lacks 'layers' (a list)")
        used = {"architecture", "vocab", "width", "norm", "token_side", "layers"}
        side = raw.get("token_side")
        return cls(vocab=_number(raw, "vocab", "config", int, 1), width=_number(raw, "width", "config", int, 1),
                   norm_eps=_number(raw.get("norm"), "eps", "norm", float),
                   side_dim=_number(side, "dim", "token_side", int, 0) if side is not None else 0,
                   layers=tuple(copy.deepcopy(dict(e)) if isinstance(e, Mapping) else e for e in raw["layers"]),
                   architecture=str(raw.get("architecture", "Fipuzen")),
                   extra={k: v for k, v in raw.items() if k not in used})

    @property
    def side_width(self) -> int:
        return self.side_table_width or self.side_dim * len(self.layers)

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "FipuzenConfig":
        """The same configuration with the side table's width as the weight file has it (layer i reads the columns
        [i * dim, (i + 1) * dim), whatever lies beyond the last layer's)."""
        shape = shapes.get("side.embed")
        if not self.side_dim or shape is None or len(shape) != 2 or shape[1] < self.side_dim * len(self.layers):
            return self
        return FipuzenConfig(self.vocab, self.width, self.norm_eps, self.side_dim, self.layers, self.architecture,
                             dict(self.extra), int(shape[1]))

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": copy.deepcopy(list(self.layers))}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out
