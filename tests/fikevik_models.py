"""Small Fikevik configurations with random weights for the tests, and what drives an engine over them.

The sizes differ from one configuration to the next in everything a layer has: head counts on the left and on the
right, key/value heads, key and value sizes (equal in one configuration, different in the others), rotated channels
(all, some, none), windows from 1 to longer than any test sequence, feed-forward widths, a layer without a
feed-forward, layers that run with another layer's tensors (directly and through a chain), models of one mixer kind.
"""
from __future__ import annotations

import copy
import json
import math
import os
from typing import Dict, List

import torch

import plain_fikevik as pf


def parallel(H, G, kd, vd, window, rot, HR, dr, vr, base=10000.0, scale=0.3, cap=12.0, ls=1.3, rs=0.8):
    return {"type": "parallel",
            "mixer": {"left": {"heads": H, "kv_heads": G, "dim": kd, "vdim": vd, "mask": {"size": window},
                               "rot": {"dims": rot, "base": base}, "scale": scale},
                      "right": {"heads": HR, "dim": dr, "vdim": vr, "gate_cap": cap}, "left_scale": ls, "right_scale": rs}}


def gla(H, d, v, tau=8.0):
    return {"type": "gla", "mixer": {"heads": H, "dim": d, "vdim": v, "tau": tau}}


def with_mlp(entry, ff):
    e = copy.deepcopy(entry)
    e["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return e


def shared(entry, j):
    e = copy.deepcopy(entry)
    e["weights_of"] = j
    return e


def config(width, vocab, layers, scale=2.0, eps=1e-5, alpha=1.7):
    return {"architecture": "Fikevik", "vocab": vocab, "width": width, "embedding": {"scale": scale},
            "norm": {"eps": eps}, "postln_alpha": alpha, "layers": layers}


def _configs():
    a0 = with_mlp(parallel(4, 2, 16, 32, 24, 8, 2, 24, 40), 96)
    a1 = with_mlp(gla(3, 20, 24), 80)
    a3 = with_mlp(parallel(6, 3, 8, 24, 9, 0, 1, 16, 16, scale=0.5), 0)
    A = config(64, 211, [a0, a1, shared(a0, 0), a3, shared(a1, 1), shared(shared(a0, 0), 2)], alpha=1.7)
    # keys and values of one size (the pages every attention kernel reads), all channels rotated, a window of 1
    b0 = with_mlp(parallel(2, 1, 32, 32, 40, 32, 3, 32, 16, base=1e6, scale=0.2), 64)
    b1 = with_mlp(parallel(4, 4, 32, 32, 1, 32, 2, 8, 48, scale=0.2), 72)
    B = config(96, 130, [b0, b1, with_mlp(gla(1, 48, 40, tau=3.0), 0)], scale=1.0, eps=1e-6, alpha=1.0)
    # one mixer kind only: no pages at all
    C = config(40, 97, [with_mlp(gla(2, 12, 20, tau=5.0), 56), with_mlp(gla(4, 8, 8, tau=20.0), 0),
                        shared(with_mlp(gla(2, 12, 20, tau=5.0), 56), 0)], scale=3.5, alpha=2.2)
    # a window longer than any sequence of the tests, wide heads, a width that is no multiple of 8
    D = config(76, 150, [with_mlp(parallel(2, 2, 48, 80, 4096, 20, 2, 80, 36, base=1e6, scale=0.15), 120)], alpha=0.9)
    # heads as wide as a served model's (128 channels, values of 256 in the recurrences), keys and values of one size
    e0 = with_mlp(parallel(4, 2, 128, 128, 100, 64, 2, 128, 256, base=2e5, scale=128 ** -0.5), 448)
    E = config(320, 300, [e0, with_mlp(gla(2, 128, 256, tau=12.0), 352), shared(e0, 0)], scale=1.5, alpha=1.2)
    # keys and values of one size that no matrix-core kernel takes (24 channels), no rotation and no rotary base
    f0 = with_mlp(parallel(3, 3, 24, 24, 13, 0, 2, 10, 12, scale=0.3), 40)
    del f0["mixer"]["left"]["rot"]["base"]
    F = config(48, 77, [with_mlp(gla(2, 16, 8, tau=2.0), 64), f0], scale=1.0, alpha=1.4)
    return {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F}


CONFIGS = _configs()
RANK = {"A": 6, "B": 10, "C": 4, "D": 8, "E": 16, "F": 3}


def tensor_shapes(cfg, rank) -> Dict[str, tuple]:
    w, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "head": (cfg["vocab"], cfg["width"]),
                            "final.norm": (cfg["width"],)}
    for i, e in enumerate(cfg["layers"]):
        if "weights_of" in e:
            continue
        p = f"l{i}."
        out.update({p + "norm1": (w,), p + "rg1": (w, w), p + "rg1.b": (w,)})
        m = e["mixer"]
        if e["type"] == "gla":
            H, D, V = m["heads"], m["dim"], m["vdim"]
            out.update({p + "mix.q": (H * D, w), p + "mix.k": (H * D, w), p + "mix.v": (H * V, w), p + "mix.g": (H * V, w),
                        p + "mix.o": (w, H * V), p + "mix.norm": (V,), p + "mix.a1": (rank, w),
                        p + "mix.a2": (H * D, rank), p + "mix.a2.b": (H * D,)})
        else:
            l, r = m["left"], m["right"]
            H, G, kd, vd = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            out.update({p + "mix.left.q": (H * kd, w), p + "mix.left.k": (G * kd, w), p + "mix.left.v": (G * vd, w),
                        p + "mix.left.q.norm": (kd,), p + "mix.left.k.norm": (kd,), p + "mix.left.temp": (H,),
                        p + "mix.left.o": (w, H * vd)})
            H, D, V = r["heads"], r["dim"], r["vdim"]
            q = p + "mix.right."
            out.update({q + "q": (H * D, w), q + "k": (H * D, w), q + "v": (H * V, w), q + "g": (H * V, w),
                        q + "o": (w, H * V), q + "norm": (H * V,), q + "i": (H, w), q + "i.b": (H,), q + "f": (H, w),
                        q + "f.b": (H,)})
        if e.get("mlp"):
            ff = e["mlp"]["ff"]
            out.update({p + "mlp.gate": (ff, w), p + "mlp.up": (ff, w), p + "mlp.down": (w, ff), p + "norm2": (w,),
                        p + "rg2": (w, w), p + "rg2.b": (w,)})
    return out


def random_weights(cfg, rank, seed, storage=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/in), gains 1 +- 0.1, biases that keep memories alive (forget and decay gates open), factors per
    head around 1: every tensor differs from the value that would make it vanish from the result."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg, rank).items()):
        if len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if name in ("embed",):
                t = torch.randn(shape, generator=g)
        elif name.endswith("f.b") or name.endswith("a2.b"):
            t = 2.5 + torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif name.endswith("temp"):
            t = 1.0 + 0.4 * torch.rand(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(storage)
    return out


def write_folder(path, cfg, tensors) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({n: t.contiguous() for n, t in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_f64(tensors):
    return {n: t.to(torch.float64) for n, t in tensors.items()}


_plain: Dict[tuple, torch.Tensor] = {}


def plain_logits(key, cfg, w64, ids) -> torch.Tensor:
    k = (key, tuple(ids))
    if k not in _plain:
        _plain[k] = pf.forward_all(ids, w64, cfg)
    return _plain[k]


def run_trace(engine, steps) -> Dict[tuple, torch.Tensor]:
    """Drive the engine's step function over a list of steps in the replay program's format: {(id, position): logits}."""
    out = {}
    for st in steps:
        starts = {e["id"]: (engine.fed(e["id"]) if e["id"] in engine.requests else 0) for e in st["entries"]}
        lg = engine.step([(e["id"], e["tokens"], e["want"]) for e in st["entries"]]).logits.float().cpu()
        row = 0
        for e in st["entries"]:
            for i in e["want"]:
                out[(e["id"], starts[e["id"]] + i)] = lg[row].clone()
                row += 1
        for rid in st["end"]:
            engine.close(rid)
    return out


def worst_error(key, cfg, w64, reqs: Dict[str, List[int]], got) -> tuple:
    """Largest error over all places that came back: the difference of the logits with its mean taken off, root mean
    square over the vocabulary, over the root mean square of the plain logits of that request. With the place."""
    worst = (0.0, None)
    for rid, ids in reqs.items():
        want = plain_logits(key, cfg, w64, ids)
        scale = float(want.std())
        for p in range(len(ids)):
            if (rid, p) in got:
                d = got[(rid, p)].double() - want[p]
                e = float((d - d.mean()).pow(2).mean().sqrt()) / scale
                if not e <= worst[0]:
                    worst = (e, (rid, p))
    return worst


def sharpen(cfg, tensors, needle: int, probe: int):
    """Make the token `probe` look for the token `needle` in the first layer: in every mixer of layer 0 the query
    matrix becomes the key matrix behind a map that sends the probe's embedding to the needle's, so the probe's query
    is the needle's key (up to rotation) and its score stands out among random ones; the decays of a first layer of
    gated linear attention are moved close to 1, so that a key far back is still there. A key that is wrongly seen or
    wrongly missed, or a state that was lost, then moves the logits by far more than rounding does."""
    t = {n: v.float().clone() for n, v in tensors.items()}
    hp, hn = t["embed"][probe], t["embed"][needle]

    def looking(wk):
        return wk + torch.outer(wk @ (hn - hp), hp) / (hp @ hp)

    e = cfg["layers"][0]
    if e["type"] == "gla":
        t["l0.mix.q"] = 3.0 * looking(t["l0.mix.k"])
        t["l0.mix.a2.b"] = t["l0.mix.a2.b"] + 4.0
        t["l0.mix.a2"] = 0.2 * t["l0.mix.a2"]
    else:
        l = e["mixer"]["left"]
        k = looking(t["l0.mix.left.k"]).view(l["kv_heads"], l["dim"], -1)
        t["l0.mix.left.q"] = k.repeat_interleave(l["heads"] // l["kv_heads"], dim=0).reshape(l["heads"] * l["dim"], -1).clone()
        t["l0.mix.left.temp"] = torch.full_like(t["l0.mix.left.temp"], 4.0 / l["scale"] / math.sqrt(l["dim"]))
        t["l0.mix.left.q.norm"] = torch.ones_like(t["l0.mix.left.q.norm"])
        t["l0.mix.left.k.norm"] = torch.ones_like(t["l0.mix.left.k.norm"])
        t["l0.mix.right.q"] = 3.0 * looking(t["l0.mix.right.k"])
    return {n: v.to(tensors[n].dtype) for n, v in t.items()}


def one_off(cfg, distance):
    """The same configuration with the first layer's window moved by one, so that a key `distance` back changes sides."""
    c = copy.deepcopy(cfg)
    win = cfg["layers"][0]["mixer"]["left"]["mask"]["size"]
    for e in c["layers"]:
        if e["type"] == "parallel" and e["mixer"]["left"]["mask"]["size"] == win:
            e["mixer"]["left"]["mask"]["size"] = win + (1 if distance >= win else -1)
    return c


def relative_error(got, want) -> float:
    d = got.double() - want
    return float((d - d.mean()).pow(2).mean().sqrt() / want.std())


def sharpness(name, cfg, w64, ids, at, distance) -> float:
    """How far the probe's logits (at position at + distance) move if the needle at `at` changes sides: with a window
    in the first layer, the plain implementation with that window one off; without, the sequence without the needle."""
    want = plain_logits((name, "sharp"), cfg, w64, ids)[at + distance]
    if cfg["layers"][0]["type"] == "parallel":
        other = pf.forward_all(ids, w64, one_off(cfg, distance))[at + distance]
    else:
        without = list(ids)
        without[at] = 11
        other = pf.forward_all(without, w64, cfg)[at + distance]
    return relative_error(other, want)
