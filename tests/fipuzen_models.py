"""Small Fipuzen configurations with random weights for the tests, and what the tests need around them.

The configurations differ in everything a layer has: order and kinds of mixers, head counts, key/value heads (one,
some, as many as query heads), key and value sizes (equal and different), query factors (with and without), decays,
latent ranks, rotated parts (all of the rotated part or only some of it), experts and identity experts (none, some,
as many as real ones), top (1 up to all), a layer without a feed-forward, a model without the per-layer token input,
a width that is no multiple of 8.

Routing and bfloat16. An expert is chosen by comparing scores, and a bfloat16 engine that comes within a percent of
the scores can turn a close comparison the other way; the plain implementation would then describe another model. With
random weights some rows of every sequence come that close (`routing_margin` says how close the closest was). So the
engine's bfloat16 tests run the configurations with every expert chosen (`all_chosen`): the weights still follow the
router, no comparison decides anything. Routing itself is tested in 32-bit through the engine, kernel by kernel in both
types, and in bfloat16 through the engine by the median error over a sequence's rows.
"""
from __future__ import annotations

import copy
import math
from typing import Dict, List

import torch

import plain_fipuzen as pz
from fikevik_models import as_f64, relative_error, run_trace, write_folder  # noqa: F401  (the tests use them from here)


def attention(H, G, D, V, scale, coef=None, every=None):
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return {"type": "attention", "mixer": m}


def lightning(H, D, V, decay):
    return {"type": "lightning", "mixer": {"heads": H, "dim": D, "vdim": V, "decay": list(decay)}}


def latent(H, D, R, V, C, scale, dims=None, base=10000.0):
    return {"type": "latent_attention", "mixer": {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": C, "scale": scale,
                                                  "rot": {"dims": R if dims is None else dims, "base": base}}}


def moe(entry, ff, experts, identity, top, scale):
    e = copy.deepcopy(entry)
    e["mlp"] = None if ff is None else {"kind": "moe", "expert": {"ff": ff},
                                        "router": {"experts": experts, "identity": identity, "top": top, "scale": scale}}
    return e


def config(width, vocab, layers, side=None, eps=1e-5):
    c = {"architecture": "Fipuzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if side:
        c["token_side"] = {"dim": side}
    return c


def _configs():
    A = config(64, 211, [moe(attention(4, 2, 16, 24, 0.2, 0.4, 16), 40, 6, 2, 2, 1.7),
                         moe(lightning(3, 8, 20, (0.5, 0.9, 0.99)), 24, 4, 0, 1, 1.0),
                         moe(latent(2, 8, 4, 12, 20, 0.3), None, 0, 0, 0, 0),
                         moe(attention(2, 2, 32, 32, 0.15), 40, 6, 2, 2, 1.7)], side=12)
    # no token input, a width that is no multiple of 8, part of the rotated part left unrotated, as many identity
    # experts as real ones and all of them chosen, one key/value head under six query heads
    B = config(44, 97, [moe(latent(3, 16, 8, 8, 24, 0.2, dims=4, base=50.0), 20, 3, 3, 6, 0.6),
                        moe(lightning(1, 16, 16, (0.97,)), None, 0, 0, 0, 0),
                        moe(attention(6, 1, 8, 8, 0.3, 0.25, 7), 28, 5, 1, 3, 2.0)], eps=1e-6)
    # heads as wide as a served model's; prompts of the tests are long enough for the scan to run in segments
    C = config(128, 300, [moe(attention(4, 1, 64, 64, 0.125, 0.3, 32), 64, 8, 1, 2, 2.2),
                          moe(lightning(2, 64, 64, (0.8, 0.995)), 64, 8, 1, 2, 2.2),
                          moe(latent(4, 32, 16, 32, 64, 0.14, base=1e5), 64, 8, 1, 2, 2.2)], side=8)
    # lightning alone (no pages at all), then attention alone with different key and value sizes and no query factor
    D = config(48, 77, [moe(lightning(2, 12, 8, (0.9, 0.6)), 32, 2, 0, 1, 1.0), moe(lightning(4, 4, 16, (1.0, 0.5, 0.99, 0.7)), None, 0, 0, 0, 0)],
               side=5)
    E = config(56, 150, [moe(attention(3, 3, 20, 36, 0.22), 48, 7, 0, 3, 1.3), moe(attention(2, 1, 40, 16, 0.16, 0.5, 3), None, 0, 0, 0, 0)])
    # attention over a latent first (sizes that the matrix-core kernel takes), then grouped-query attention
    F = config(96, 180, [moe(latent(4, 32, 16, 32, 64, 0.14, base=5e4), 48, 4, 1, 2, 1.5), moe(attention(2, 1, 16, 16, 0.25, 0.3, 64), None, 0, 0, 0, 0)],
               side=6)
    return {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F}


CONFIGS = _configs()


def tensor_shapes(cfg) -> Dict[str, tuple]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "head": (cfg["vocab"], w), "final.norm": (w,), "final.norm.b": (w,)}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        out["side.embed"] = (cfg["vocab"], side * len(cfg["layers"]))
    for i, e in enumerate(cfg["layers"]):
        p, m = f"l{i}.", e["mixer"]
        out.update({p + "norm1": (w,), p + "norm1.b": (w,)})
        H, D, V = m["heads"], m["dim"], m["vdim"]
        q = p + "mix."
        if e["type"] == "attention":
            G = m["kv_heads"]
            out.update({q + "q": (H * D, w), q + "q.b": (H * D,), q + "k": (G * D, w), q + "k.b": (G * D,), q + "v": (G * V, w),
                        q + "v.b": (G * V,), q + "g": (H, w), q + "o": (w, H * V)})
        elif e["type"] == "lightning":
            out.update({q + "q": (H * D, w), q + "k": (H * D, w), q + "v": (H * V, w), q + "g": (H * V, w), q + "o": (w, H * V),
                        q + "norm": (H * V,)})
        else:
            R, C = m["rot_dim"], m["kv_rank"]
            out.update({q + "q": (H * (D + R), w), q + "dkv": (C + R, w), q + "dkv.norm": (C,), q + "uk": (H * D, C),
                        q + "uv": (H * V, C), q + "o": (w, H * V)})
        if e.get("mlp"):
            r = e["mlp"]["router"]
            out.update({p + "norm2": (w,), p + "norm2.b": (w,), p + "mlp.router": (r["experts"] + r["identity"], w),
                        p + "mlp.correction": (r["experts"] + r["identity"],)})
            for k in range(r["experts"]):
                out.update({f"{p}mlp.e{k}.up": (e["mlp"]["expert"]["ff"], w), f"{p}mlp.e{k}.down": (w, e["mlp"]["expert"]["ff"])})
        if side:
            out.update({p + "side.gate": (side, w), p + "side.proj": (w, side), p + "side.norm": (w,)})
    return out


def random_weights(cfg, seed, storage=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/in); tables N(0, 1); gains 1 +- 0.1; biases and corrections that differ from zero; a router
    strong enough for its scores to differ between experts."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        if name in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g)
        elif name.endswith("router"):
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith("correction"):
            t = 0.05 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(storage)
    return out


# ---- the plain implementation, kept per sequence ------------------------------------------------------------------

_plain: Dict[tuple, tuple] = {}


def plain(key, cfg, w64, ids):
    """(logits [T, vocab], the smallest routing margin of the sequence) from the plain implementation."""
    k = (key, tuple(ids))
    if k not in _plain:
        margins: List[float] = []
        _plain[k] = (pz.forward(cfg, w64, list(ids), margins=margins), min(margins, default=math.inf))
    return _plain[k]


def plain_logits(key, cfg, w64, ids):
    return plain(key, cfg, w64, ids)[0]


def routing_margin(key, cfg, w64, ids) -> float:
    return plain(key, cfg, w64, ids)[1]


def worst_error(key, cfg, w64, reqs: Dict[str, List[int]], got) -> tuple:
    """Largest error over all places that came back: the difference of the logits with its mean taken off, root mean
    square over the vocabulary, over the spread of the plain logits of that request. With the place."""
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


TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def check(key, cfg, w64, reqs, got, dtype):
    """32-bit: every place within 3e-5 of the plain logits' spread. bfloat16: 98 of 100 places within 4 %, none beyond
    25 %. The design norms short vectors (a layer's token input is a handful of gated numbers, projected and divided by
    its own root mean square), and where such a vector happens to be small its rounding is blown up to full size: a
    single row then differs by several percent while its neighbours differ by a few tenths. The torch stand-in for
    the kernels, run in bfloat16 on the host, shows the same rows with the same errors."""
    errs = []
    for rid, ids in reqs.items():
        want = plain_logits(key, cfg, w64, ids)
        scale = float(want.std())
        for p in range(len(ids)):
            if (rid, p) in got:
                d = got[(rid, p)].double() - want[p]
                errs.append((float((d - d.mean()).pow(2).mean().sqrt()) / scale, (rid, p)))
    errs.sort()
    if dtype == "float32":
        assert errs[-1][0] <= TOL[dtype], errs[-1]
    else:
        assert errs[int(0.98 * (len(errs) - 1))][0] <= TOL[dtype], errs[int(0.98 * (len(errs) - 1))]
        assert errs[-1][0] <= 0.25, errs[-1]


# ---- weights that make one key stand out ----------------------------------------------------------------------------

def sharpen(cfg, tensors, needle: int, probe: int, strength: float = 6.0):
    """Make the token `probe` look for the token `needle` in the first layer's mixer: its query matrix becomes the key
    matrix behind a map that sends the probe's normed embedding to the needle's, so that the probe's query is the
    needle's key and that one score stands out among hundreds. Biases of queries and keys are cleared so that nothing
    else lifts every score alike. In a lightning layer the decays in the configuration decide how much of a far key is
    left; the test chooses them."""
    t = {n: v.float().clone() for n, v in tensors.items()}
    eps = cfg["norm"]["eps"]

    def normed(tok):
        x = t["embed"][tok].double()
        return pz.layer_norm(x, t["l0.norm1"].double(), t["l0.norm1.b"].double(), eps).float()

    hp, hn = normed(probe), normed(needle)

    def looking(wk):
        return wk + torch.outer(wk @ (hn - hp), hp) / (hp @ hp)

    e, m = cfg["layers"][0], cfg["layers"][0]["mixer"]
    if e["type"] == "attention":
        k = looking(t["l0.mix.k"]).view(m["kv_heads"], m["dim"], -1)
        q = k.repeat_interleave(m["heads"] // m["kv_heads"], dim=0).reshape(m["heads"] * m["dim"], -1)
        kn = (t["l0.mix.k"] @ hn).view(m["kv_heads"], m["dim"]).norm(dim=-1).mean()
        t["l0.mix.q"] = q * (strength / m["scale"] / float(kn) ** 2)
        t["l0.mix.q.b"].zero_()
        t["l0.mix.k.b"].zero_()
    elif e["type"] == "lightning":
        t["l0.mix.q"] = looking(t["l0.mix.k"])
    else:
        # a head's unrotated query becomes its own unrotated key of the needle: Wuk[h] applied to the needle's latent
        # (the gain times the latent's rows, behind the map from the probe to the needle; the norm's factor is a
        # number per position and goes into the strength)
        H, D, R, C = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
        rows = looking(t["l0.mix.dkv.norm"][:, None] * t["l0.mix.dkv"][:C])            # [C, width]
        uk = t["l0.mix.uk"].view(H, D, C)
        q = t["l0.mix.q"].view(H, D + R, -1).clone()
        down = t["l0.mix.dkv"][:C] @ hn
        c_n = down / torch.sqrt((down * down).mean() + eps) * t["l0.mix.dkv.norm"]
        hit = torch.stack([(uk[h] @ rows @ hp) @ (uk[h] @ c_n) for h in range(H)]).mean()
        for h in range(H):
            q[h, :D] = uk[h] @ rows * (strength / m["scale"] / float(hit))
        t["l0.mix.q"] = q.reshape(H * (D + R), -1)
    return {n: v.to(tensors[n].dtype) for n, v in t.items()}


def all_chosen(cfg):
    """The same configuration with every expert of every layer chosen for every row: the weights still follow the
    router, but no comparison of scores decides anything, so a bfloat16 engine and the plain implementation describe
    the same model however close two scores come."""
    c = copy.deepcopy(cfg)
    for e in c["layers"]:
        if e.get("mlp"):
            r = e["mlp"]["router"]
            r["top"] = r["experts"] + r["identity"]
    return c
