"""The Fikevik decoder as a spec of parts.

Scaled token embedding into a 32-bit stream; blocks with the norm after the sum, x <- norm(alpha x + gate * sub(x)),
once for the mixer and once for the feed-forward (a layer may have none); a closing RMS norm and an output table of
its own. A layer's mixer is either gated linear attention ("gla") or two mixers side by side on the same input
("parallel"): windowed grouped-query attention with per-head query/key norms, partial rotary, unit-RMS values and a
factor per head on the left, a matrix memory with exponential gating on the right, summed with a factor each. A layer
with `weights_of` is a second call of another layer's block with a cache and state of its own.

Tensor names: `embed`, `head`, `final.norm`, and per layer i that has tensors `l<i>.norm1`, `l<i>.norm2`, `l<i>.rg1`
(+ `.b`), `l<i>.rg2` (+ `.b`), `l<i>.mix.*` (under `.left.` / `.right.` in a parallel layer) and `l<i>.mlp.*`.
"""
from __future__ import annotations

from ..config.fikevik_config import FikevikConfig
from ..config.model_config import ARCHITECTURES, Architecture, ConfigError
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec

NO_CONTEXT_LIMIT = 1 << 30      # nothing in the design bounds a sequence's length


def _norm(cfg, name):
    return PartSpec("norm", "rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps}, {"gain": name})


def _gate(cfg, name):
    return PartSpec("gate", "sigmoid_linear", {"width": cfg.width}, {"w": name, "b": name + ".b"})


def _gla(cfg, m, pre):
    if "rank" not in m:
        raise ConfigError(f"the rank of {pre}a1 is not known: load the configuration from a model folder "
                          f"(the weight file's header gives it) or give mixer.rank")
    params = {"width": cfg.width, "n_heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"], "tau": m["tau"],
              "rank": m["rank"], "eps": cfg.norm_eps}
    names = {k: pre + k for k in ("q", "k", "v", "g", "o", "norm", "a1", "a2")}
    names["a2_bias"] = pre + "a2.b"
    return PartSpec("mixer", "gated_linear_attention", params, names)


def _left(cfg, m, pre):
    params = {"width": cfg.width, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"],
              "value_dim": m["vdim"], "window": m["mask"]["size"], "rot_dims": m["rot"]["dims"],
              "rot_base": m["rot"].get("base", 1.0), "scale": m["scale"], "eps": cfg.norm_eps}
    names = {k: pre + k for k in ("q", "k", "v", "o", "temp")}
    names.update(q_norm=pre + "q.norm", k_norm=pre + "k.norm")
    return PartSpec("mixer", "windowed_qknorm_attention", params, names)


def _right(cfg, m, pre):
    params = {"width": cfg.width, "n_heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"], "gate_cap": m["gate_cap"],
              "eps": cfg.norm_eps}
    names = {k: pre + k for k in ("q", "k", "v", "g", "o", "norm", "i", "f")}
    names.update(i_bias=pre + "i.b", f_bias=pre + "f.b")
    return PartSpec("mixer", "matrix_memory", params, names)


def _block(cfg, entry, i):
    pre = f"l{i}."
    parts = {"mixer_norm": _norm(cfg, pre + "norm1"), "mixer_gate": _gate(cfg, pre + "rg1")}
    scales = {}
    m = entry["mixer"]
    if entry["type"] == "gla":
        parts["mixer"] = _gla(cfg, m, pre + "mix.")
    else:
        parts["left"] = _left(cfg, m["left"], pre + "mix.left.")
        parts["right"] = _right(cfg, m["right"], pre + "mix.right.")
        scales = {"left": m["left_scale"], "right": m["right_scale"]}
    if entry.get("mlp") is not None:
        parts["feed_forward"] = PartSpec("feed_forward", "gated_dense", {"width": cfg.width, "hidden": entry["mlp"]["ff"]},
                                         {k: f"{pre}mlp.{k}" for k in ("gate", "up", "down")})
        parts["feed_forward_norm"] = _norm(cfg, pre + "norm2")
        parts["feed_forward_gate"] = _gate(cfg, pre + "rg2")
    return LayerSpec("postnorm_gated", parts, {"alpha": cfg.postln_alpha, "scales": scales})


def build_spec(cfg: FikevikConfig) -> ModelSpec:
    owners = sorted({cfg.owner_of(i) for i in range(len(cfg.layers))})
    index = {i: n for n, i in enumerate(owners)}
    layers = tuple(_block(cfg, cfg.layers[i], i) for i in owners)
    calls = tuple(LayerCall(index[cfg.owner_of(i)]) for i in range(len(cfg.layers)))
    ignorable = []
    for i in owners:       # a layer without a feed-forward has no second half; a file may still carry its tensors
        if cfg.layers[i].get("mlp") is None:
            ignorable += [f"l{i}.norm2", f"l{i}.rg2", f"l{i}.rg2.b"]
    stage = StageSpec(name="trunk", lag=0,
                      input=PartSpec("stage_input", "scaled_token_embedding", {"scale": cfg.embedding_scale}),
                      calls=calls, out_norm=_norm(cfg, "final.norm"))
    return ModelSpec(d_model=cfg.width, vocab_size=cfg.vocab, max_context=NO_CONTEXT_LIMIT, layers=layers,
                     stages=(stage,), embedding="embed", lm_head="head", eos_token_id=-1, ignorable=tuple(ignorable))


ARCHITECTURES.register("Fikevik", Architecture("Fikevik", FikevikConfig, build_spec))
