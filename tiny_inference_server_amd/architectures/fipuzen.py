"""The Fipuzen decoder as a spec of parts.

Token embedding into a 32-bit stream; pre-norm blocks x <- x + mixer(norm1(x)), x <- x + ff(norm2(x)) with layer norms
(gain and bias), then a per-layer token input x <- x + rmsnorm(proj(gelu_tanh(gate x) * side[token])); a closing layer
norm and an output table of its own. A layer's mixer is grouped-query attention with biases, a position-dependent query
factor, a sink in the softmax and a gate per head ("attention"), linear attention with a fixed decay per head
("lightning"), or attention over a low-rank latent with one shared rotated key part ("latent_attention"). The
feed-forward is a mixture of experts with identity experts, or absent.

Tensor names: `embed`, `head`, `final.norm` (+ `.b`), `side.embed`, and per layer i `l<i>.norm1`, `l<i>.norm2` (+ `.b`),
`l<i>.mix.*`, `l<i>.mlp.*` (`router`, `correction`, `e<k>.up`, `e<k>.down`) and `l<i>.side.*` (`gate`, `proj`, `norm`).
"""
from __future__ import annotations

from ..config.fipuzen_config import FipuzenConfig
from ..config.model_config import ARCHITECTURES, Architecture
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec

NO_CONTEXT_LIMIT = 1 << 30      # nothing in the design bounds a sequence's length


def _norm(cfg, name):
    return PartSpec("norm", "layernorm", {"width": cfg.width, "eps": cfg.norm_eps}, {"gain": name, "bias": name + ".b"})


def _attention(cfg, m, pre):
    qt = m.get("q_temp") or {}
    params = {"width": cfg.width, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"],
              "value_dim": m["vdim"], "scale": m["scale"], "temp_coef": qt.get("coef", 0.0), "temp_every": qt.get("every", 1),
              "sink": True, "head_gate": True}
    names = {k: pre + k for k in ("q", "k", "v", "g", "o")}
    names.update(q_bias=pre + "q.b", k_bias=pre + "k.b", v_bias=pre + "v.b")
    return PartSpec("mixer", "sink_gated_attention", params, names)


def _lightning(cfg, m, pre):
    params = {"width": cfg.width, "n_heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"], "decay": tuple(m["decay"]),
              "eps": cfg.norm_eps}
    return PartSpec("mixer", "lightning_attention", params, {k: pre + k for k in ("q", "k", "v", "g", "o", "norm")})


def _latent(cfg, m, pre):
    rot = m.get("rot") or {}
    params = {"width": cfg.width, "n_heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "value_dim": m["vdim"],
              "rank": m["kv_rank"], "rot_dims": rot.get("dims", 0) if m["rot_dim"] else 0, "rot_base": rot.get("base", 1.0),
              "scale": m["scale"], "eps": cfg.norm_eps}
    names = {k: pre + k for k in ("q", "dkv", "uk", "uv", "o")}
    names["dkv_norm"] = pre + "dkv.norm"
    return PartSpec("mixer", "latent_attention", params, names)


_MIXERS = {"attention": _attention, "lightning": _lightning, "latent_attention": _latent}


def _experts(cfg, mlp, pre):
    r = mlp["router"]
    n = r["experts"]
    params = {"width": cfg.width, "hidden": mlp["expert"]["ff"] if n else 0, "n_experts": n,
              "n_identity": r.get("identity", 0), "top": r["top"], "scale": r.get("scale", 1.0)}
    names = {"router": pre + "router", "correction": pre + "correction"}
    for e in range(n):
        names[f"up{e}"] = f"{pre}e{e}.up"
        names[f"down{e}"] = f"{pre}e{e}.down"
    return PartSpec("feed_forward", "routed_experts", params, names)


def _block(cfg, entry, i):
    pre = f"l{i}."
    parts = {"mixer_norm": _norm(cfg, pre + "norm1"), "mixer": _MIXERS[entry["type"]](cfg, entry["mixer"], pre + "mix.")}
    if entry.get("mlp") is not None:
        parts["feed_forward_norm"] = _norm(cfg, pre + "norm2")
        parts["feed_forward"] = _experts(cfg, entry["mlp"], pre + "mlp.")
    if cfg.side_dim:
        params = {"width": cfg.width, "dim": cfg.side_dim, "vocab": cfg.vocab, "table_width": cfg.side_width,
                  "offset": i * cfg.side_dim, "eps": cfg.norm_eps, "act": "gelu_tanh"}
        parts["token_input"] = PartSpec("token_input", "gated_token_table", params,
                                        {"table": "side.embed", "gate": pre + "side.gate", "proj": pre + "side.proj",
                                         "norm": pre + "side.norm"})
    return LayerSpec("prenorm_stream32", parts)


def build_spec(cfg: FipuzenConfig) -> ModelSpec:
    layers = tuple(_block(cfg, entry, i) for i, entry in enumerate(cfg.layers))
    ignorable = []
    for i, entry in enumerate(cfg.layers):     # a layer without a feed-forward has no second norm; a file may carry one
        if entry.get("mlp") is None:
            ignorable += [f"l{i}.norm2", f"l{i}.norm2.b"]
    stage = StageSpec(name="trunk", lag=0, input=PartSpec("stage_input", "scaled_token_embedding", {"scale": 1.0}),
                      calls=tuple(LayerCall(i) for i in range(len(layers))), out_norm=_norm(cfg, "final.norm"))
    return ModelSpec(d_model=cfg.width, vocab_size=cfg.vocab, max_context=NO_CONTEXT_LIMIT, layers=layers,
                     stages=(stage,), embedding="embed", lm_head="head", eos_token_id=-1, ignorable=tuple(ignorable))


ARCHITECTURES.register("Fipuzen", Architecture("Fipuzen", FipuzenConfig, build_spec))
