"""The Fipuzen architecture on the host: its configuration and spec, the plain implementation's mechanisms against
closed forms, and the engine (step function, cache manager, scheduler, generate) on the torch stand-ins for the kernels
against the plain implementation, in 32-bit."""
import copy
import math

import pytest
import torch

import fipuzen_models as ZM
import helpers as H
import plain_fipuzen as pz
from torch_ops import TorchOps
from tiny_inference_server_amd.config import ARCHITECTURES, ConfigError, config_from_dict, load_config
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.weights.loader import spec_tensors

TOL32 = 3e-5
F64 = torch.float64


def model(name, seed=5):
    cfg = ZM.CONFIGS[name]
    w = ZM.random_weights(cfg, seed)
    return cfg, w, ZM.as_f64(w)


def engine_for(cfg, w, **kw):
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 8)
    kw.setdefault("max_tokens", 640)
    return Engine(config=config_from_dict(cfg), tensors={n: t.float() for n, t in w.items()}, dtype="float32",
                  ops=TorchOps(graphs=kw.pop("graphs", False)), **kw)


# ---- configuration and spec ------------------------------------------------------------------------------------

def test_spec_names_every_tensor(tmp_path):
    for name, cfg in ZM.CONFIGS.items():
        w = ZM.random_weights(cfg, 1)
        folder = ZM.write_folder(str(tmp_path / name), cfg, w)
        c = load_config(folder)
        assert c.to_dict() == config_from_dict(c.to_dict()).to_dict()
        spec = ARCHITECTURES.get(c.architecture).build_spec(c)
        assert spec_tensors(spec) == {n: tuple(t.shape) for n, t in w.items()}
        assert len(spec.stages[0].calls) == len(spec.layers) == len(cfg["layers"])
        for layer, entry in zip(spec.layers, cfg["layers"]):
            assert ("feed_forward" in layer.parts) == (entry["mlp"] is not None)
            assert ("token_input" in layer.parts) == ("token_side" in cfg)


def test_a_side_table_wider_than_the_layers_need(tmp_path):
    """Layer i reads the columns [i * dim, (i + 1) * dim) of the side table; the table's width comes from the file."""
    cfg, w, _ = model("D")
    w = dict(w)
    w["side.embed"] = torch.cat((w["side.embed"], torch.randn(cfg["vocab"], 3).to(w["side.embed"].dtype)), dim=1)
    folder = ZM.write_folder(str(tmp_path / "wide"), cfg, w)
    assert load_config(folder).side_width == w["side.embed"].shape[1]
    eng = Engine(folder, dtype="float32", max_tokens=64, max_requests=2, page_size=8, ops=TorchOps())
    ids = H.random_ids(cfg["vocab"], 20, 3)
    got = ZM.run_trace(eng, H.whole_trace({"a": ids}))
    assert ZM.worst_error("Dwide", cfg, ZM.as_f64(w), {"a": ids}, got)[0] <= TOL32


def test_configuration_errors_name_the_key():
    good = ZM.CONFIGS["A"]
    for path, value, word in [(("layers", 0, "type"), "conv", "type"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 1, "mixer", "decay"), [0.5], "decay"), (("layers", 2, "mixer", "rot", "dims"), 3, "rot.dims"),
                              (("layers", 0, "mlp", "kind"), "dense", "mlp"), (("layers", 0, "mlp", "router", "top"), 9, "top"),
                              (("layers", 0, "mixer", "q_temp", "every"), 0, "every"), (("norm",), {}, "eps")]:
        bad = copy.deepcopy(good)
        d = bad
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            config_from_dict(bad)


# ---- the plain implementation's mechanisms against closed forms ----------------------------------------------------

def test_plain_sink_softmax_and_query_factor():
    torch.manual_seed(0)
    s = torch.randn(5, 5, dtype=F64) * 3
    vis = pz.causal(5)
    p = pz.sink_softmax(s, vis)
    for i in range(5):
        e = torch.exp(s[i, :i + 1])
        assert torch.allclose(p[i, :i + 1], e / (1.0 + e.sum()), atol=1e-14)
        assert p[i, i + 1:].abs().sum() == 0
    assert (p.sum(-1) < 1).all()                      # what is missing went to the sink
    # scores far below zero: nearly everything goes to the sink and nothing overflows
    assert pz.sink_softmax(torch.full((1, 3), -800.0, dtype=F64), torch.ones(1, 3, dtype=torch.bool)).sum() == 0
    f = pz.query_temperature(40, 0.5, 8)
    assert f[0] == 1.0 and f[6] == 1.0 and torch.isclose(f[7], torch.tensor(1 + 0.5 * math.log(2.0), dtype=F64))
    assert f[14] == f[7] and torch.isclose(f[15], torch.tensor(1 + 0.5 * math.log(3.0), dtype=F64))


def test_plain_lightning_is_the_decayed_sum():
    torch.manual_seed(1)
    T, W, Hh, D, V = 9, 12, 2, 4, 3
    m = {"heads": Hh, "dim": D, "vdim": V, "decay": [0.8, 0.3]}
    t = {"q": torch.randn(Hh * D, W), "k": torch.randn(Hh * D, W), "v": torch.randn(Hh * V, W), "g": torch.randn(Hh * V, W),
         "o": torch.eye(Hh * V), "norm": torch.rand(Hh * V) + 0.5}
    h = torch.randn(T, W, dtype=F64)
    got = pz.lightning(h, t, "", m, 1e-6)
    q, k = (pz.silu(h @ t[n].double().T).view(T, Hh, D) for n in ("q", "k"))
    v = pz.silu(h @ t["v"].double().T).view(T, Hh, V)
    o = torch.zeros(T, Hh, V, dtype=F64)
    for i in range(T):
        for j in range(i + 1):
            for hd in range(Hh):
                o[i, hd] += m["decay"][hd] ** (i - j) * (q[i, hd] @ k[j, hd]) * v[j, hd]
    o = o.reshape(T, -1)
    want = o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-6) * t["norm"].double() * torch.sigmoid(h @ t["g"].double().T)
    assert torch.allclose(got, want, atol=1e-10)


def test_plain_latent_attention_both_ways():
    """Keys and values built from the latent for every head, against the products moved to the query's side."""
    torch.manual_seed(2)
    T, W, Hh, D, R, V, C = 11, 10, 3, 4, 6, 5, 7
    m = {"heads": Hh, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": C, "scale": 0.4, "rot": {"dims": 4, "base": 30.0}}
    t = {n: torch.randn(s) for n, s in {"q": (Hh * (D + R), W), "dkv": (C + R, W), "uk": (Hh * D, C), "uv": (Hh * V, C),
                                        "o": (W, Hh * V)}.items()}
    t["dkv.norm"] = torch.rand(C) + 0.5
    h = torch.randn(T, W, dtype=F64)
    got = pz.latent_attention(h, t, "", m, 1e-5)
    pos = torch.arange(T)
    q = (h @ t["q"].double().T).view(T, Hh, D + R)
    down = h @ t["dkv"].double().T
    c = pz.rms_norm(down[:, :C], t["dkv.norm"].double(), 1e-5)
    key = torch.cat((c, pz.rotate_pairs(down[:, C:], pos, 4, 30.0)), dim=-1)
    out = torch.zeros(T, Hh, V, dtype=F64)
    for hd in range(Hh):
        uk, uv = t["uk"].double().view(Hh, D, C)[hd], t["uv"].double().view(Hh, V, C)[hd]
        qq = torch.cat((q[:, hd, :D] @ uk, pz.rotate_pairs(q[:, hd, D:], pos, 4, 30.0)), dim=-1)
        p = pz.plain_softmax(qq @ key.T * 0.4, pz.causal(T))
        out[:, hd] = (p @ c) @ uv.T
    assert torch.allclose(got, out.reshape(T, -1) @ t["o"].double().T, atol=1e-10)
    # rotation: a pair's scalar product depends on the distance alone, and the channels beyond `dims` pass unchanged
    x, y = torch.randn(1, 6, dtype=F64).expand(3, 6), torch.randn(1, 6, dtype=F64).expand(3, 6)
    a, b = pz.rotate_pairs(x, torch.tensor([3, 10, 40]), 4, 50.0), pz.rotate_pairs(y, torch.tensor([1, 8, 38]), 4, 50.0)
    s = (a * b).sum(-1)
    assert torch.allclose(s, s[0].expand(3), atol=1e-12) and torch.equal(a[:, 4:], x[:, 4:])


def test_plain_router_identity_experts_and_correction():
    torch.manual_seed(3)
    W, E, I = 6, 3, 2
    mlp = {"expert": {"ff": 4}, "router": {"experts": E, "identity": I, "top": 2, "scale": 1.5}}
    t = {"router": torch.randn(E + I, W), "correction": torch.zeros(E + I)}
    for e in range(E):
        t[f"e{e}.up"], t[f"e{e}.down"] = torch.randn(4, W), torch.randn(W, 4)
    h = torch.randn(7, W, dtype=F64)
    s = torch.softmax(h @ t["router"].double().T, dim=-1)
    # a correction that lifts the identity experts above everything: the result is h times their summed weights,
    # and the weights are the scores without the correction
    t["correction"] = torch.tensor([0.0, 0.0, 0.0, 5.0, 6.0])
    got = pz.routed_experts(h, t, "", mlp)
    assert torch.allclose(got, h * (1.5 * (s[:, 3] + s[:, 4]))[:, None], atol=1e-12)
    # ... and one that lifts the first two real experts
    t["correction"] = torch.tensor([9.0, 7.0, 0.0, 0.0, 0.0])
    got = pz.routed_experts(h, t, "", mlp)
    want = sum((1.5 * s[:, e])[:, None] * (pz.gelu_erf(h @ t[f"e{e}.up"].double().T) @ t[f"e{e}.down"].double().T) for e in (0, 1))
    assert torch.allclose(got, want, atol=1e-12)
    assert abs(float(pz.gelu_erf(torch.tensor(1.0, dtype=F64))) - 0.8413447460685429) < 1e-12
    assert abs(float(pz.gelu_tanh(torch.tensor(1.0, dtype=F64))) - 0.8411919906082768) < 1e-12


# ---- the engine on the stand-ins against the plain implementation ---------------------------------------------------

@pytest.mark.parametrize("name", list(ZM.CONFIGS))
def test_schedules_on_the_stand_in(name):
    cfg, w, w64 = model(name)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 58, 23, 70])}
    eng = engine_for(cfg, w)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=12), H.portions_trace(reqs, seed=3)):
        got = ZM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        worst = ZM.worst_error(name, cfg, w64, reqs, got)
        assert worst[0] <= TOL32, worst
        assert eng.cache.n_live == 0
        eng.cache.check()
    # several requests at a time with pages for the live ones only: pages and state slots are used again
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, max_requests=3, max_tokens=peak, graphs=True)
    got = ZM.run_trace(eng, steps)
    worst = ZM.worst_error(name, cfg, w64, reqs, got)
    assert worst[0] <= TOL32, worst
    eng.cache.check()


def test_a_used_state_slot_starts_from_zero():
    cfg, w, w64 = model("D")
    eng = engine_for(cfg, w, max_requests=1)
    ids_a, ids_b = H.random_ids(cfg["vocab"], 30, 1), H.random_ids(cfg["vocab"], 9, 2)
    ZM.run_trace(eng, H.whole_trace({"a": ids_a}))
    assert eng.cache.groups == {}                       # lightning alone keeps no pages
    for key, t in eng.cache.states.items():
        assert t[0].abs().max() > 0                     # the first request left its state in the only slot
    got = ZM.run_trace(eng, H.portions_trace({"b": ids_b}, sizes=(2, 3)))
    assert ZM.worst_error("D", cfg, w64, {"b": ids_b}, got)[0] <= TOL32


def needle_case(name, distance, at, length=None, seed=60):
    """A sequence in which the probe token, `distance` after the needle at `at`, looks for it in the first layer; and
    how far the probe's logits move when the needle is replaced by another token."""
    cfg, w, _ = model(name)
    if cfg["layers"][0]["type"] == "lightning":        # a state that still holds what it saw hundreds of tokens ago
        cfg = copy.deepcopy(cfg)
        cfg["layers"][0]["mixer"]["decay"][0] = 0.9995
    needle, probe = 3, 7
    w = ZM.sharpen(cfg, w, needle, probe)
    w64 = ZM.as_f64(w)
    n = length or at + distance + 4
    ids = [t if t not in (needle, probe) else 11 for t in H.random_ids(cfg["vocab"], n, seed + at)]
    ids[at], ids[at + distance] = needle, probe
    without = list(ids)
    without[at] = 11
    want = ZM.plain_logits((name, "sharp"), cfg, w64, ids)[at + distance]
    moved = ZM.relative_error(pz.forward(cfg, w64, without)[at + distance], want)
    return cfg, w, w64, ids, moved


@pytest.mark.parametrize("name,distance", [("A", 1), ("A", 300), ("E", 200), ("D", 150), ("F", 1), ("F", 250)])
def test_a_token_that_stands_out(name, distance):
    """The probe looks for a needle right before it or hundreds of tokens back (through attention's pages or a
    recurrent state), with the needle on both sides of a page's border; whole, decoded alone and in portions."""
    for at in (15, 16):
        cfg, w, w64, ids, moved = needle_case(name, distance, at)
        assert moved >= 0.01, moved              # losing that one key would show
        eng = engine_for(cfg, w)
        for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=6),
                      H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
            got = ZM.run_trace(eng, steps)
            worst = ZM.worst_error((name, "sharp"), cfg, w64, {"s": ids}, got)
            assert worst[0] <= TOL32, (worst, at)


def test_the_sink_and_the_query_factor_show_in_the_logits():
    """Dropping the sink, or moving the query factor's step by one position, moves the plain logits by far more than
    the engine's tolerance: the schedules above would catch either."""
    cfg, w, w64 = model("A")
    ids = H.random_ids(cfg["vocab"], 40, 9)
    want = ZM.plain_logits("A", cfg, w64, ids)
    other = copy.deepcopy(cfg)
    other["layers"][0]["mixer"]["q_temp"]["every"] = 17          # the step from position 15 to 16 comes one later
    assert ZM.relative_error(pz.forward(other, w64, ids)[15], want[15]) > 100 * TOL32
    assert ZM.relative_error(pz.forward(other, w64, ids)[14], want[14]) < 1e-12
    keep = pz.sink_softmax
    try:
        pz.sink_softmax = pz.plain_softmax
        assert ZM.relative_error(pz.forward(cfg, w64, ids)[0], want[0]) > 100 * TOL32       # the very first token too
    finally:
        pz.sink_softmax = keep


def test_greedy_generation_through_the_scheduler():
    for name in ("A", "B"):
        cfg, w, w64 = model(name, seed=8)
        prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6))]
        want = [pz.greedy_generate(cfg, w64, p, 7) for p in prompts]
        eng = engine_for(cfg, w, max_requests=2, max_tokens=160, graphs=True)
        out, s = generate(eng, prompts, max_new_tokens=7, temperature=0.0, max_batch=2, token_budget=11,
                          return_scheduler=True)
        assert out == want
        assert s.peak_running == 2 and eng.cache.n_live == 0
        eng.cache.check()


def test_the_named_size_runs_with_random_weights(tmp_path):
    from tiny_inference_server_amd.__main__ import preset_names, size_config
    from tiny_inference_server_amd.weights import write_random_model
    assert "fipuzen-small" in preset_names()
    cfg = size_config("fipuzen-small")
    folder = write_random_model(cfg, 3, str(tmp_path / "m"))
    assert load_config(folder).to_dict() == cfg.to_dict()
    eng = Engine(folder, dtype="float32", max_tokens=64, max_requests=2, ops=TorchOps())
    out = eng.step([("a", [5, 9, 1, 300], [3]), ("b", [7], [0])]).logits
    assert out.shape == (2, cfg.vocab) and torch.isfinite(out).all()
