"""The Fikevik architecture on the host: its configuration and spec, the plain implementation's mechanisms against
closed forms, and the engine (step function, cache manager, scheduler, generate) on the torch stand-ins for the
kernels against the plain implementation, in 32-bit."""
import copy
import math

import pytest
import torch

import fikevik_models as FM
import helpers as H
import plain_fikevik as pf
from torch_ops import TorchOps
from tiny_inference_server_amd.config import ARCHITECTURES, ConfigError, config_from_dict, load_config
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.weights.loader import spec_tensors

TOL32 = 3e-5


def model(name, seed=5):
    cfg = FM.CONFIGS[name]
    w = FM.random_weights(cfg, FM.RANK[name], seed)
    return cfg, w, FM.as_f64(w)


def engine_for(cfg, w, **kw):
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 8)
    kw.setdefault("max_tokens", 640)
    return Engine(config=config_from_dict(cfg), tensors={n: t.float() for n, t in w.items()}, dtype="float32",
                  ops=TorchOps(graphs=kw.pop("graphs", False)), **kw)


# ---- configuration and spec ------------------------------------------------------------------------------------

def test_spec_names_every_tensor_and_reads_the_rank_from_a_shape(tmp_path):
    for name, cfg in FM.CONFIGS.items():
        w = FM.random_weights(cfg, FM.RANK[name], 1)
        folder = FM.write_folder(str(tmp_path / name), cfg, w)
        c = load_config(folder)
        spec = ARCHITECTURES.get(c.architecture).build_spec(c)
        assert spec_tensors(spec) == {n: tuple(t.shape) for n, t in w.items()}
        gla_ranks = {e["mixer"]["rank"] for e in c.layers if e["type"] == "gla"}
        assert gla_ranks <= {FM.RANK[name]}
        assert len(spec.stages[0].calls) == len(cfg["layers"])
        assert len(spec.layers) == sum("weights_of" not in e for e in cfg["layers"])
        # a layer that runs with another's tensors is a second call of that block with a cache of its own
        owners = [c.owner_of(i) for i in range(len(c.layers))]
        assert [spec.stages[0].calls[i].layer for i in range(len(owners))] == [sorted(set(owners)).index(o) for o in owners]


def test_configuration_errors_name_the_key():
    good = FM.CONFIGS["A"]
    for path, value, word in [(("layers", 0, "type"), "conv", "type"), (("layers", 1, "mixer", "tau"), -1.0, "tau"),
                              (("layers", 0, "mixer", "left", "rot", "dims"), 7, "rot.dims"),
                              (("layers", 0, "mlp", "kind"), "moe", "mlp"), (("layers", 2, "weights_of"), 9, "weights_of"),
                              (("layers", 2, "weights_of"), 1, "takes the weights")]:
        bad = copy.deepcopy(good)
        d = bad
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            config_from_dict(bad)
    bad = copy.deepcopy(good)
    del bad["postln_alpha"]
    with pytest.raises(ConfigError, match="postln_alpha"):
        config_from_dict(bad)
    with pytest.raises(ConfigError, match="rank"):      # no shapes, no rank: the spec cannot be built
        c = config_from_dict(good)
        ARCHITECTURES.get("Fikevik").build_spec(c)


# ---- the plain implementation's mechanisms against closed forms ----------------------------------------------------

def test_plain_gated_linear_attention_is_the_decayed_sum():
    torch.manual_seed(0)
    T, W, Hh, D, V, tau, r = 9, 12, 2, 4, 3, 2.5, 3
    p = {"heads": Hh, "dim": D, "vdim": V, "tau": tau}
    w = {"q": torch.randn(Hh * D, W), "k": torch.randn(Hh * D, W), "v": torch.randn(Hh * V, W), "g": torch.randn(Hh * V, W),
         "o": torch.eye(Hh * V), "norm": torch.ones(V), "a1": torch.randn(r, W), "a2": torch.randn(Hh * D, r),
         "a2.b": torch.randn(Hh * D)}
    w = {k: v.double() for k, v in w.items()}
    h = torch.randn(T, W).double()
    got = pf.gated_linear_attention(h, w, "", p, 1e-6)
    q = (h @ w["q"].T).view(T, Hh, D) / math.sqrt(D)
    k, v = (h @ w["k"].T).view(T, Hh, D), (h @ w["v"].T).view(T, Hh, V)
    a = torch.sigmoid((h @ w["a1"].T) @ w["a2"].T + w["a2.b"]).pow(1 / tau).view(T, Hh, D)
    o = torch.zeros(T, Hh, V, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            carry = torch.prod(a[s + 1:t + 1], dim=0)                 # what is left of token s's keys at t
            o[t] += ((q[t] * carry * k[s]).sum(-1))[:, None] * v[s]
    g = h @ w["g"].T
    want = (pf.rms_norm(o, 1e-6).reshape(T, -1) * g * torch.sigmoid(g))
    assert torch.allclose(got, want, atol=1e-10)


def test_plain_matrix_memory_is_the_unstabilised_recurrence():
    torch.manual_seed(1)
    T, W, Hh, D, V, cap = 12, 10, 2, 3, 4, 6.0
    p = {"heads": Hh, "dim": D, "vdim": V, "gate_cap": cap}
    w = {n: torch.randn(s).double() for n, s in {"q": (Hh * D, W), "k": (Hh * D, W), "v": (Hh * V, W), "g": (Hh * V, W),
                                                 "i": (Hh, W), "f": (Hh, W), "i.b": (Hh,), "f.b": (Hh,)}.items()}
    w["o"], w["norm"] = torch.eye(Hh * V).double(), torch.ones(Hh * V).double()
    h = torch.randn(T, W).double()
    got = pf.matrix_memory(h, w, "", p, 1e-6)
    q = (h @ w["q"].T).view(T, Hh, D) / math.sqrt(D)
    k, v = (h @ w["k"].T).view(T, Hh, D), (h @ w["v"].T).view(T, Hh, V)
    gi = torch.exp(cap * torch.tanh((h @ w["i"].T + w["i.b"]) / cap))
    gf = torch.sigmoid(cap * torch.tanh((h @ w["f"].T + w["f.b"]) / cap))
    C, n = torch.zeros(Hh, D, V).double(), torch.zeros(Hh, D).double()
    logm = torch.zeros(Hh).double()
    o = torch.zeros(T, Hh, V).double()
    for t in range(T):
        C = gf[t][:, None, None] * C + gi[t][:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = gf[t][:, None] * n + gi[t][:, None] * k[t]
        logm = torch.maximum(torch.log(gf[t]) + logm, torch.log(gi[t]))
        # the stabilised form divides numerator and denominator by exp(m); its floor exp(-m) is 1 here
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.ones(Hh).double()) + 1e-6 * torch.exp(logm)
        o[t] = torch.einsum("hdv,hd->hv", C, q[t]) / den[:, None]
    want = pf.rms_norm(o, 1e-6).reshape(T, -1) * torch.sigmoid(h @ w["g"].T)
    assert torch.allclose(got, want, atol=1e-9)


def test_plain_window_and_rotation():
    torch.manual_seed(2)
    T, W = 14, 16
    p = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "mask": {"size": 4}, "rot": {"dims": 4, "base": 50.0}, "scale": 0.7}
    w = {n: torch.randn(s).double() for n, s in {"q": (24, W), "k": (12, W), "v": (10, W), "o": (W, 20)}.items()}
    w.update({"q.norm": torch.rand(6).double() + 0.5, "k.norm": torch.rand(6).double() + 0.5, "temp": torch.rand(4).double() + 0.5})
    h = torch.randn(T, W).double()
    base = pf.windowed_attention(h, w, "", p, 1e-5)
    h2 = h.clone()
    h2[5] += 1.0
    moved = pf.windowed_attention(h2, w, "", p, 1e-5)
    changed = [(moved[t] - base[t]).abs().max().item() > 1e-9 for t in range(T)]
    assert changed == [5 <= t <= 8 for t in range(T)]          # position 9 is the first that no longer sees 5
    # rotation: a pair's scalar product depends on the distance alone
    x = torch.randn(1, 1, 6).double().expand(3, 1, 6)
    y = torch.randn(1, 1, 6).double().expand(3, 1, 6)
    a = pf.rotate_pairs(x, torch.tensor([3, 10, 40]), 4, 50.0)
    b = pf.rotate_pairs(y, torch.tensor([1, 8, 38]), 4, 50.0)
    s = (a * b).sum(-1).flatten()
    assert torch.allclose(s, s[0].expand(3), atol=1e-12)
    assert torch.equal(a[..., 4:], x[..., 4:])                 # the channels beyond the rotated ones pass unchanged


# ---- the engine on the stand-ins against the plain implementation ---------------------------------------------------

@pytest.mark.parametrize("name", list(FM.CONFIGS))
def test_schedules_on_the_stand_in(name):
    cfg, w, w64 = model(name)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 58, 23, 70])}
    eng = engine_for(cfg, w)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=12), H.portions_trace(reqs, seed=3)):
        got = FM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        worst = FM.worst_error(name, cfg, w64, reqs, got)
        assert worst[0] <= TOL32, worst
        assert eng.cache.n_live == 0
        eng.cache.check()
    # several requests at a time with pages for the live ones only: pages and state slots are used again
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, max_requests=3, max_tokens=peak, graphs=True)
    got = FM.run_trace(eng, steps)
    worst = FM.worst_error(name, cfg, w64, reqs, got)
    assert worst[0] <= TOL32, worst
    eng.cache.check()


def test_a_used_state_slot_starts_from_zero():
    cfg, w, w64 = model("C")
    eng = engine_for(cfg, w, max_requests=1)
    ids_a, ids_b = H.random_ids(cfg["vocab"], 30, 1), H.random_ids(cfg["vocab"], 9, 2)
    FM.run_trace(eng, H.whole_trace({"a": ids_a}))
    for key, t in eng.cache.states.items():
        assert t[0].abs().max() > 0            # the first request left its state in the only slot
    got = FM.run_trace(eng, H.portions_trace({"b": ids_b}, sizes=(2, 3)))
    assert FM.worst_error("C", cfg, w64, {"b": ids_b}, got)[0] <= TOL32


@pytest.mark.parametrize("name,distance", [("A", 23), ("A", 24), ("B", 39), ("B", 40), ("C", 150)])
def test_a_token_that_stands_out(name, distance):
    """The probe token looks for the needle `distance` positions back: just inside and just outside the first layer's
    window (24 and 40), or far back in a recurrent state; in a prompt's portion and decoded alone, with the needle
    on both sides of a page's border."""
    cfg, w, _ = model(name)
    needle, probe = 3, 7
    w = FM.sharpen(cfg, w, needle, probe)
    w64 = FM.as_f64(w)
    for at in (15, 16):                                         # last slot of a page of 8, first slot of the next
        ids = [t if t not in (needle, probe) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, 60 + at)]
        ids[at], ids[at + distance] = needle, probe
        assert FM.sharpness(name, cfg, w64, ids, at, distance) >= 0.005
        eng = engine_for(cfg, w)
        for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=6),
                      H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
            got = FM.run_trace(eng, steps)
            worst = FM.worst_error((name, "sharp"), cfg, w64, {"s": ids}, got)
            assert worst[0] <= TOL32, (worst, at)


def test_greedy_generation_through_the_scheduler():
    for name in ("A", "C"):
        cfg, w, w64 = model(name, seed=8)
        prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6))]
        want = [pf.greedy_generate(p, 7, w64, cfg) for p in prompts]
        eng = engine_for(cfg, w, max_requests=2, max_tokens=160, graphs=True)
        out, s = generate(eng, prompts, max_new_tokens=7, temperature=0.0, max_batch=2, token_budget=11,
                          return_scheduler=True)
        assert out == want
        assert s.peak_running == 2 and eng.cache.n_live == 0
        eng.cache.check()


def test_the_named_size_runs_with_random_weights(tmp_path):
    """`--random fikevik-small`: the preset's configuration, random tensors for its spec, a model folder that loads
    again (with the decay's rank read back from the file's header), and a few tokens through the engine."""
    from tiny_inference_server_amd.__main__ import preset_names, size_config
    from tiny_inference_server_amd.weights import write_random_model
    assert "fikevik-small" in preset_names()
    cfg = size_config("fikevik-small")
    folder = write_random_model(cfg, 3, str(tmp_path / "m"))
    again = load_config(folder)
    assert again.to_dict() == cfg.to_dict()
    eng = Engine(folder, dtype="float32", max_tokens=64, max_requests=2, ops=TorchOps())
    out = eng.step([("a", [5, 9, 1, 300], [3]), ("b", [7], [0])]).logits
    assert out.shape == (2, 4096) and torch.isfinite(out).all()
