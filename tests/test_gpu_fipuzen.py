"""The Fipuzen architecture on the GPU: each new kernel against plain torch, and the engine with its HIP kernels
against the plain implementation through every kind of schedule, in 32-bit and in bfloat16."""
import json
import os
import statistics
import subprocess
import sys

import numpy as np
import pytest
import torch

import fipuzen_models as ZM
import helpers as H
import plain_fipuzen as pz
from test_gpu_fikevik import fake_batch
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 3e-5, "bfloat16": 4e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def hip_ops(dtype):
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    return HipOps("cuda:0", DT[dtype])


def model(name, dtype="float32", seed=5):
    """In bfloat16 every expert is chosen (see fipuzen_models.all_chosen); routing itself is tested in 32-bit, kernel by
    kernel in both types, and by test_routing_in_bfloat16."""
    cfg = ZM.CONFIGS[name] if dtype == "float32" else ZM.all_chosen(ZM.CONFIGS[name])
    w = ZM.random_weights(cfg, seed)
    return cfg, w, ZM.as_f64(w)


def engine_for(cfg, w, dtype, **kw):
    from tiny_inference_server_amd.config import config_from_dict
    from tiny_inference_server_amd.engine import Engine
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_tokens", 1024)
    eng = Engine(config=config_from_dict(cfg), tensors=w, dtype=dtype, **kw)
    H.fill_cache_with_nan(eng)       # what a row may not see must not reach a result
    return eng


def close(a, b, dtype, what, tol=None):
    tol = tol or (2e-5 if dtype == "float32" else 1.6e-2)
    err = (a.float().cpu() - b.float().cpu()).abs().max().item()
    assert err <= tol * max(1.0, b.float().abs().max().item()), (what, err)


# ---- kernels ---------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("D", [44, 300, 1500, 4200])      # (a row in 4 or 16 registers a thread, or in memory)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sums_and_norms_of_the_stream(dtype, D):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(D)
    n = 23
    x = torch.randn(n, D, generator=g) * 3 + 0.7
    wide = torch.randn(n, D + 9, generator=g)
    gain, bias, ygain = (1 + 0.2 * torch.randn(D, generator=g) for _ in range(3))
    close(ops.layernorm32(x.cuda(), gain.cuda(), bias.cuda(), 1e-5), ref.layernorm32(x, gain, bias, 1e-5), dtype, "layernorm32")
    close(ops.layernorm32(x.cuda(), gain.cuda(), None, 1e-5), ref.layernorm32(x, gain, None, 1e-5), dtype, "layernorm32 no bias")
    for y_rms, copy, norm in ((None, False, ("layer", gain, bias, 1e-5)), ((ygain, 1e-6), True, None), (None, True, ("rms", gain, None, 1e-6)),
                              ((ygain, 1e-6), False, ("layer", gain, None, 1e-5))):
        dev = lambda t: None if t is None else t.cuda()
        got = ops.residual_norm(x.cuda(), wide.cuda()[:, 9:], y_rms=(dev(y_rms[0]), y_rms[1]) if y_rms else None, copy=copy,
                                norm=(norm[0], dev(norm[1]), dev(norm[2]), norm[3]) if norm else None)
        want = ref.residual_norm(x.clone(), wide[:, 9:], y_rms=y_rms, copy=copy, norm=norm)
        close(got[0], want[0], "float32", "sum")
        for a, b, what in ((got[1], want[1], "copy"), (got[2], want[2], "norm")):
            assert (a is None) == (b is None)
            if a is not None:
                close(a, b, dtype, what)
    got = ops.residual_norm(x.cuda(), None, copy=True)                 # nothing to add: the copy alone
    close(got[1], x.to(DT[dtype]), dtype, "copy alone")
    table = torch.randn(31, 20, generator=g).to(DT[dtype])
    tokens = torch.randint(0, 31, (n,), generator=g, dtype=torch.int32)
    for act in ("gelu_tanh", "silu", "sigmoid"):
        close(ops.gate_table(wide.cuda()[:, 3:23], table.cuda(), tokens.cuda(), act), ref.gate_table(wide[:, 3:23], table, tokens, act),
              dtype, "gate_table " + act)
        z = wide.clone().cuda()
        ops.activate32(z[:, 2:D], act)
        zr = wide.clone()
        ref.activate32(zr[:, 2:D], act)
        close(z, zr, "float32", "activate32 " + act)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,G,kd,vd,coef,every", [(6, 2, 24, 40, 0.4, 5), (4, 4, 64, 64, 0.0, 1), (2, 1, 10, 300, 0.3, 16),
                                                   (3, 1, 320, 16, 0.2, 2)])
def test_attention_with_bias_sink_query_factor_and_head_gate(dtype, Hq, G, kd, vd, coef, every):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(kd)
    ps, n_pages = 8, 12
    tables = [[5, 2, 9, 0, 0, 0], [7, 1, 3, 11, 4, 0]]
    cols = Hq * kd + G * kd + G * vd + Hq + 3
    biases = [0.3 * torch.randn(s, generator=g) for s in (Hq * kd, G * kd, G * vd)]
    planes = [torch.full((n_pages, G * ps * (kd + vd)), float("nan"), dtype=DT[dtype]) for _ in range(2)]
    planes[0] = planes[0].cuda()
    for seq_rows in ([(0, 0, 19)], [(0, 0, 21), (21, 19, 17)]):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        slots = [0] if len(seq_rows) == 1 else [1, 0]
        tabs = [tables[1]] if len(seq_rows) == 1 else [tables[0], tables[1]]
        for sink, gated in ((True, True), (False, True), (True, False)):
            res = []
            for o, plane, dev in ((ops, planes[0], "cuda"), (ref, planes[1], "cpu")):
                b = fake_batch(seq_rows, slots, tabs, ps, dev)
                mv = lambda t: t.to(dev)
                p = mv(proj)[:, 3:]
                q = o.attention_prepare(p, 0, Hq * kd, Hq * kd + G * kd, b.positions, b.write_slots["g"], plane, Hq, G, kd, vd, ps,
                                        value_norm=False, q_bias=mv(biases[0]), k_bias=mv(biases[1]), v_bias=mv(biases[2]),
                                        temp_coef=coef, temp_every=every)
                gate = p[:, Hq * kd + G * kd + G * vd:] if gated else None
                res.append((q, o.paged_attention_kv(q, plane, b, "g", Hq, G, kd, vd, ps, 0, 0.37 / kd ** 0.5, sink=sink, gate=gate)))
            close(res[0][0], res[1][0], dtype, "queries")
            close(res[0][1], res[1][1], dtype, "attention")
            assert torch.isfinite(res[0][1].float()).all()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,D,R,V,C,dims", [(3, 16, 8, 12, 24, 8), (2, 5, 6, 7, 300, 4), (8, 64, 32, 64, 128, 32), (1, 12, 0, 9, 40, 0),
                                             (20, 24, 16, 8, 48, 16), (16, 128, 64, 128, 512, 64), (70, 8, 8, 16, 32, 8)])
def test_attention_over_a_latent(dtype, Hq, D, R, V, C, dims):
    """The step before (norm of the latent, rotation, the pages), the product per head into the latent's space, the
    attention whose values are part of its keys, and the product per head back out. Pages of 16 slots with key sizes
    in steps of 8 and value sizes in steps of 16 take the matrix-core kernel in bfloat16 (fewer heads than 16, exactly
    16 and more), the others the kernel for any sizes."""
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(C)
    ps, n_pages = (16, 12) if C % 16 == 0 else (8, 12)
    tables = [[5, 2, 9, 0, 0, 0], [7, 1, 3, 11, 4, 0]]
    cols = Hq * (D + R) + C + R + 5
    gain = 1 + 0.2 * torch.randn(C, generator=g)
    freqs = (50.0 ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1))).float()
    w_in = (torch.randn(Hq, C, D, generator=g) / D ** 0.5).to(DT[dtype])
    w_out = (torch.randn(Hq, V, C, generator=g) / C ** 0.5).to(DT[dtype])
    planes = [torch.full((n_pages, ps * (2 * C + R)), float("nan"), dtype=DT[dtype]) for _ in range(2)]
    planes[0] = planes[0].cuda()
    for seq_rows in ([(0, 0, 19)], [(0, 0, 21), (21, 19, 17)]):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        slots = [0] if len(seq_rows) == 1 else [1, 0]
        tabs = [tables[1]] if len(seq_rows) == 1 else [tables[0], tables[1]]
        res = []
        for o, plane, dev in ((ops, planes[0], "cuda"), (ref, planes[1], "cpu")):
            b = fake_batch(seq_rows, slots, tabs, ps, dev)
            mv = lambda t: t.to(dev)
            q, q_plain = o.latent_prepare(mv(proj)[:, 5:], 0, Hq * (D + R), b.positions, b.write_slots["g"], plane, Hq, D, R, C, ps,
                                          mv(gain), mv(freqs), dims, 1e-5)
            o.heads_linear(q_plain, mv(w_in), q, C + R)
            mixed = o.latent_attention(q, plane, b, "g", Hq, C + R, C, ps, 0.3 / C ** 0.5)
            out = torch.zeros(n, Hq * V + 2, dtype=DT[dtype], device=dev)
            o.heads_linear(mixed, mv(w_out), out, V, 2)
            res.append((q, mixed, out))
        for a, b_, what in zip(res[0], res[1], ("queries", "attention", "values")):
            close(a, b_, dtype, what)
        assert res[0][2][:, :2].abs().max() == 0                  # columns outside the heads' stay as they were


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,W,F,E,I,top", [(37, 64, 40, 6, 2, 2), (5, 44, 20, 3, 3, 6), (200, 128, 72, 16, 1, 3), (9, 48, 30, 2, 0, 1), (600, 64, 48, 4, 1, 2), (700, 128, 72, 4, 0, 2),
                                           (4, 32, 8, 0, 3, 2)])
def test_router_and_experts(dtype, n, W, F, E, I, top):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(n)
    z = 2 * torch.randn(n, E + I + 3, generator=g)
    corr = 0.1 * torch.randn(E + I, generator=g)
    ids, wts = ops.route_topk(z.cuda()[:, 3:], corr.cuda(), 1.7, top)
    ids_r, wts_r = ref.route_topk(z[:, 3:], corr, 1.7, top)
    assert torch.equal(ids.cpu().sort(dim=1).values, ids_r.sort(dim=1).values)
    order = ids.cpu().long().argsort(dim=1), ids_r.long().argsort(dim=1)
    close(torch.gather(wts.cpu(), 1, order[0]), torch.gather(wts_r, 1, order[1]), "float32", "weights")
    x = torch.randn(n, W, generator=g).to(DT[dtype])
    up = (torch.randn(E, F, W, generator=g) / W ** 0.5).to(DT[dtype]) if E else None
    down = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(DT[dtype]) if E else None
    got = ops.routed_experts(x.cuda(), ids, wts, up.cuda() if E else None, down.cuda() if E else None)
    want = ref.routed_experts(x, ids.cpu(), wts.cpu(), up, down)
    close(got, want, dtype, "experts")
    # the same sum taken inside the residual sum's kernel, with the norm that follows
    x32, gain = torch.randn(n, W, generator=g), 1 + 0.1 * torch.randn(W, generator=g)
    a = ops.residual_norm(x32.cuda(), ops.routed_experts(x.cuda(), ids, wts, up.cuda() if E else None, down.cuda() if E else None,
                                                         combine=False), copy=True, norm=("layer", gain.cuda(), None, 1e-5))
    b = ref.residual_norm(x32.clone(), ref.routed_experts(x, ids.cpu(), wts.cpu(), up, down, combine=False), copy=True,
                          norm=("layer", gain, None, 1e-5))
    for u, v, what in zip(a, b, ("sum with experts", "its copy", "its norm")):
        close(u, v, dtype, what)
    close(a[0], x32 + want.float(), dtype, "sum with experts against the separate sum")
    # a tie goes to the lower index
    tie = torch.zeros(2, 5).cuda()
    ids, _ = ops.route_topk(tie, None, 1.0, 2)
    assert ids.cpu().tolist() == [[0, 1], [0, 1]]


# ---- the engine ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(ZM.CONFIGS))
def test_schedules(name, dtype):
    cfg, w, w64 = model(name, dtype)
    key = (name, dtype)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 158, 23, 70])}
    eng = engine_for(cfg, w, dtype)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=20), H.portions_trace(reqs, seed=3)):
        got = ZM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        ZM.check(key, cfg, w64, reqs, got, dtype)
        eng.cache.check()
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, dtype, max_requests=3, max_tokens=peak)
    got = ZM.run_trace(eng, steps)
    ZM.check(key, cfg, w64, reqs, got, dtype)
    eng.cache.check()


def test_routing_in_bfloat16():
    """With experts chosen by comparing scores, a bfloat16 engine may turn a close comparison the other way and differ
    there by more than rounding; most rows are not close."""
    cfg, w, w64 = model("C", "float32")
    reqs = {"a": H.random_ids(cfg["vocab"], 150, 3), "b": H.random_ids(cfg["vocab"], 60, 4)}
    eng = engine_for(cfg, w, "bfloat16")
    got = ZM.run_trace(eng, H.portions_trace(reqs, seed=5))
    errs = []
    for rid, ids in reqs.items():
        want = ZM.plain_logits("C", cfg, w64, ids)
        errs += [ZM.relative_error(got[(rid, p)], want[p]) * float(want[p].std() / want.std()) for p in range(len(ids))]
    assert statistics.median(errs) <= TOL["bfloat16"] / 2, statistics.median(errs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,distance", [("A", 1), ("A", 300), ("E", 200), ("D", 150), ("F", 1), ("F", 250)])
def test_a_token_that_stands_out(name, distance, dtype):
    """A probe token that looks for a needle right before it or hundreds of tokens back, through attention's pages or a
    recurrent state, with the needle on both sides of a page's border: whole, decoded alone, in portions."""
    for at in (15, 16):
        cfg, w, _ = model(name, dtype)
        if cfg["layers"][0]["type"] == "lightning":
            cfg["layers"][0]["mixer"]["decay"][0] = 0.9995
        w = ZM.sharpen(cfg, w, 3, 7)
        w64 = ZM.as_f64(w)
        ids = [t if t not in (3, 7) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, 60 + at)]
        ids[at], ids[at + distance] = 3, 7
        key = (name, dtype, "sharp")
        want = ZM.plain_logits(key, cfg, w64, ids)
        without = list(ids)
        without[at] = 11
        moved = ZM.relative_error(pz.forward(cfg, w64, without)[at + distance], want[at + distance])
        eng = engine_for(cfg, w, dtype)
        for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=6),
                      H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
            got = ZM.run_trace(eng, steps)
            err = ZM.relative_error(got[("s", at + distance)], want[at + distance])
            assert err <= min(TOL[dtype], moved / 3), (err, moved, at)
            ZM.check(key, cfg, w64, {"s": ids}, got, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_and_wide_heads(dtype):
    """Heads of 64 channels, prompts long enough for the scan to run in segments, then decoded tokens; alone and two
    requests together, the second cut into portions."""
    cfg, w, w64 = model("C", dtype, seed=9)
    key = ("C9", dtype)
    reqs = {"a": H.random_ids(cfg["vocab"], 330, 1), "b": H.random_ids(cfg["vocab"], 215, 2)}
    eng = engine_for(cfg, w, dtype)
    got = ZM.run_trace(eng, H.tail_decode_trace(reqs, tail=12))
    ZM.check(key, cfg, w64, reqs, got, dtype)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:300], "want": list(range(0, 300, 7))},
                                     {"id": "b", "tokens": reqs["b"][:3], "want": [0, 1, 2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][300:301], "want": [0]},
                                     {"id": "b", "tokens": reqs["b"][3:200], "want": list(range(0, 197, 5))}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": reqs["a"][301:], "want": list(range(29))},
                                     {"id": "b", "tokens": reqs["b"][200:], "want": list(range(15))}], "end": ["a", "b"]}]
    got = ZM.run_trace(eng, steps)
    ZM.check(key, cfg, w64, reqs, got, dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_captured_steps(dtype):
    """Three requests decode 150 tokens together, over many page borders and past several steps of the query factor;
    steps of single tokens are replayed from captured graphs, and every replay is checked."""
    for name in ("A", "B"):
        cfg, w, w64 = model(name, dtype, seed=6)
        reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 90 + i) for i, n in enumerate([160, 171, 153])}
        eng = engine_for(cfg, w, dtype, max_requests=3)
        steps = [{"step": 0, "entries": [{"id": r, "tokens": ids[:len(ids) - 150], "want": [0]} for r, ids in reqs.items()],
                  "end": []}]
        for t in range(150):
            steps.append({"step": t + 1, "entries": [{"id": r, "tokens": [ids[len(ids) - 150 + t]], "want": [0]}
                                                     for r, ids in reqs.items()], "end": list(reqs) if t == 149 else []})
        got = ZM.run_trace(eng, steps)
        assert eng.graph_replays >= 100
        ZM.check((name, dtype, 6), cfg, w64, reqs, got, dtype)


def test_generation_command_line_and_replay_program(tmp_path):
    from tiny_inference_server_amd.engine.generate import generate
    cfg, w, w64 = model("A", seed=8)
    folder = ZM.write_folder(str(tmp_path / "m"), cfg, w)
    prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6, 21))]
    want = [pz.greedy_generate(cfg, w64, p, 9) for p in prompts]
    out, s = generate(folder, prompts, max_new_tokens=9, temperature=0.0, dtype="float32", max_batch=3, token_budget=12,
                      pool_tokens=192, return_scheduler=True)
    assert out == want and s.peak_running == 3
    out = generate(folder, prompts[:2], max_new_tokens=5, temperature=0.8, top_k=20, top_p=0.9, rep_penalty=1.1, seed=3)
    assert all(len(o) == 5 and all(0 <= t < cfg["vocab"] for t in o) for o in out)
    proc = subprocess.run([sys.executable, "-m", "tiny_inference_server_amd", "--model", folder, "--prompt-ids",
                           ",".join(map(str, prompts[0])), "--max-new-tokens", "9", "--greedy", "--dtype", "float32"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    line = [l for l in proc.stdout.splitlines() if l.startswith("OUTPUT:")][0]
    assert [int(t) for t in line.split()[1:]] == want[0]
    # the replay program: mixed steps on four state slots and pages for the live requests only
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 70 + i) for i, n in enumerate([40, 64, 30, 70, 12, 50])}
    steps, peak = H.mixed_trace(reqs, max_live=4, seed=8)
    out_dir = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(out_dir), "--max-tokens", str(peak)],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert proc.stdout.split() == [x for s in steps for x in ("done", str(s["step"]))]
    got, fed = {}, {r: 0 for r in reqs}
    for s in steps:
        arr = np.fromfile(out_dir / f"{s['step']}.f32", dtype="<f4").reshape(-1, cfg["vocab"])
        row = 0
        for e in s["entries"]:
            for i in e["want"]:
                got[(e["id"], fed[e["id"]] + i)] = torch.from_numpy(arr[row].copy())
                row += 1
            fed[e["id"]] += len(e["tokens"])
    assert len(got) == sum(len(v) for v in reqs.values())
    assert ZM.worst_error("A8", cfg, w64, reqs, got)[0] <= TOL["float32"]


@pytest.mark.parametrize("hd,Hq,G", [(64, 8, 2), (128, 4, 1), (32, 6, 6)])
def test_matrix_core_attention_with_a_sink_and_a_gate(hd, Hq, G):
    """Keys and values of one size in bfloat16 go to the matrix-core kernels: a long portion (tiles, cut into key
    splits and merged), decoded tokens deep in their requests (single waves, splits, merge) and short portions, each
    with the sink in the denominator and the gate per head, against plain torch over the same pages."""
    ops, ref = hip_ops("bfloat16"), TorchOps("cpu", torch.bfloat16)
    g = torch.Generator().manual_seed(hd)
    ps, n_pages = 16, 200
    plane = torch.randn(n_pages, 2, G, ps, hd, generator=g).to(torch.bfloat16)
    perm = torch.randperm(n_pages, generator=g).tolist()
    tables = [perm[:64] + [0] * 64, perm[64:192]]
    for seq_rows in ([(0, 0, 700)], [(0, 1000, 1), (1, 1900, 1)], [(0, 990, 9), (9, 40, 1), (10, 0, 3)][:2]):
        n = sum(r[2] for r in seq_rows)
        q = (torch.randn(n, Hq * hd, generator=g) * 1.5).to(torch.bfloat16)
        gate = torch.randn(n, Hq + 2, generator=g)
        tabs = tables[:len(seq_rows)] if len(seq_rows) > 1 else [tables[0]]
        for sink, gated in ((True, True), (True, False), (False, True)):
            got = ops.paged_attention(q.cuda(), plane.cuda(), fake_batch(seq_rows, list(range(len(seq_rows))), tabs, ps, "cuda"), "g",
                                      Hq, G, hd, 0, hd ** -0.5, sink=sink, gate=gate.cuda()[:, 2:] if gated else None)
            want = ref.paged_attention(q, plane, fake_batch(seq_rows, list(range(len(seq_rows))), tabs, ps, "cpu"), "g", Hq, G,
                                       hd, 0, hd ** -0.5, sink=sink, gate=gate[:, 2:] if gated else None)
            close(got, want, "bfloat16", f"attention {seq_rows} sink={sink}")
