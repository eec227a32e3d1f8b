"""The Fikevik architecture on the GPU: each new kernel against plain torch, and the engine with its HIP kernels
against the plain implementation through every kind of schedule, in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import fikevik_models as FM
import helpers as H
import plain_fikevik as pf
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 3e-5, "bfloat16": 4e-2}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def hip_ops(dtype):
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    return HipOps("cuda:0", DT[dtype])


def model(name, seed=5):
    cfg = FM.CONFIGS[name]
    w = FM.random_weights(cfg, FM.RANK[name], seed)
    return cfg, w, FM.as_f64(w)


def engine_for(cfg, w, dtype, **kw):
    from tiny_inference_server_amd.config import config_from_dict
    from tiny_inference_server_amd.engine import Engine
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_tokens", 1024)
    eng = Engine(config=config_from_dict(cfg), tensors=w, dtype=dtype, **kw)
    H.fill_cache_with_nan(eng)       # what a row may not see must not reach a result
    return eng


# ---- kernels ---------------------------------------------------------------------------------------------------

def close(a, b, dtype, what):
    tol = 2e-5 if dtype == "float32" else 1.6e-2
    err = (a.float().cpu() - b.float().cpu()).abs().max().item()
    assert err <= tol * max(1.0, b.float().abs().max().item()), (what, err)


@pytest.mark.parametrize("D", [300, 2500, 4200])      # (the sum-and-norm kernel keeps a row in 4 or 16 registers a thread, or in memory)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rowwise_kernels_of_the_32_bit_stream(dtype, D):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(3)
    n = 37
    table = torch.randn(50, D, generator=g).to(DT[dtype])
    tokens = torch.randint(0, 50, (n,), generator=g, dtype=torch.int32)
    x32, x = ops.embed_scaled(table.cuda(), tokens.cuda(), 2.5)
    r32, r = ref.embed_scaled(table, tokens, 2.5)
    assert torch.equal(x32.cpu(), r32) and torch.equal(x.cpu(), r)
    wide = torch.randn(n, 3 * D + 8, generator=g)
    y0, y1, gate = wide[:, :D], wide[:, D:2 * D], wide[:, 2 * D + 8:]
    bias, gain = torch.randn(D, generator=g), 1 + 0.1 * torch.randn(D, generator=g)
    wd = wide.cuda()
    for branches, gt in (([(0, 1.3), (1, 0.7)], True), ([(1, 1.0)], False)):
        views = [wd[:, :D], wd[:, D:2 * D]]
        got32, got = ops.gated_postnorm(x32, [(views[i].contiguous() if i else views[i], s) for i, s in branches],
                                        wd[:, 2 * D + 8:] if gt else None, bias.cuda() if gt else None, 1.9, gain.cuda(), 1e-5)
        want32, want = ref.gated_postnorm(r32, [((y0, y1)[i], s) for i, s in branches], gate if gt else None,
                                          bias if gt else None, 1.9, gain, 1e-5)
        close(got32, want32, "float32", "gated_postnorm 32-bit")
        close(got, want, dtype, "gated_postnorm")
    close(ops.rmsnorm32(x32, gain.cuda(), 1e-6), ref.rmsnorm32(r32, gain, 1e-6), dtype, "rmsnorm32")
    for Hh, V, act, per_head in ((3, 100, "silu", False), (5, 60, "sigmoid", True), (1, 300, "sigmoid", True)):
        o = torch.randn(n, Hh * V, generator=g)
        gn = 1 + 0.2 * torch.randn(Hh * V if per_head else V, generator=g)
        got = ops.head_norm_gate(o.cuda(), wd[:, 4:4 + Hh * V], gn.cuda(), Hh, V, 1e-5, act)
        close(got, ref.head_norm_gate(o, wide[:, 4:4 + Hh * V], gn, Hh, V, 1e-5, act), dtype, "head_norm_gate")
    w2, b2 = torch.randn(77, 9, generator=g), torch.randn(77, generator=g)
    close(ops.lowrank_decay(wd[:, 5:14], w2.cuda(), b2.cuda(), 7.0), ref.lowrank_decay(wide[:, 5:14], w2, b2, 7.0), "float32",
          "lowrank_decay")


def fake_batch(seq_rows, slots, tables, page_size, device):
    """The few fields of a stage's batch that the attention and scan kernels read."""
    pos = [p0 + i for _, p0, n in seq_rows for i in range(n)]
    row_seq = [k for k, (_, _, n) in enumerate(seq_rows) for _ in range(n)]
    t = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    cu = [0]
    for _, _, n in seq_rows:
        cu.append(cu[-1] + n)
    ws = [tables[k][p // page_size] * page_size + p % page_size for k, p in zip(row_seq, pos)] if tables else []
    return SimpleNamespace(positions=t(pos), row_seq=t(row_seq), cu_rows=t(cu), seq_slots=t(slots), n_seqs=len(seq_rows),
                           host_slots=list(slots), seq_rows=list(seq_rows), max_kv_len=max(p0 + n for _, p0, n in seq_rows),
                           max_seq_rows=max(n for _, _, n in seq_rows), block_tables={"g": t(tables)} if tables else {},
                           write_slots={"g": t(ws)}, extras={})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,G,kd,vd,window,rot", [(6, 2, 24, 40, 7, 10), (4, 4, 64, 16, 0, 64), (2, 1, 10, 200, 33, 0)])
def test_attention_with_keys_and_values_of_different_sizes(dtype, Hq, G, kd, vd, window, rot):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(kd)
    ps, n_pages = 8, 12
    # two requests: one starts at 0, one goes on at 19 (its earlier keys are written by a first call)
    tables = [[5, 2, 9, 0, 0, 0], [7, 1, 3, 11, 4, 0]]
    cols = Hq * kd + G * kd + G * vd + 3
    gains = [1 + 0.2 * torch.randn(kd, generator=g) for _ in range(2)]
    factor = 0.5 + torch.rand(Hq, generator=g)
    freqs = (50.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / max(rot, 1))).float()
    planes = [torch.full((n_pages, G * ps * (kd + vd)), float("nan"), dtype=DT[dtype]) for _ in range(2)]
    planes[0] = planes[0].cuda()
    outs = []
    for seq_rows in ([(0, 0, 19)], [(0, 0, 21), (21, 19, 17)]):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        slots = [0] if len(seq_rows) == 1 else [1, 0]
        tabs = [tables[1]] if len(seq_rows) == 1 else [tables[0], tables[1]]
        res = []
        for o, plane, dev in ((ops, planes[0], "cuda"), (ref, planes[1], "cpu")):
            b = fake_batch(seq_rows, slots, tabs, ps, dev)
            mv = lambda t: t.to(dev)
            q = o.attention_prepare(mv(proj)[:, 3:], 0, Hq * kd, Hq * kd + G * kd, b.positions, b.write_slots["g"], plane,
                                    Hq, G, kd, vd, ps, mv(gains[0]), mv(gains[1]), mv(factor), mv(freqs), rot, 1e-5)
            res.append((q, o.paged_attention_kv(q, plane, b, "g", Hq, G, kd, vd, ps, window, 0.37)))
        close(res[0][0], res[1][0], dtype, "queries")
        close(res[0][1], res[1][1], dtype, "attention")
        assert torch.isfinite(res[0][1].float()).all()


@pytest.mark.parametrize("segment", [64, 8, 5])
@pytest.mark.parametrize("kind,Hh,D,V", [("decay", 3, 20, 24), ("gated_max", 2, 24, 40), ("decay", 1, 130, 17),
                                         ("gated_max", 5, 7, 16), ("gated_max", 1, 256, 70), ("gated_max", 2, 64, 130),
                                         ("decay", 2, 128, 64), ("gated_max", 2, 128, 128), ("decay", 1, 96, 192)])
def test_state_scan_against_the_token_by_token_rule(kind, Hh, D, V, segment):
    """Portions of three requests in one call, then their next portions and single tokens in further calls, on state
    lines that start from what an earlier owner left: every result and the final state against plain torch. With
    segments of 8 and 5 rows the portions of 37, 18 and 40 rows run in segments side by side (beside a request that
    brings one row), the single tokens after them in order."""
    ops, ref = hip_ops("float32"), TorchOps("cpu", torch.float32)
    ops.scan_segment = segment
    g = torch.Generator().manual_seed(D)
    floats = ops.state_scan_floats(kind, Hh, D, V)
    assert floats == ref.state_scan_floats(kind, Hh, D, V)
    state = torch.zeros(5, floats + 3)
    state_gpu = state.cuda()
    cols = 2 * Hh * D + Hh * V + 2 * Hh + 5
    qo, ko, vo, io, fo = 5, 5 + Hh * D, 5 + 2 * Hh * D, 5 + 2 * Hh * D + Hh * V, 5 + 2 * Hh * D + Hh * V + Hh
    bi, bf = torch.randn(Hh, generator=g), 2 + torch.randn(Hh, generator=g)
    for seq_rows, slots in (([(0, 0, 37), (37, 0, 1), (38, 0, 18)], [3, 0, 4]), ([(0, 37, 2), (2, 1, 1), (3, 18, 40)], [3, 0, 4]),
                            ([(0, 39, 1), (1, 2, 1), (2, 58, 1)], [3, 0, 4])):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        decay = torch.rand(n, Hh * D, generator=g) * 0.3 + 0.7
        kw = dict(decay=None, i_off=io, f_off=fo, bias_i=bi, bias_f=bf, cap=9.0) if kind == "gated_max" else dict(decay=decay)
        want = ref.state_scan(kind, proj, qo, ko, vo, D ** -0.5, state, fake_batch(seq_rows, slots, None, 1, "cpu"), Hh, D, V, **kw)
        kw = {k: (v.cuda() if torch.is_tensor(v) else v) for k, v in kw.items()}
        got = ops.state_scan(kind, proj.cuda(), qo, ko, vo, D ** -0.5, state_gpu, fake_batch(seq_rows, slots, None, 1, "cuda"),
                             Hh, D, V, **kw)
        close(got, want, "float32", "scan output")
    close(state_gpu[:, :Hh * D * V], state[:, :Hh * D * V], "float32", "state")
    assert state_gpu[[1, 2]].abs().max() == 0 and state_gpu[:, floats:].abs().max() == 0


# ---- the engine ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(FM.CONFIGS))
def test_schedules(name, dtype):
    cfg, w, w64 = model(name)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 158, 23, 70])}
    eng = engine_for(cfg, w, dtype)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=20), H.portions_trace(reqs, seed=3)):
        got = FM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        worst = FM.worst_error(name, cfg, w64, reqs, got)
        assert worst[0] <= TOL[dtype], worst
        eng.cache.check()
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, dtype, max_requests=3, max_tokens=peak)
    got = FM.run_trace(eng, steps)
    worst = FM.worst_error(name, cfg, w64, reqs, got)
    assert worst[0] <= TOL[dtype], worst
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,distance", [("A", 23), ("A", 24), ("B", 39), ("B", 40), ("C", 150)])
def test_a_token_that_stands_out(name, distance, dtype):
    """A probe token that looks for a needle just inside or just outside the first layer's window, or far back in a
    recurrent state, with the needle on both sides of a page's border: in a whole prompt, decoded alone, in portions."""
    cfg, w, _ = model(name)
    w = FM.sharpen(cfg, w, 3, 7)
    w64 = FM.as_f64(w)
    for at in (15, 16):
        ids = [t if t not in (3, 7) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, 60 + at)]
        ids[at], ids[at + distance] = 3, 7
        sharp = FM.sharpness(name, cfg, w64, ids, at, distance)
        eng = engine_for(cfg, w, dtype)
        for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=6),
                      H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
            got = FM.run_trace(eng, steps)
            want = FM.plain_logits((name, "sharp"), cfg, w64, ids)
            err = FM.relative_error(got[("s", at + distance)], want[at + distance])
            assert err <= min(TOL[dtype], sharp / 4), (err, sharp, at)
            assert FM.worst_error((name, "sharp"), cfg, w64, {"s": ids}, got)[0] <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_heads_of_served_sizes(dtype):
    """Heads of 128 channels (the matrix-core attention kernels in bfloat16, eight state elements a thread in the
    scans), prompts long enough for the scans to run in segments and for the window to pass, then decoded tokens;
    alone and two requests together, the second cut into portions."""
    cfg, w, w64 = model("E", seed=9)
    reqs = {"a": H.random_ids(cfg["vocab"], 330, 1), "b": H.random_ids(cfg["vocab"], 215, 2)}
    eng = engine_for(cfg, w, dtype)
    got = FM.run_trace(eng, H.tail_decode_trace(reqs, tail=12))
    worst = FM.worst_error("E", cfg, w64, reqs, got)
    assert worst[0] <= TOL[dtype], worst
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:300], "want": list(range(0, 300, 7))},
                                     {"id": "b", "tokens": reqs["b"][:3], "want": [0, 1, 2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][300:301], "want": [0]},
                                     {"id": "b", "tokens": reqs["b"][3:200], "want": list(range(0, 197, 5))}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": reqs["a"][301:], "want": list(range(29))},
                                     {"id": "b", "tokens": reqs["b"][200:], "want": list(range(15))}], "end": ["a", "b"]}]
    got = FM.run_trace(eng, steps)
    worst = FM.worst_error("E", cfg, w64, reqs, got)
    assert worst[0] <= TOL[dtype], worst
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_step_that_repeats_is_replayed(dtype):
    """Prompts of one length, one after the other: from its third occurrence the step (attention over the pages, the
    scans in segments with their workspace, the state slot of whoever was there before) is replayed from a captured
    graph; every run is checked, with other work between the replays."""
    cfg, w, w64 = model("E", seed=9)
    eng = engine_for(cfg, w, dtype, max_requests=2)
    other = H.random_ids(cfg["vocab"], 40, 77)
    for k in range(6):
        ids = H.random_ids(cfg["vocab"], 200, 30 + k)
        got = FM.run_trace(eng, [{"step": 0, "entries": [{"id": "p", "tokens": ids, "want": [0, 64, 127, 128, 199]}],
                                  "end": ["p"]}])
        assert FM.worst_error(("E", k), cfg, w64, {"p": ids}, got)[0] <= TOL[dtype]
        got = FM.run_trace(eng, H.portions_trace({"o": other}, sizes=(7, 1, 12)))
        assert FM.worst_error("Eo", cfg, w64, {"o": other}, got)[0] <= TOL[dtype]
    assert eng.graph_replays >= 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_captured_steps(dtype):
    """Three requests decode 150 tokens together, past every window and over many page borders; steps of single tokens
    are replayed from captured graphs, and every replay is checked."""
    for name in ("A", "B"):
        cfg, w, w64 = model(name, seed=6)
        reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 90 + i) for i, n in enumerate([160, 171, 153])}
        eng = engine_for(cfg, w, dtype, max_requests=3)
        steps = [{"step": 0, "entries": [{"id": r, "tokens": ids[:len(ids) - 150], "want": [0]} for r, ids in reqs.items()],
                  "end": []}]
        for t in range(150):
            steps.append({"step": t + 1, "entries": [{"id": r, "tokens": [ids[len(ids) - 150 + t]], "want": [0]}
                                                     for r, ids in reqs.items()], "end": list(reqs) if t == 149 else []})
        got = FM.run_trace(eng, steps)
        assert eng.graph_replays >= 100
        worst = FM.worst_error(name, cfg, w64, reqs, got)
        assert worst[0] <= TOL[dtype], worst


def test_generation_command_line_and_replay_program(tmp_path):
    from tiny_inference_server_amd.engine.generate import generate
    cfg, w, w64 = model("A", seed=8)
    folder = FM.write_folder(str(tmp_path / "m"), cfg, w)
    prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6, 21))]
    want = [pf.greedy_generate(p, 9, w64, cfg) for p in prompts]
    out, s = generate(folder, prompts, max_new_tokens=9, temperature=0.0, dtype="float32", max_batch=3, token_budget=12,
                      pool_tokens=192, return_scheduler=True)
    assert out == want and s.peak_running == 3
    # sampled generation runs too (the sampling kernel on this model's logits)
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
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
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
        assert FM.worst_error("A8", cfg, w64, reqs, got)[0] <= TOL[dtype]
