"""The Fesupel architecture on the GPU: each new kernel against plain torch, and the engine with its HIP kernels against
the plain implementation through every kind of schedule, in 32-bit and in bfloat16."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import fesupel_models as FM
import helpers as H
import plain_fesupel as pf
from test_gpu_fikevik import fake_batch
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = FM.TOL
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def hip_ops(dtype):
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    return HipOps("cuda:0", DT[dtype])


def model(name, dtype="float32", seed=5):
    """In bfloat16 every expert is chosen (see fesupel_models.all_chosen); routing itself is tested in 32-bit and kernel
    by kernel in both types."""
    cfg = FM.CONFIGS[name] if dtype == "float32" else FM.all_chosen(FM.CONFIGS[name])
    w = FM.random_weights(cfg, seed)
    return copy.deepcopy(cfg), w, FM.as_f64(w)


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

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,G,kd,vd,chunk,cap", [(6, 2, 24, 40, 7, 3.0), (4, 4, 64, 16, 0, 0.0), (2, 1, 10, 200, 33, 30.0), (3, 1, 96, 48, 16, 1.0),
                                                  (16, 4, 32, 32, 5, 0.0), (1, 1, 64, 1, 1, 2.0), (5, 5, 7, 9, 300, 0.0)])
def test_attention_with_mixed_sigmoid_weights(dtype, Hq, G, kd, vd, chunk, cap):
    """Chunks that end mid-page, a whole prompt and a portion that goes on at 19 beside a new request; few rows, so
    the keys of a row are cut over several workgroups and added up."""
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(kd + chunk)
    ps, n_pages = 8, 12
    tables = [[5, 2, 9, 0, 0, 0], [7, 1, 3, 11, 4, 0]]
    cols = Hq * kd + G * kd + G * vd + 3
    biases = [0.3 * torch.randn(s, generator=g) for s in (Hq * kd, G * kd, G * vd)]
    head_bias, talk = torch.randn(Hq, generator=g) - 1, torch.eye(Hq) + 0.4 * torch.randn(Hq, Hq, generator=g)
    planes = [torch.full((n_pages, G * ps * (kd + vd)), float("nan"), dtype=DT[dtype]) for _ in range(2)]
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
            q = o.attention_prepare(mv(proj)[:, 3:], 0, Hq * kd, Hq * kd + G * kd, b.positions, b.write_slots["g"], plane, Hq, G, kd, vd,
                                    ps, value_norm=False, q_bias=mv(biases[0]), k_bias=mv(biases[1]), v_bias=mv(biases[2]))
            res.append(o.mixed_sigmoid_attention(q, plane, b, "g", Hq, G, kd, vd, ps, chunk, 0.37, cap, mv(head_bias), mv(talk)))
        close(res[0], res[1], dtype, "attention")
        assert torch.isfinite(res[0].float()).all()


@pytest.mark.parametrize("Hq,G,kd,vd,chunk,cap", [(4, 1, 64, 64, 100, 30.0), (16, 4, 128, 128, 333, 0.0), (5, 5, 24, 32, 7, 2.0), (6, 2, 40, 16, 0, 0.0),
                                                  (2, 1, 128, 64, 64, 10.0), (13, 1, 16, 48, 1, 0.0), (8, 8, 32, 32, 1000, 5.0)])
def test_matrix_core_attention_with_mixed_sigmoid_weights(Hq, G, kd, vd, chunk, cap):
    """bfloat16 and pages of 16 slots: tiles of rows that cross chunk edges and page borders, a portion that goes on in the
    middle of a page beside a new request, and single rows whose keys are cut over many workgroups; the pool is full of
    NaN where nothing was written."""
    ops, ref = hip_ops("bfloat16"), TorchOps("cpu", torch.bfloat16)
    g = torch.Generator().manual_seed(kd + chunk)
    ps, n_pages = 16, 40
    perm = torch.randperm(n_pages, generator=g).tolist()
    tables = [perm[:18] + [0, 0], perm[18:38]]
    cols = Hq * kd + G * kd + G * vd
    head_bias, talk = torch.randn(Hq, generator=g) - 2, torch.eye(Hq) + 0.4 * torch.randn(Hq, Hq, generator=g)
    planes = [torch.full((n_pages, G * ps * (kd + vd)), float("nan"), dtype=torch.bfloat16) for _ in range(2)]
    planes[0] = planes[0].cuda()
    for seq_rows, slots, tabs in (([(0, 0, 203)], [0], [tables[1]]), ([(0, 0, 37), (37, 203, 70)], [1, 0], [tables[0], tables[1]]),
                                  ([(0, 37, 1), (1, 273, 1)], [1, 0], [tables[0], tables[1]]),
                                  ([(0, 38, 2), (2, 274, 1), (3, 0, 0)][:2], [1, 0], [tables[0], tables[1]])):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        res = []
        for o, plane, dev in ((ops, planes[0], "cuda"), (ref, planes[1], "cpu")):
            b = fake_batch(seq_rows, slots, tabs, ps, dev)
            q = o.attention_prepare(proj.to(dev), 0, Hq * kd, Hq * kd + G * kd, b.positions, b.write_slots["g"], plane, Hq, G, kd, vd,
                                    ps, value_norm=False)
            res.append(o.mixed_sigmoid_attention(q, plane, b, "g", Hq, G, kd, vd, ps, chunk, kd ** -0.5, cap, head_bias.to(dev),
                                                 talk.to(dev)))
        assert ops._mixed_on_matrix_cores(res[0], kd, vd, ps, Hq)
        assert torch.isfinite(res[0].float()).all()
        close(res[0], res[1], "bfloat16", f"attention of {seq_rows}", tol=2.5e-2)


def test_attention_of_many_rows_and_long_chunks():
    """Hundreds of rows (one workgroup a row, no key splits) over chunks longer than a block of keys."""
    ops, ref = hip_ops("float32"), TorchOps("cpu", torch.float32)
    g = torch.Generator().manual_seed(3)
    Hq, G, kd, vd, ps, n = 4, 2, 16, 8, 16, 700
    table = [list(torch.randperm(48, generator=g)[:44].tolist())]
    plane = torch.randn(48, G * ps * (kd + vd), generator=g)
    q = torch.randn(n, Hq * kd, generator=g)
    head_bias, talk = torch.randn(Hq, generator=g) - 3, torch.randn(Hq, Hq, generator=g)
    for chunk in (0, 300):
        outs = []
        for o, dev in ((ops, "cuda"), (ref, "cpu")):
            b = fake_batch([(0, 0, n)], [0], table, ps, dev)
            outs.append(o.mixed_sigmoid_attention(q.to(dev), plane.to(dev), b, "g", Hq, G, kd, vd, ps, chunk, 0.2, 4.0,
                                                  head_bias.to(dev), talk.to(dev)))
        close(outs[0], outs[1], "float32", f"chunks of {chunk}", tol=1e-4)


@pytest.mark.parametrize("Hh,G,D,V,K", [(4, 2, 12, 8, 4), (6, 3, 8, 4, 2), (2, 1, 20, 6, 1), (4, 2, 64, 32, 4), (2, 1, 128, 64, 3), (1, 1, 1, 8, 2),
                                        (3, 1, 6, 1, 1), (2, 2, 200, 20, 2), (2, 1, 33, 17, 3)])
def test_the_delta_rules_kernels(Hh, G, D, V, K):
    """The step before the walk and the walk: a whole prompt from an empty line, then portions and single rows that go on
    from used lines, beside a new request."""
    ops, ref = hip_ops("float32"), TorchOps("cpu", torch.float32)
    g = torch.Generator().manual_seed(D + V)
    C = 2 * G * D + Hh * V
    cols = 5 + C + Hh
    taps = torch.randn(C, K, generator=g) / K ** 0.5
    at = Hh * -(-V // 16) * D * 16           # the matrix state in blocks of 16 value channels, then the convolution's inputs
    floats = at + (K - 1) * C
    floats += -floats % 4 + 4                # lines start 16 bytes aligned
    states = [torch.zeros(3, floats), torch.zeros(3, floats).cuda()]
    for seq_rows, slots in (([(0, 0, 37)], [2]), ([(0, 37, 1), (1, 0, 9)], [2, 0]), ([(0, 9, 70), (70, 38, 2)], [0, 2]),
                            ([(0, 40, 1), (1, 79, 1)], [2, 0])):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        decay = torch.rand(n, Hh * D, generator=g) * 0.5 + 0.5
        res = []
        for o, st, dev in ((ref, states[0], "cpu"), (ops, states[1], "cuda")):
            b = fake_batch(seq_rows, slots, None, 8, dev)
            u = o.delta_prepare(proj.to(dev), 5, 5 + C, taps.to(dev), st, at, b, Hh, G, D, V)
            o.conv_state_update(proj.to(dev), 5, C, K, st, at, b)
            res.append((u, o.delta_scan(u, 0, G * D, 2 * G * D, C, decay.to(dev), st, b, Hh, G, D, V)))
        close(res[1][0], res[0][0], "float32", "prepared rows", tol=1e-5)
        close(res[1][1], res[0][1], "float32", "outputs", tol=1e-4)
        close(states[1], states[0], "float32", "state lines", tol=1e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,W", [(23, 44), (5, 328), (300, 1500)])
def test_row_kernels_of_the_block(dtype, n, W):
    from tiny_inference_server_amd.ops.hip_ops import ChosenExperts
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(W)
    y0, y1 = torch.randn(n, W + 3, generator=g) * 3, torch.randn(n, W, generator=g) * 0.1
    g0, g1 = 1 + 0.3 * torch.randn(W, generator=g), 1 + 0.3 * torch.randn(W, generator=g)
    close(ops.normed_mean([(y0.cuda()[:, 3:], g0.cuda()), (y1.cuda(), g1.cuda())], 1e-5), ref.normed_mean([(y0[:, 3:], g0), (y1, g1)], 1e-5),
          "float32", "mean of two normed rows")
    close(ops.normed_mean([(y1.cuda(), g1.cuda())], 1e-6), ref.normed_mean([(y1, g1)], 1e-6), "float32", "one normed row")
    for act in ("relu2", "gelu_tanh", "silu", "sigmoid"):
        close(ops.activate_rows(y0.cuda()[:, 3:], act), ref.activate_rows(y0[:, 3:], act), dtype, act)
    z = torch.randn(n, 2 * 40 + 1, generator=g) * 2
    close(ops.gated_act(z.cuda(), 40, "clamped_swish", limit=0.8), ref.gated_act(z, 40, "clamped_swish", limit=0.8), dtype, "clamped gate")
    rank = 7
    low, w2, bias, rate = torch.randn(n, rank + 2, generator=g), torch.randn(W, rank, generator=g), torch.randn(W, generator=g), torch.rand(W // 4, generator=g)
    if W % 4 == 0:
        close(ops.lowrank_act(low.cuda()[:, 2:], w2.cuda(), bias.cuda(), "exp_softplus", rate=rate.cuda(), group=4),
              ref.lowrank_act(low[:, 2:], w2, bias, "exp_softplus", rate=rate, group=4), "float32", "decays")
    close(ops.lowrank_act(low.cuda()[:, 2:], w2.cuda(), None, "none"), ref.lowrank_act(low[:, 2:], w2, None, "none"), "float32", "low-rank product")
    # the residual sum with a row's chosen experts, identity experts, a gated shared term and a norm on the branch
    top, E = 3, 4
    x = torch.randn(n, W, generator=g)
    lines, extra, gate = torch.randn(n * top, W, generator=g), torch.randn(n, W, generator=g), torch.randn(n, 5, generator=g)
    ids = torch.randint(0, E + 2, (n, top), generator=g, dtype=torch.int32)
    wts = torch.rand(n, top, generator=g)
    rows = x.to(DT[dtype])
    res = []
    for o, dev in ((ops, "cuda"), (ref, "cpu")):
        ch = ChosenExperts(lines.to(dev), ids.to(dev), wts.to(dev), E, rows.to(dev), extra.to(dev), gate.to(dev)[:, 2:3])
        res.append(o.residual_norm(x.clone().to(dev), ch, y_rms=(g0.to(dev), 1e-5), copy=True, norm=("rms", g1.to(dev), None, 1e-5)))
    close(res[0][0], res[1][0], "float32", "sum", tol=1e-4 if dtype == "float32" else 2e-2)
    close(res[0][2], res[1][2], dtype, "the next norm", tol=1e-4 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("n,N,top,groups", [(37, 8, 2, (4, 2)), (5, 12, 3, (3, 1)), (200, 16, 3, (2, 1)), (9, 6, 6, None), (64, 64, 4, (16, 3)),
                                            (33, 10, 1, (10, 1)), (20, 130, 5, (13, 2))])
def test_choice_in_groups(n, N, top, groups):
    ops, ref = hip_ops("float32"), TorchOps("cpu", torch.float32)
    g = torch.Generator().manual_seed(N)
    z, c = torch.randn(n, N + 2, generator=g) * 2, torch.randn(N, generator=g) * 0.1 - 0.5      # corrected scores are negative
    ids, w = ops.route_topk(z.cuda()[:, 2:], c.cuda(), 1.0, top, groups=groups, renorm=True)
    ids_r, w_r = ref.route_topk(z[:, 2:], c, 1.0, top, groups=groups, renorm=True)
    assert torch.equal(ids.cpu(), ids_r)
    close(w, w_r, "float32", "weights")
    assert torch.allclose(w.sum(-1).cpu(), torch.ones(n), atol=1e-5)
    if groups:
        per = N // groups[0]
        assert all(len({int(e) // per for e in row}) <= groups[1] for row in ids.cpu())


# ---- the engine ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(FM.CONFIGS))
def test_schedules(name, dtype):
    if name == "D" and dtype == "bfloat16":
        pytest.skip("the configuration of ones divides single numbers by their own size: bfloat16 rounding is all of it")
    cfg, w, w64 = model(name, dtype)
    key = (name, dtype)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 158, 23, 70])}
    eng = engine_for(cfg, w, dtype)
    tol = 3e-4 if name == "D" else None

    def check(got):
        if tol:
            assert FM.worst_error(key, cfg, w64, reqs, got)[0] <= tol
        else:
            FM.check(key, cfg, w64, reqs, got, dtype)

    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=20), H.portions_trace(reqs, seed=3)):
        got = FM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        check(got)
        eng.cache.check()
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, dtype, max_requests=3, max_tokens=peak)
    check(FM.run_trace(eng, steps))
    eng.cache.check()


def needle_case(name, dtype, at, distance, side, chunk):
    cfg, w, _ = model(name, dtype)
    if chunk is not None:
        cfg["layers"][0]["mixer"]["left"]["mask"] = {"size": chunk}
    w = FM.sharpen(cfg, w, 3, 7, side)
    w64 = FM.as_f64(w)
    ids = [t if t not in (3, 7) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, 60 + at)]
    ids[at], ids[at + distance] = 3, 7
    key = (name, dtype, "sharp", side, chunk)
    want = FM.plain_logits(key, cfg, w64, ids)
    without = list(ids)
    without[at] = 11
    moved = FM.relative_error(pf.forward(cfg, w64, without)[at + distance], want[at + distance])
    return key, cfg, w, w64, ids, want, moved


def run_three_ways(key, cfg, w, w64, ids, want, place, bound, dtype, tail=6):
    eng = engine_for(cfg, w, dtype)
    for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=tail), H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
        got = FM.run_trace(eng, steps)
        err = FM.relative_error(got[("s", place)], want[place])
        assert err <= bound, (err, bound, place)
        FM.check(key, cfg, w64, {"s": ids}, got, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,distance,side,chunk", [("A", 1, "left", None), ("C", 300, "left", 400), ("C", 150, "right", None),
                                                      ("B", 60, "right", None)])
def test_a_token_that_stands_out(name, distance, side, chunk, dtype):
    """A probe token that looks for a needle right before it or hundreds of tokens back, through attention's pages or the
    delta rule's state, with the needle on both sides of a page's border: whole, decoded alone, in portions."""
    for at in (15, 16):
        key, cfg, w, w64, ids, want, moved = needle_case(name, dtype, at, distance, side, chunk)
        assert moved >= 0.01, moved
        run_three_ways(key, cfg, w, w64, ids, want, at + distance, min(TOL[dtype], moved / 3), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,chunk", [("A", 21), ("A", 32), ("C", 48)])
def test_keys_just_inside_and_just_outside_a_chunk(name, chunk, dtype):
    """The needle at a chunk's first position and the probe at its last (the farthest key a row ever sees), the probe at
    the next chunk's first position (the needle has just gone out of sight), and the two on either side of an edge.
    Chunks that end inside a page and at a page's border."""
    c0 = 2 * chunk
    for at, distance, seen in ((c0, chunk - 1, True), (c0, chunk, False), (c0 + chunk - 1, 1, False), (c0 + chunk - 2, 1, True)):
        key, cfg, w, w64, ids, want, moved = needle_case(name, dtype, at, distance, "left", chunk)
        assert (moved >= 0.01) if seen else True, (at, distance, moved)
        run_three_ways(key, cfg, w, w64, ids, want, at + distance, TOL[dtype] if not seen else min(TOL[dtype], moved / 3), dtype,
                       tail=chunk + 3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_and_wide_heads(dtype):
    """Heads of 64 and 128 channels, prompts over many pages and chunks, then decoded tokens; alone and two requests
    together, the second cut into portions."""
    cfg, w, w64 = model("C", dtype, seed=9)
    key = ("C9", dtype)
    reqs = {"a": H.random_ids(cfg["vocab"], 330, 1), "b": H.random_ids(cfg["vocab"], 215, 2)}
    eng = engine_for(cfg, w, dtype)
    got = FM.run_trace(eng, H.tail_decode_trace(reqs, tail=12))
    FM.check(key, cfg, w64, reqs, got, dtype)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:300], "want": list(range(0, 300, 7))},
                                     {"id": "b", "tokens": reqs["b"][:3], "want": [0, 1, 2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][300:301], "want": [0]},
                                     {"id": "b", "tokens": reqs["b"][3:200], "want": list(range(0, 197, 5))}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": reqs["a"][301:], "want": list(range(29))},
                                     {"id": "b", "tokens": reqs["b"][200:], "want": list(range(15))}], "end": ["a", "b"]}]
    got = FM.run_trace(eng, steps)
    FM.check(key, cfg, w64, reqs, got, dtype)
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_captured_steps(dtype):
    """Three requests decode 150 tokens together, over many page borders and chunk edges; steps of single tokens are
    replayed from captured graphs, and every replay is checked."""
    for name in ("A", "C"):
        cfg, w, w64 = model(name, dtype, seed=6)
        reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 90 + i) for i, n in enumerate([160, 171, 153])}
        eng = engine_for(cfg, w, dtype, max_requests=3)
        steps = [{"step": 0, "entries": [{"id": r, "tokens": ids[:len(ids) - 150], "want": [0]} for r, ids in reqs.items()],
                  "end": []}]
        for t in range(150):
            steps.append({"step": t + 1, "entries": [{"id": r, "tokens": [ids[len(ids) - 150 + t]], "want": [0]}
                                                     for r, ids in reqs.items()], "end": list(reqs) if t == 149 else []})
        got = FM.run_trace(eng, steps)
        assert eng.graph_replays >= 100
        FM.check((name, dtype, 6), cfg, w64, reqs, got, dtype)


def test_generation_command_line_and_replay_program(tmp_path):
    from tiny_inference_server_amd.engine.generate import generate
    cfg, w, w64 = model("A", seed=8)
    bare = copy.deepcopy(cfg)
    for e in bare["layers"]:                   # as a model folder comes: the two ranks are the weight file's to say
        del e["mixer"]["right"]["decay_rank"], e["mixer"]["right"]["gate_rank"]
    folder = FM.write_folder(str(tmp_path / "m"), bare, w)
    prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6, 21))]
    want = [pf.greedy_generate(cfg, w64, p, 9) for p in prompts]
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
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / ("out_" + dtype)
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
        if dtype == "float32":
            assert FM.worst_error("A8", cfg, w64, reqs, got)[0] <= TOL["float32"]
        else:
            errs = FM.errors("A8", cfg, w64, reqs, got)        # (the router chooses here: most rows are not close calls)
            assert errs[len(errs) // 2][0] <= TOL["bfloat16"] / 2
