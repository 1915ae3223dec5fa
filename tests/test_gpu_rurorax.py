"""The Rurorax architecture on the GPU: each new kernel against plain torch, and the engine with its HIP kernels against
the plain implementation through every kind of schedule, in 32-bit and in bfloat16."""
import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers as H
import plain_rurorax as pr
import rurorax_models as RM
from test_gpu_fikevik import fake_batch
from torch_ops import TorchOps

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = RM.TOL
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def hip_ops(dtype):
    from tiny_inference_server_amd.ops.hip_ops import HipOps
    return HipOps("cuda:0", DT[dtype])


def model(name, dtype="float32", seed=5):
    """In bfloat16 every expert is chosen (see rurorax_models.all_chosen); routing itself is tested in 32-bit and kernel
    by kernel in both types."""
    cfg = RM.CONFIGS[name] if dtype == "float32" else RM.all_chosen(RM.CONFIGS[name])
    w = RM.random_weights(cfg, seed)
    return copy.deepcopy(cfg), w, RM.as_f64(w)


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

@pytest.mark.parametrize("D", [44, 328, 1500, 4200])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_dynamic_tanh_scaled_sum_gated_act_and_cap(dtype, D):
    from tiny_inference_server_amd.ops.hip_ops import ChosenExperts
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(D)
    n, top = 23, 3
    x = torch.randn(n, D, generator=g) * 2 + 0.3
    gain, bias, s1, s2, b1 = (1 + 0.3 * torch.randn(D, generator=g) for _ in range(5))
    dev = lambda t: None if t is None else t.cuda()
    close(ops.dyt32(x.cuda(), 0.7, gain.cuda(), bias.cuda()), ref.dyt32(x, 0.7, gain, bias), dtype, "dyt32")
    close(ops.dyt32(x.cuda(), 1.3, gain.cuda()), ref.dyt32(x, 1.3, gain), dtype, "dyt32 without a bias")
    y1, y2 = torch.randn(n, D + 5, generator=g), torch.randn(n, D, generator=g)
    lines = torch.randn(n * top, D, generator=g)
    ids = torch.randint(0, 4, (n, top), generator=g, dtype=torch.int32)
    rows = x.to(DT[dtype])
    for branches, norm in (([(y1[:, 5:], s1, b1), (y2, s2, None)], ("dyt", 0.6, gain, bias)),
                           ([(y1[:, 5:], None, None)], None),
                           ([(y2, s1, None), (ChosenExperts(lines, ids, None, 4, rows), s2, None)], ("dyt", 0.9, gain, bias)),
                           ([(y2, s1, b1), (ChosenExperts(lines, ids, None, 4, rows), None, None)], None)):
        def on(move):
            out = []
            for y, s, b in branches:
                if isinstance(y, ChosenExperts):
                    y = ChosenExperts(move(y.results), move(y.ids), None, 4, move(y.rows))
                else:
                    y = move(y)
                out.append((y, None if s is None else move(s), None if b is None else move(b)))
            return out
        got = ops.scaled_sum(x.clone().cuda(), on(lambda t: t.cuda()), norm=(norm[0], norm[1], dev(norm[2]), dev(norm[3])) if norm else None)
        want = ref.scaled_sum(x.clone(), on(lambda t: t), norm=norm)
        close(got[0], want[0], "float32", "sum")
        assert (got[1] is None) == (want[1] is None)
        if want[1] is not None:
            close(got[1], want[1], dtype, "the norm of the sum")
    hidden = D // 2
    z = torch.randn(n, 2 * hidden + 3, generator=g)
    gb, ub, rs = torch.randn(hidden, generator=g), torch.randn(hidden, generator=g), torch.rand(n, generator=g)
    for act in ("gelu_tanh", "silu"):
        close(ops.gated_act(z.cuda(), hidden, act, gate_bias=gb.cuda(), up_bias=ub.cuda()), ref.gated_act(z, hidden, act, gb, ub), dtype,
              "gated_act with biases " + act)
        close(ops.gated_act(z.cuda(), hidden, act, row_scale=rs.cuda()), ref.gated_act(z, hidden, act, row_scale=rs), dtype,
              "gated_act with a factor per row " + act)
    lg = 30 * torch.randn(n, D, generator=g)
    close(ops.softcap(lg.clone().cuda(), 15.0), ref.softcap(lg.clone(), 15.0), "float32", "softcap")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Hq,G,kd,vd,chunk,rot", [(6, 2, 24, 40, 7, 10), (4, 4, 64, 16, 0, 64), (2, 1, 10, 200, 33, 0), (3, 1, 96, 48, 16, 24),
                                                  (4, 2, 32, 32, 5, 8), (2, 1, 64, 64, 1, 0)])
def test_attention_inside_chunks(dtype, Hq, G, kd, vd, chunk, rot):
    """The step before attention (biases, a norm over all heads at once, rotation of pairs half the rotated part apart,
    the pages) and attention inside chunks of positions that end mid-page, for a whole prompt and for a portion that
    goes on at 19 beside a new request."""
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(kd + chunk)
    ps, n_pages = 8, 12
    tables = [[5, 2, 9, 0, 0, 0], [7, 1, 3, 11, 4, 0]]
    cols = Hq * kd + G * kd + G * vd + 3
    q_gain, k_gain = 1 + 0.2 * torch.randn(Hq * kd, generator=g), 1 + 0.2 * torch.randn(G * kd, generator=g)
    biases = [0.3 * torch.randn(s, generator=g) for s in (Hq * kd, G * kd, G * vd)]
    freqs = (50.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / max(rot, 1)) / 3.0).float()
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
                                    ps, mv(q_gain), mv(k_gain), freqs=mv(freqs), rot_dims=rot, eps=1e-5, value_norm=False,
                                    q_bias=mv(biases[0]), k_bias=mv(biases[1]), v_bias=mv(biases[2]), whole_norm=True, pair_half=True)
            res.append((q, o.paged_attention_kv(q, plane, b, "g", Hq, G, kd, vd, ps, 0, 0.37, chunk=chunk)))
        close(res[0][0], res[1][0], dtype, "queries")
        close(res[0][1], res[1][1], dtype, "attention")
        assert torch.isfinite(res[0][1].float()).all()


@pytest.mark.parametrize("hd,Hq,G,chunk", [(64, 8, 2, 100), (128, 4, 1, 333), (32, 6, 6, 64), (128, 16, 4, 1024)])
def test_matrix_core_attention_inside_chunks(hd, Hq, G, chunk):
    """Keys and values of one size in bfloat16 go to the matrix-core kernels, which are told of chunks by a negative
    window: a long portion whose tiles of rows cross chunk edges, decoded tokens deep in their requests right before and
    right after an edge, and short portions that straddle one, against plain torch over the same pages."""
    ops, ref = hip_ops("bfloat16"), TorchOps("cpu", torch.bfloat16)
    g = torch.Generator().manual_seed(hd)
    ps, n_pages = 16, 200
    plane = torch.randn(n_pages, 2, G, ps, hd, generator=g).to(torch.bfloat16)
    perm = torch.randperm(n_pages, generator=g).tolist()
    tables = [perm[:64] + [0] * 64, perm[64:192]]
    edge = 5 * chunk if chunk < 300 else chunk
    for seq_rows in ([(0, 0, 700)], [(0, edge - 1, 1), (1, edge, 1)], [(0, edge - 4, 9), (9, 40, 1)], [(0, edge - 30, 300)],
                     [(0, 1000, 1), (1, 1900, 1)]):
        n = sum(r[2] for r in seq_rows)
        q = (torch.randn(n, Hq * hd, generator=g) * 1.5).to(torch.bfloat16)
        tabs = tables[:len(seq_rows)] if len(seq_rows) > 1 else [tables[1]]
        got = ops.paged_attention(q.cuda(), plane.cuda(), fake_batch(seq_rows, list(range(len(seq_rows))), tabs, ps, "cuda"), "g",
                                  Hq, G, hd, -chunk, hd ** -0.5)
        want = ref.paged_attention(q, plane, fake_batch(seq_rows, list(range(len(seq_rows))), tabs, ps, "cpu"), "g", Hq, G, hd,
                                   -chunk, hd ** -0.5)
        close(got, want, "bfloat16", f"attention {seq_rows} in chunks of {chunk}")


@pytest.mark.parametrize("segment", [64, 8, 5])
@pytest.mark.parametrize("Hh,P,N,G,K,parts", [(4, 8, 12, 2, 4, 2), (6, 4, 5, 3, 3, 3), (4, 64, 64, 2, 4, 2), (4, 6, 4, 4, 1, 4), (2, 32, 128, 1, 2, 1),
                                               (8, 64, 128, 1, 4, 1)])
def test_the_state_space_mixers_kernels(Hh, P, N, G, K, parts, segment):
    """The convolution over a request's kept inputs with silu, the step sizes and decays, the inputs kept for the next
    call, the scan with a decay per head and keys shared by a group of heads, and the gate before the norm in parts:
    portions of three requests in one call, then their next portions and single tokens, on state lines that start from
    what an earlier owner left (cleared, as the cache manager clears a slot that is taken)."""
    ops, ref = hip_ops("float32"), TorchOps("cpu", torch.float32)
    ops.scan_segment = segment
    g = torch.Generator().manual_seed(N + K)
    inner, C = Hh * P, Hh * P + 2 * G * N
    conv_at = ops.state_scan_floats("decay", Hh, N, P)
    state = torch.zeros(5, conv_at + (K - 1) * C)
    state_gpu = state.cuda()
    taps, tap_bias = torch.randn(C, K, generator=g) / K ** 0.5, 0.2 * torch.randn(C, generator=g)
    dt_bias, neg_a = -1.5 + torch.rand(Hh, generator=g), -torch.exp(-2 + 2 * torch.rand(Hh, generator=g))
    skip, gain = torch.randn(Hh, generator=g), 1 + 0.2 * torch.randn(inner, generator=g)
    cols = inner + C + Hh + 3
    for seq_rows, slots in (([(0, 0, 37), (37, 0, 1), (38, 0, 18)], [3, 0, 4]), ([(0, 37, 2), (2, 1, 1), (3, 18, 40)], [3, 0, 4]),
                            ([(0, 39, 1), (1, 2, 1), (2, 58, 1)], [3, 0, 4])):
        n = sum(r[2] for r in seq_rows)
        proj = torch.randn(n, cols, generator=g)
        outs = []
        for o, st, dev in ((ops, state_gpu, "cuda"), (ref, state, "cpu")):
            mv = lambda t: t.to(dev)
            b = fake_batch(seq_rows, slots, None, 1, dev)
            p = mv(proj)[:, 3:]
            u = o.conv_prepare(p, inner, inner + C, mv(taps), mv(tap_bias), mv(dt_bias), mv(neg_a), st, conv_at, b, Hh, P)
            o.conv_state_update(p, inner, C, K, st, conv_at, b)
            y = o.state_scan("decay", u, inner + G * N, inner, C, 1.0, st, b, Hh, N, P, decay=u[:, C + inner:], qk_group=Hh // G,
                             decay_per_head=True)
            outs.append((u, y, o.gated_group_norm(y, u[:, :inner], mv(skip), P, p[:, :inner], mv(gain), 1e-5, parts)))
        for a, b_, what in zip(outs[0], outs[1], ("convolution, steps and decays", "scan", "gate and norm")):
            close(a, b_, "float32", what)
    close(state_gpu, state, "float32", "state and kept inputs")
    assert state_gpu[[1, 2]].abs().max() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,W,F,E,top", [(37, 64, 40, 6, 2), (5, 44, 20, 3, 3), (200, 128, 72, 16, 3), (9, 48, 30, 2, 1), (600, 64, 48, 4, 1),
                                         (700, 128, 80, 10, 2), (1, 328, 72, 9, 1)])
def test_sigmoid_router_and_experts_that_read_a_weighted_row(dtype, n, W, F, E, top):
    ops, ref = hip_ops(dtype), TorchOps("cpu", DT[dtype])
    g = torch.Generator().manual_seed(n)
    z = 2 * torch.randn(n, E + 3, generator=g)
    ids, wts = ops.route_topk(z.cuda()[:, 3:], None, 1.0, top, score="sigmoid")
    ids_r, wts_r = ref.route_topk(z[:, 3:], None, 1.0, top, score="sigmoid")
    assert torch.equal(ids.cpu().sort(dim=1).values, ids_r.sort(dim=1).values)
    order = ids.cpu().long().argsort(dim=1), ids_r.long().argsort(dim=1)
    close(torch.gather(wts.cpu(), 1, order[0]), torch.gather(wts_r, 1, order[1]), "float32", "weights")
    want_w = torch.sigmoid(z[:, 3:]).topk(top, dim=1).values          # the scores themselves, not made to sum to one
    close(wts.cpu().sort(dim=1, descending=True).values, want_w, "float32", "weights against sigmoid")
    x = torch.randn(n, W, generator=g).to(DT[dtype])
    gate_up = (torch.randn(E, 2 * F, W, generator=g) / W ** 0.5).to(DT[dtype])
    down = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(DT[dtype])
    got = ops.gated_experts(x.cuda(), ids, wts, gate_up.cuda(), down.cuda())
    want = ref.gated_experts(x, ids.cpu(), wts.cpu(), gate_up, down)
    assert got.weights is None and want.weights is None
    close(got.results, want.results, dtype, "experts")
    # against the definition: expert(w * x) with the row scaled before the first product
    xs = x.double()
    for r in range(0, n, max(1, n // 7)):
        for c in range(top):
            e, wgt = int(ids[r, c]), float(wts[r, c])
            gu = gate_up[e].double() @ (wgt * xs[r])
            line = down[e].double() @ (gu[:F] * torch.sigmoid(gu[:F]) * gu[F:])
            close(got.results[r * top + c], line, dtype, "an expert's line", tol=3e-5 if dtype == "float32" else 3e-2)


# ---- the engine ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(RM.CONFIGS))
def test_schedules(name, dtype):
    cfg, w, w64 = model(name, dtype)
    key = (name, dtype)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 158, 23, 70])}
    eng = engine_for(cfg, w, dtype)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=20), H.portions_trace(reqs, seed=3)):
        got = RM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        RM.check(key, cfg, w64, reqs, got, dtype)
        eng.cache.check()
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, dtype, max_requests=3, max_tokens=peak)
    got = RM.run_trace(eng, steps)
    RM.check(key, cfg, w64, reqs, got, dtype)
    eng.cache.check()


def needle_case(name, dtype, at, distance, chunk):
    cfg, w, _ = model(name, dtype)
    if chunk is not None:
        cfg["layers"][0]["mixer"]["mask"] = {"size": chunk}
    w = RM.sharpen(cfg, w, 3, 7)
    w64 = RM.as_f64(w)
    ids = [t if t not in (3, 7) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, 60 + at)]
    ids[at], ids[at + distance] = 3, 7
    key = (name, dtype, "sharp", chunk)
    want = RM.plain_logits(key, cfg, w64, ids)
    without = list(ids)
    without[at] = 11
    moved = RM.relative_error(pr.forward(cfg, w64, without)[at + distance], want[at + distance])
    return key, cfg, w, w64, ids, want, moved


def run_three_ways(key, cfg, w, w64, ids, want, place, bound, dtype, tail=6):
    eng = engine_for(cfg, w, dtype)
    for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=tail), H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
        got = RM.run_trace(eng, steps)
        err = RM.relative_error(got[("s", place)], want[place])
        assert err <= bound, (err, bound, place)
        RM.check(key, cfg, w64, {"s": ids}, got, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,distance,chunk", [("A", 1, None), ("C", 300, 400), ("E", 250, None), ("D", 150, None)])
def test_a_token_that_stands_out(name, distance, chunk, dtype):
    """A probe token that looks for a needle right before it or hundreds of tokens back, through attention's pages or the
    recurrent state, with the needle on both sides of a page's border: whole, decoded alone, in portions."""
    for at in (15, 16):
        key, cfg, w, w64, ids, want, moved = needle_case(name, dtype, at, distance, chunk)
        assert moved >= 0.01, moved
        run_three_ways(key, cfg, w, w64, ids, want, at + distance, min(TOL[dtype], moved / 3), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,chunk", [("A", 21), ("A", 32), ("C", 48), ("C", 100)])
def test_keys_just_inside_and_just_outside_a_chunk(name, chunk, dtype):
    """The needle at a chunk's first position and the probe at its last (the farthest key a row ever sees), the probe at
    the next chunk's first position (the needle has just gone out of sight), and the two on either side of an edge.
    Chunks that end inside a page and at a page's border; keys and values of different sizes and of one size (the
    matrix-core kernels in bfloat16)."""
    c0 = 2 * chunk
    for at, distance, seen in ((c0, chunk - 1, True), (c0, chunk, False), (c0 + chunk - 1, 1, False), (c0 + chunk - 2, 1, True)):
        key, cfg, w, w64, ids, want, moved = needle_case(name, dtype, at, distance, chunk)
        assert (moved >= 0.01) if seen else True, (at, distance, moved)
        run_three_ways(key, cfg, w, w64, ids, want, at + distance, TOL[dtype] if not seen else min(TOL[dtype], moved / 3), dtype,
                       tail=chunk + 3)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_and_wide_heads(dtype):
    """Heads of 64 and 128 channels, prompts long enough for the scan to run in segments and for tiles of rows to cross
    chunk edges, then decoded tokens; alone and two requests together, the second cut into portions."""
    cfg, w, w64 = model("C", dtype, seed=9)
    key = ("C9", dtype)
    reqs = {"a": H.random_ids(cfg["vocab"], 330, 1), "b": H.random_ids(cfg["vocab"], 215, 2)}
    eng = engine_for(cfg, w, dtype)
    got = RM.run_trace(eng, H.tail_decode_trace(reqs, tail=12))
    RM.check(key, cfg, w64, reqs, got, dtype)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs["a"][:300], "want": list(range(0, 300, 7))},
                                     {"id": "b", "tokens": reqs["b"][:3], "want": [0, 1, 2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": reqs["a"][300:301], "want": [0]},
                                     {"id": "b", "tokens": reqs["b"][3:200], "want": list(range(0, 197, 5))}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": reqs["a"][301:], "want": list(range(29))},
                                     {"id": "b", "tokens": reqs["b"][200:], "want": list(range(15))}], "end": ["a", "b"]}]
    got = RM.run_trace(eng, steps)
    RM.check(key, cfg, w64, reqs, got, dtype)
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
        got = RM.run_trace(eng, steps)
        assert eng.graph_replays >= 100
        RM.check((name, dtype, 6), cfg, w64, reqs, got, dtype)


def test_generation_command_line_and_replay_program(tmp_path):
    from tiny_inference_server_amd.engine.generate import generate
    cfg, w, w64 = model("A", seed=8)
    folder = RM.write_folder(str(tmp_path / "m"), cfg, w)
    prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6, 21))]
    want = [pr.greedy_generate(cfg, w64, p, 9) for p in prompts]
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
            assert RM.worst_error("A8", cfg, w64, reqs, got)[0] <= TOL["float32"]
        else:
            errs = RM.errors("A8", cfg, w64, reqs, got)        # (the router chooses here: most rows are not close calls)
            assert errs[len(errs) // 2][0] <= TOL["bfloat16"] / 2
