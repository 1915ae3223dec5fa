"""The Rurorax architecture on the host: its configuration and spec, the plain implementation's mechanisms against
closed forms, and the engine (step function, cache manager, scheduler, generate) on the torch stand-ins for the kernels
against the plain implementation, in 32-bit."""
import copy
import math

import pytest
import torch

import helpers as H
import plain_rurorax as pr
import rurorax_models as RM
from torch_ops import TorchOps
from tiny_inference_server_amd.config import ARCHITECTURES, ConfigError, config_from_dict, load_config
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.weights.loader import spec_tensors

TOL32 = 3e-5
F64 = torch.float64


def model(name, seed=5):
    cfg = RM.CONFIGS[name]
    w = RM.random_weights(cfg, seed)
    return cfg, w, RM.as_f64(w)


def engine_for(cfg, w, **kw):
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 8)
    kw.setdefault("max_tokens", 640)
    return Engine(config=config_from_dict(cfg), tensors={n: t.float() for n, t in w.items()}, dtype="float32",
                  ops=TorchOps(graphs=kw.pop("graphs", False)), **kw)


# ---- configuration and spec ------------------------------------------------------------------------------------

def test_spec_names_every_tensor(tmp_path):
    for name, cfg in RM.CONFIGS.items():
        w = RM.random_weights(cfg, 1)
        folder = RM.write_folder(str(tmp_path / name), cfg, w)
        c = load_config(folder)
        assert c.architecture == "Rurorax" and c.to_dict() == config_from_dict(c.to_dict()).to_dict()
        spec = ARCHITECTURES.get(c.architecture).build_spec(c)
        assert spec_tensors(spec) == {n: tuple(t.shape) for n, t in w.items()}
        assert len(spec.stages[0].calls) == len(spec.layers) == len(cfg["layers"])
        assert spec.lm_head == spec.embedding == "embed"                  # one table at both ends
        assert spec.logit_softcap == cfg.get("logit_softcap", 0.0)
        for layer, entry in zip(spec.layers, cfg["layers"]):
            assert ("feed_forward" in layer.parts) == (entry["mlp"] is not None)
            assert layer.parts["mixer"].kind == {"attention": "chunked_attention", "mamba2": "selective_state_space"}[entry["type"]]


def test_configuration_errors_name_the_key():
    good = RM.CONFIGS["A"]
    for path, value, word in [(("layers", 0, "type"), "conv", "type"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mixer", "rot", "dims"), 3, "rot.dims"), (("layers", 0, "mixer", "mask", "size"), 0, "size"),
                              (("layers", 1, "mixer", "groups"), 3, "groups"), (("layers", 1, "mixer", "norm_groups"), 5, "norm_groups"),
                              (("layers", 1, "mlp", "router", "top"), 9, "top"), (("layers", 0, "mlp", "kind"), "gated", "mlp"),
                              (("norm",), {}, "eps"), (("logit_softcap",), -1.0, "logit_softcap")]:
        bad = copy.deepcopy(good)
        d = bad
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            config_from_dict(bad)


# ---- the plain implementation's mechanisms against closed forms ----------------------------------------------------

def test_plain_chunks_and_rotation():
    vis = pr.chunk_visible(11, 4)
    for i in range(11):
        assert vis[i].nonzero().flatten().tolist() == list(range(i - i % 4, i + 1))
    assert torch.equal(pr.chunk_visible(6, 0), torch.tril(torch.ones(6, 6, dtype=torch.bool)))
    assert torch.equal(pr.chunk_visible(5, 1), torch.eye(5, dtype=torch.bool))
    # rotation: a pair's scalar product depends on the distance alone; channel i turns with channel i + dims/2 by
    # p * base^(-2i/dims) / factor; the channels beyond `dims` pass unchanged
    torch.manual_seed(0)
    x, y = torch.randn(1, 1, 10, dtype=F64).expand(3, 1, 10), torch.randn(1, 1, 10, dtype=F64).expand(3, 1, 10)
    a, b = pr.rotate_half(x, torch.tensor([3, 10, 40]), 6, 50.0, 4.0), pr.rotate_half(y, torch.tensor([1, 8, 38]), 6, 50.0, 4.0)
    s = (a * b).sum(-1)
    assert torch.allclose(s, s[0].expand(3, 1), atol=1e-12) and torch.equal(a[..., 6:], x[..., 6:])
    p, i = 40, 1
    ang = p * 50.0 ** (-2.0 * i / 6) / 4.0
    assert torch.isclose(a[2, 0, i], x[2, 0, i] * math.cos(ang) - x[2, 0, i + 3] * math.sin(ang), atol=1e-12)
    assert torch.isclose(a[2, 0, i + 3], x[2, 0, i + 3] * math.cos(ang) + x[2, 0, i] * math.sin(ang), atol=1e-12)
    assert torch.equal(pr.rotate_half(x, torch.tensor([3, 10, 40]), 0, 50.0), x)


def test_plain_attention_norms_the_whole_projection():
    """The query norm divides by the root mean square of all heads' queries together: scaling one head's rows of Wq
    changes the other heads' queries too."""
    torch.manual_seed(1)
    T, W = 7, 10
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "scale": 0.5, "mask": {"size": 3}, "rot": {"dims": 2, "base": 20.0}}
    t = {"q": torch.randn(8, W), "q.b": torch.randn(8), "k": torch.randn(4, W), "k.b": torch.randn(4), "v": torch.randn(3, W),
         "v.b": torch.randn(3), "q.norm": torch.rand(8) + 0.5, "k.norm": torch.rand(4) + 0.5, "o": torch.randn(W, 6), "o.b": torch.randn(W)}
    h = torch.randn(T, W, dtype=F64)
    got = pr.chunked_attention(h, t, "", m, 1e-5)
    q = h @ t["q"].double().T + t["q.b"].double()
    k = h @ t["k"].double().T + t["k.b"].double()
    v = h @ t["v"].double().T + t["v.b"].double()
    q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + 1e-5) * t["q.norm"].double()
    k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + 1e-5) * t["k.norm"].double()
    pos = torch.arange(T)
    q = pr.rotate_half(q.view(T, 2, 4), pos, 2, 20.0)
    k = pr.rotate_half(k.view(T, 1, 4), pos, 2, 20.0)
    out = torch.zeros(T, 2, 3, dtype=F64)
    for i in range(T):
        js = list(range(i - i % 3, i + 1))
        for hd in range(2):
            p = torch.softmax(torch.stack([q[i, hd] @ k[j, 0] for j in js]) * 0.5, dim=0)
            out[i, hd] = sum(p[n] * v[j] for n, j in enumerate(js))
    assert torch.allclose(got, out.reshape(T, 6) @ t["o"].double().T + t["o.b"].double(), atol=1e-12)


def test_plain_scan_is_the_decayed_sum_and_the_convolution_looks_back():
    torch.manual_seed(2)
    T, Hh, P, N = 8, 2, 3, 4
    x, B, C = torch.randn(T, Hh, P, dtype=F64), torch.randn(T, Hh, N, dtype=F64), torch.randn(T, Hh, N, dtype=F64)
    dt, a, D = torch.rand(T, Hh, dtype=F64) + 0.1, -torch.rand(Hh, dtype=F64), torch.randn(Hh, dtype=F64)
    got = pr.selective_scan(x, B, C, dt, a, D)
    for i in range(T):
        for hd in range(Hh):
            y = D[hd] * x[i, hd]
            for j in range(i + 1):
                y = y + torch.exp(a[hd] * dt[j + 1:i + 1, hd].sum()) * dt[j, hd] * (C[i, hd] @ B[j, hd]) * x[j, hd]
            assert torch.allclose(got[i, hd], y, atol=1e-12)
    u, taps, bias = torch.randn(6, 3, dtype=F64), torch.randn(3, 4, dtype=F64), torch.randn(3, dtype=F64)
    y = pr.causal_conv(u, taps, bias)
    for i in range(6):
        want = bias + sum(taps[:, 3 - d] * u[i - d] for d in range(4) if i - d >= 0)
        assert torch.allclose(y[i], want, atol=1e-12)
    assert abs(float(pr.softplus(torch.tensor(50.0, dtype=F64))) - 50.0) < 1e-12
    assert abs(float(pr.softplus(torch.tensor(0.0, dtype=F64))) - math.log(2.0)) < 1e-12


def test_plain_state_space_gate_comes_before_the_norm_in_parts():
    torch.manual_seed(3)
    T, W = 5, 9
    m = {"heads": 4, "vdim": 2, "state": 3, "groups": 2, "conv": 2, "norm_groups": 2}
    inner, C = 8, 8 + 12
    t = {"in": torch.randn(inner + C + 4, W), "conv": torch.randn(C, 2), "conv.b": torch.randn(C), "dt_bias": torch.randn(4),
         "A_log": torch.randn(4), "D": torch.randn(4), "norm": torch.rand(inner) + 0.5, "o": torch.eye(inner)}
    h = torch.randn(T, W, dtype=F64)
    got = pr.state_space(h, t, "", m, 1e-5)
    p = h @ t["in"].double().T
    z = p[:, :inner]
    xbc = pr.silu(pr.causal_conv(p[:, inner:inner + C], t["conv"].double(), t["conv.b"].double()))
    dt = torch.log1p(torch.exp(p[:, inner + C:] + t["dt_bias"].double()))
    x = xbc[:, :inner].view(T, 4, 2)
    Bm, Cm = xbc[:, inner:inner + 6].view(T, 2, 3), xbc[:, inner + 6:].view(T, 2, 3)
    y = torch.zeros(T, 4, 2, dtype=F64)
    for hd in range(4):
        g = hd // 2                                    # heads 0, 1 read group 0; heads 2, 3 group 1
        S = torch.zeros(3, 2, dtype=F64)
        for i in range(T):
            S = torch.exp(-torch.exp(t["A_log"].double()[hd]) * dt[i, hd]) * S + dt[i, hd] * torch.outer(Bm[i, g], x[i, hd])
            y[i, hd] = S.T @ Cm[i, g] + t["D"].double()[hd] * x[i, hd]
    y = y.reshape(T, inner) * pr.silu(z)
    halves = [part / torch.sqrt((part * part).mean(-1, keepdim=True) + 1e-5) for part in (y[:, :4], y[:, 4:])]
    assert torch.allclose(got, torch.cat(halves, dim=-1) * t["norm"].double(), atol=1e-12)


def test_plain_router_weight_scales_the_experts_input():
    torch.manual_seed(4)
    W, E = 6, 4
    mlp = {"expert": {"ff": 5}, "router": {"experts": E, "top": 2}}
    t = {"router": torch.randn(E, W)}
    for e in range(E):
        t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"] = torch.randn(5, W), torch.randn(5, W), torch.randn(W, 5)
    h = torch.randn(7, W, dtype=F64)
    s = torch.sigmoid(h @ t["router"].double().T)
    got = pr.moe_ff(h, t, "", mlp)
    inside, outside = torch.zeros_like(h), torch.zeros_like(h)
    for r in range(7):
        for e in torch.topk(s[r], 2).indices.tolist():
            f = lambda v: (pr.silu(v @ t[f"e{e}.gate"].double().T) * (v @ t[f"e{e}.up"].double().T)) @ t[f"e{e}.down"].double().T
            inside[r] += f(s[r, e] * h[r])
            outside[r] += s[r, e] * f(h[r])
    assert torch.allclose(got, inside, atol=1e-12)
    assert (inside - outside).abs().max() > 0.05                    # weighting the result instead is another model
    assert (s.topk(2).values.sum(-1) - 1).abs().max() > 0.05         # the weights are not made to sum to one
    assert abs(float(pr.gelu_tanh(torch.tensor(1.0, dtype=F64))) - 0.8411919906082768) < 1e-12
    x = torch.tensor([0.3, -2.0], dtype=F64)
    assert torch.allclose(pr.dynamic_tanh(x, 0.7, torch.tensor(1.5), torch.tensor(0.2)), torch.tanh(0.7 * x) * 1.5 + 0.2)


# ---- the engine on the stand-ins against the plain implementation ---------------------------------------------------

@pytest.mark.parametrize("name", list(RM.CONFIGS))
def test_schedules_on_the_stand_in(name):
    cfg, w, w64 = model(name)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 40 + i) for i, n in enumerate([37, 1, 58, 23, 70])}
    eng = engine_for(cfg, w)
    for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=12), H.portions_trace(reqs, seed=3)):
        got = RM.run_trace(eng, steps)
        assert len(got) == sum(len(v) for v in reqs.values())
        worst = RM.worst_error(name, cfg, w64, reqs, got)
        assert worst[0] <= TOL32, worst
        assert eng.cache.n_live == 0
        eng.cache.check()
    # several requests at a time with pages for the live ones only: pages and state slots are used again
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, max_requests=3, max_tokens=peak, graphs=True)
    got = RM.run_trace(eng, steps)
    worst = RM.worst_error(name, cfg, w64, reqs, got)
    assert worst[0] <= TOL32, worst
    eng.cache.check()


def test_a_used_state_slot_starts_from_zero():
    cfg, w, w64 = model("D")
    eng = engine_for(cfg, w, max_requests=1)
    ids_a, ids_b = H.random_ids(cfg["vocab"], 30, 1), H.random_ids(cfg["vocab"], 9, 2)
    RM.run_trace(eng, H.whole_trace({"a": ids_a}))
    assert eng.cache.groups == {}                       # the state-space mixer alone keeps no pages
    assert any(t[0].abs().max() > 0 for t in eng.cache.states.values())     # the first request left its state in the only slot
    got = RM.run_trace(eng, H.portions_trace({"b": ids_b}, sizes=(2, 3)))
    assert RM.worst_error("D", cfg, w64, {"b": ids_b}, got)[0] <= TOL32


def needle_case(name, at, distance, chunk=None, seed=60):
    """A sequence in which the probe token, `distance` after the needle at `at`, looks for it in the first layer (whose
    chunk is set to `chunk` if given); and how far the probe's logits move when the needle is replaced."""
    cfg, w, _ = model(name)
    cfg = copy.deepcopy(cfg)
    if chunk is not None:
        cfg["layers"][0]["mixer"]["mask"] = {"size": chunk}
    needle, probe = 3, 7
    w = RM.sharpen(cfg, w, needle, probe)
    w64 = RM.as_f64(w)
    ids = [t if t not in (needle, probe) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, seed + at)]
    ids[at], ids[at + distance] = needle, probe
    without = list(ids)
    without[at] = 11
    key = (name, "sharp", chunk)
    want = RM.plain_logits(key, cfg, w64, ids)[at + distance]
    moved = RM.relative_error(pr.forward(cfg, w64, without)[at + distance], want)
    return key, cfg, w, w64, ids, moved


def run_three_ways(key, cfg, w, w64, ids, tail=6):
    eng = engine_for(cfg, w)
    for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=tail),
                  H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
        got = RM.run_trace(eng, steps)
        worst = RM.worst_error(key, cfg, w64, {"s": ids}, got)
        assert worst[0] <= TOL32, worst


@pytest.mark.parametrize("name,distance,chunk", [("A", 1, None), ("C", 300, 400), ("E", 250, None), ("D", 150, None)])
def test_a_token_that_stands_out(name, distance, chunk):
    """The probe looks for a needle right before it or hundreds of tokens back (through attention's pages or the
    recurrent state), with the needle on both sides of a page's border; whole, decoded alone and in portions."""
    for at in (15, 16):
        key, cfg, w, w64, ids, moved = needle_case(name, at, distance, chunk)
        assert moved >= 0.01, moved              # losing that one key would show
        run_three_ways(key, cfg, w, w64, ids)


@pytest.mark.parametrize("chunk", [21, 32])
def test_keys_just_inside_and_just_outside_a_chunk(chunk):
    """A chunk that ends inside a page and one that ends at a page's border. The needle is the first position of a
    chunk and the probe the last of the same chunk (the farthest key a row ever sees), then the probe is the first
    position of the next chunk (the needle has just gone out of sight), then the needle is the last position of a chunk
    and the probe right after it. Seen: the logits rest on the needle; not seen: replacing it changes nothing at all."""
    c0 = 2 * chunk
    for at, distance, seen in ((c0, chunk - 1, True), (c0, chunk, False), (c0 + chunk - 1, 1, False), (c0 + chunk - 2, 1, True)):
        key, cfg, w, w64, ids, moved = needle_case("A", at, distance, chunk)
        if seen:
            assert moved >= 0.01, (at, distance, moved)
        else:
            without = list(ids)
            without[at] = 11
            other = pr.forward(cfg, w64, without, streams=(s1 := []))
            pr.forward(cfg, w64, ids, streams=(s0 := []))
            assert torch.equal(s0[0][at + distance], s1[0][at + distance])      # the first layer's row does not see it
        run_three_ways(key, cfg, w, w64, ids, tail=chunk + 3)      # decoding passes the chunk's edge too


def test_the_first_tokens_and_one_token_alone():
    for name in ("A", "B", "D"):
        cfg, w, w64 = model(name, seed=7)
        eng = engine_for(cfg, w)
        reqs = {"one": H.random_ids(cfg["vocab"], 1, 1), "two": H.random_ids(cfg["vocab"], 2, 2), "five": H.random_ids(cfg["vocab"], 5, 3)}
        for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=4)):
            got = RM.run_trace(eng, steps)
            assert RM.worst_error((name, 7), cfg, w64, reqs, got)[0] <= TOL32


def test_long_decoding_of_unequal_requests():
    """Three requests of unequal lengths decode 90 tokens together, over page borders and many chunk edges, each
    against itself alone."""
    cfg, w, w64 = model("A", seed=6)
    reqs = {f"r{i}": H.random_ids(cfg["vocab"], n, 90 + i) for i, n in enumerate([100, 131, 93])}
    eng = engine_for(cfg, w, max_requests=3, graphs=True)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": ids[:len(ids) - 90], "want": [0]} for r, ids in reqs.items()], "end": []}]
    for t in range(90):
        steps.append({"step": t + 1, "entries": [{"id": r, "tokens": [ids[len(ids) - 90 + t]], "want": [0]} for r, ids in reqs.items()],
                      "end": list(reqs) if t == 89 else []})
    got = RM.run_trace(eng, steps)
    assert RM.worst_error(("A", 6), cfg, w64, reqs, got)[0] <= TOL32


def test_the_routers_weight_and_the_gates_place_show_in_the_logits():
    """Weighting an expert's result instead of its input, or gating after the norm instead of before, moves the plain
    logits by far more than the engine's tolerance: the schedules above would catch either."""
    cfg, w, w64 = model("A")
    ids = H.random_ids(cfg["vocab"], 40, 9)
    want = RM.plain_logits("A", cfg, w64, ids)
    keep = pr.moe_ff, pr.state_space
    try:
        def outside(h, t, pre, mlp, choose=None, margins=None):
            idx, wt = pr.route(h, t, pre, mlp["router"]["top"])
            y = torch.zeros_like(h)
            for r in range(h.shape[0]):
                for e, we in zip(idx[r].tolist(), wt[r]):
                    y[r] += we * pr.expert_ff(h[r].unsqueeze(0), t, f"{pre}e{e}.")[0]
            return y
        pr.moe_ff = outside
        assert RM.relative_error(pr.forward(cfg, w64, ids)[20], want[20]) > 100 * TOL32
    finally:
        pr.moe_ff, pr.state_space = keep
    capless = copy.deepcopy(cfg)
    del capless["logit_softcap"]
    assert RM.relative_error(pr.forward(capless, w64, ids)[20], want[20]) > 100 * TOL32


def test_greedy_generation_through_the_scheduler():
    for name in ("A", "B"):
        cfg, w, w64 = model(name, seed=8)
        prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6))]
        want = [pr.greedy_generate(cfg, w64, p, 7) for p in prompts]
        eng = engine_for(cfg, w, max_requests=2, max_tokens=160, graphs=True)
        out, s = generate(eng, prompts, max_new_tokens=7, temperature=0.0, max_batch=2, token_budget=11,
                          return_scheduler=True)
        assert out == want
        assert s.peak_running == 2 and eng.cache.n_live == 0
        eng.cache.check()


def test_the_named_size_runs_with_random_weights(tmp_path):
    from tiny_inference_server_amd.__main__ import preset_names, size_config
    from tiny_inference_server_amd.weights import write_random_model
    assert "rurorax-small" in preset_names()
    cfg = size_config("rurorax-small")
    folder = write_random_model(cfg, 3, str(tmp_path / "m"))
    assert load_config(folder).to_dict() == cfg.to_dict()
    eng = Engine(folder, dtype="float32", max_tokens=64, max_requests=2, ops=TorchOps())
    out = eng.step([("a", [5, 9, 1, 300], [3]), ("b", [7], [0])]).logits
    assert out.shape == (2, cfg.vocab) and torch.isfinite(out).all()
    assert out.abs().max() <= cfg.logit_softcap
