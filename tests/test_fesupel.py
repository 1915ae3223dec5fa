"""The Fesupel architecture on the host: its configuration and spec, the plain implementation's mechanisms against
closed forms, and the engine (step function, cache manager, scheduler, generate) on the torch stand-ins for the kernels
against the plain implementation, in 32-bit."""
import copy
import math

import pytest
import torch

import fesupel_models as FM
import helpers as H
import plain_fesupel as pf
from torch_ops import TorchOps
from tiny_inference_server_amd.config import ARCHITECTURES, ConfigError, config_from_dict, load_config
from tiny_inference_server_amd.engine import Engine
from tiny_inference_server_amd.engine.generate import generate
from tiny_inference_server_amd.parts.attention import banded_frequencies
from tiny_inference_server_amd.weights.loader import spec_tensors

TOL32 = 3e-5
# the configuration of ones divides single numbers by their own size (a token input of one number, unit vectors of one
# channel): where such a number is small, 32-bit rounding is a larger share of it
TOL_OF = {"D": 3e-4}
F64 = torch.float64


def model(name, seed=5):
    cfg = FM.CONFIGS[name]
    w = FM.random_weights(cfg, seed)
    return cfg, w, FM.as_f64(w)


def engine_for(cfg, w, **kw):
    kw.setdefault("max_requests", 4)
    kw.setdefault("page_size", 8)
    kw.setdefault("max_tokens", 640)
    return Engine(config=config_from_dict(cfg), tensors={n: t.float() for n, t in w.items()}, dtype="float32",
                  ops=TorchOps(graphs=kw.pop("graphs", False)), **kw)


# ---- configuration and spec ------------------------------------------------------------------------------------

def test_spec_names_every_tensor(tmp_path):
    for name, cfg in FM.CONFIGS.items():
        w = FM.random_weights(cfg, 1)
        bare = copy.deepcopy(cfg)
        for e in bare["layers"]:                   # the two ranks are in no key: the weight file's shapes give them
            del e["mixer"]["right"]["decay_rank"], e["mixer"]["right"]["gate_rank"]
        folder = FM.write_folder(str(tmp_path / name), bare, w)
        c = load_config(folder)
        assert c.architecture == "Fesupel" and c.to_dict() == config_from_dict(c.to_dict()).to_dict()
        assert [e["mixer"]["right"]["decay_rank"] for e in c.layers] == [e["mixer"]["right"]["decay_rank"] for e in cfg["layers"]]
        spec = ARCHITECTURES.get(c.architecture).build_spec(c)
        assert spec_tensors(spec) == {n: tuple(t.shape) for n, t in w.items()}
        assert len(spec.stages[0].calls) == len(spec.layers) == len(cfg["layers"])
        for layer, entry in zip(spec.layers, cfg["layers"]):
            assert ("feed_forward" in layer.parts) == (entry["mlp"] is not None) == ("feed_forward_post_norm" in layer.parts)
            assert ("token_input" in layer.parts) == ("token_side" in cfg)
            assert [n for n, _ in layer.mixers()] == ["left", "right"]


def test_configuration_errors_name_the_key():
    good = FM.CONFIGS["A"]
    for path, value, word in [(("layers", 0, "type"), "attention", "type"), (("layers", 0, "mixer", "left", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mixer", "left", "rot", "dims"), 3, "rot.dims"),
                              (("layers", 0, "mixer", "left", "rot", "scaling", "low"), 0.0, "scaling"),
                              (("layers", 0, "mixer", "left", "mask", "size"), 0, "size"),
                              (("layers", 0, "mixer", "right", "kv_heads"), 3, "kv_heads"), (("layers", 0, "mixer", "right", "conv"), 0, "conv"),
                              (("layers", 1, "mlp", "router", "top"), 9, "top"), (("layers", 1, "mlp", "router", "groups", "count"), 3, "groups"),
                              (("layers", 1, "mlp", "expert", "limit"), 0.0, "limit"), (("layers", 0, "mlp", "kind"), "gated", "mlp"),
                              (("norm",), {}, "eps")]:
        bad = copy.deepcopy(good)
        d = bad
        for k in path[:-1]:
            d = d[k]
        d[path[-1]] = value
        with pytest.raises(ConfigError, match=word):
            config_from_dict(bad)


# ---- the plain implementation's mechanisms against closed forms ----------------------------------------------------

def test_plain_chunks_and_slowed_waves():
    vis = pf.chunk_mask(11, 4)
    for i in range(11):
        assert vis[i].nonzero().flatten().tolist() == list(range(i - i % 4, i + 1))
    assert torch.equal(pf.chunk_mask(6, 0), torch.tril(torch.ones(6, 6, dtype=torch.bool)))
    assert torch.equal(pf.chunk_mask(5, 1), torch.eye(5, dtype=torch.bool))
    # waves shorter than original / high are kept, longer than original / low slowed by the factor, between blended
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    f0, f = pf.rotary_frequencies(16, 1000.0), pf.rotary_frequencies(16, 1000.0, sc)
    wave = 2 * math.pi / f0
    assert (wave < 16).any() and (wave > 64).any() and ((wave >= 16) & (wave <= 64)).any()      # all three kinds are there
    for i in range(8):
        if wave[i] < 16:
            assert f[i] == f0[i]
        elif wave[i] > 64:
            assert torch.isclose(f[i], f0[i] / 4.0, rtol=1e-14)
        else:
            s = (64 / wave[i] - 1.0) / 3.0
            assert torch.isclose(f[i], (1 - s) * f0[i] / 4.0 + s * f0[i], rtol=1e-14) and f0[i] / 4 < f[i] < f0[i]
    # the engine's table of frequencies is the same function written another way
    assert torch.allclose(banded_frequencies(16, 1000.0, (4.0, 1.0, 4.0, 64)), f, rtol=1e-13)
    assert torch.allclose(banded_frequencies(6, 50.0), pf.rotary_frequencies(6, 50.0), rtol=1e-14)
    # rotation: a pair's scalar product depends on the distance alone; channel i turns with channel i + dims/2
    torch.manual_seed(0)
    x, y = torch.randn(1, 1, 10, dtype=F64).expand(3, 1, 10), torch.randn(1, 1, 10, dtype=F64).expand(3, 1, 10)
    fr = pf.rotary_frequencies(6, 50.0)
    a, b = pf.rotate_half(x, torch.tensor([3, 10, 40]), 6, fr), pf.rotate_half(y, torch.tensor([1, 8, 38]), 6, fr)
    s = (a * b).sum(-1)
    assert torch.allclose(s, s[0].expand(3, 1), atol=1e-12) and torch.equal(a[..., 6:], x[..., 6:])
    ang = 40 * 50.0 ** (-2.0 / 6)
    assert torch.isclose(a[2, 0, 1], x[2, 0, 1] * math.cos(ang) - x[2, 0, 4] * math.sin(ang), atol=1e-12)
    assert torch.isclose(a[2, 0, 4], x[2, 0, 4] * math.cos(ang) + x[2, 0, 1] * math.sin(ang), atol=1e-12)


def test_plain_attention_key_by_key():
    """Sigmoid weights, each key on its own, mixed across the heads before the values; head h reads its own key/value
    head's values whatever heads its weights were mixed from."""
    torch.manual_seed(1)
    T, W = 7, 10
    m = {"heads": 4, "kv_heads": 2, "dim": 4, "vdim": 3, "scale": 0.5, "softcap": 2.0, "mask": {"size": 3},
         "rot": {"dims": 2, "base": 20.0}}
    t = {"q": torch.randn(16, W), "q.b": torch.randn(16), "k": torch.randn(8, W), "k.b": torch.randn(8), "v": torch.randn(6, W),
         "v.b": torch.randn(6), "pb": torch.randn(4), "talk": torch.randn(4, 4), "o": torch.randn(W, 12)}
    t = {k: v.double() for k, v in t.items()}
    h = torch.randn(T, W, dtype=F64)
    got = pf.left_mixer(h, t, "", m, torch.arange(T))
    fr = pf.rotary_frequencies(2, 20.0)
    q = pf.rotate_half((h @ t["q"].T + t["q.b"]).view(T, 4, 4), torch.arange(T), 2, fr)
    k = pf.rotate_half((h @ t["k"].T + t["k.b"]).view(T, 2, 4), torch.arange(T), 2, fr)
    v = (h @ t["v"].T + t["v.b"]).view(T, 2, 3)
    out = torch.zeros(T, 4, 3, dtype=F64)
    for i in range(T):
        for j in range(i - i % 3, i + 1):
            wg = torch.stack([torch.sigmoid(2.0 * torch.tanh(q[i, g] @ k[j, g // 2] * 0.5 / 2.0) + t["pb"][g]) for g in range(4)])
            for hd in range(4):
                out[i, hd] += (t["talk"][hd] @ wg) * v[j, hd // 2]
    assert torch.allclose(got, out.reshape(T, 12) @ t["o"].T, atol=1e-12)
    # weights are not normalised: a row that sees more keys gathers more
    w = pf.sigmoid_weights(q, k, 0.5, 2.0, t["pb"], pf.chunk_mask(T, 0))
    assert (w.sum(-1)[:, -1] > w.sum(-1)[:, 0]).all()


def test_plain_delta_rule_writes_reads_and_forgets():
    torch.manual_seed(2)
    T, Hh, D, V = 6, 2, 4, 3
    q, v = torch.randn(T, Hh, D, dtype=F64), torch.randn(T, Hh, V, dtype=F64)
    k = pf.unit(torch.randn(T, Hh, D, dtype=F64))
    beta, decay = torch.rand(T, Hh, dtype=F64), torch.rand(T, Hh, D, dtype=F64)
    got = pf.delta_rule(q, k, v, beta, decay)
    S = torch.zeros(Hh, D, V, dtype=F64)
    for i in range(T):
        for hd in range(Hh):
            S[hd] = decay[i, hd].view(D, 1) * S[hd]
            before = S[hd].T @ k[i, hd]
            S[hd] = S[hd] + torch.outer(k[i, hd], beta[i, hd] * (v[i, hd] - before))
            # what the key now reads lies between what it read before and the new value (k is a unit vector up to 1e-6)
            assert torch.allclose(S[hd].T @ k[i, hd], before + beta[i, hd] * (v[i, hd] - before), atol=1e-5)
            assert torch.allclose(got[i, hd], S[hd].T @ q[i, hd], atol=1e-12)      # the row reads its own write
    # the convolution looks back taps - 1 rows and sees nothing before the first
    u, taps = torch.randn(6, 3, dtype=F64), torch.randn(3, 4, dtype=F64)
    y = pf.causal_conv(u, taps)
    for i in range(6):
        want = sum(taps[:, 3 - d] * u[i - d] for d in range(4) if i - d >= 0)
        assert torch.allclose(y[i], want, atol=1e-12)
    assert torch.allclose(pf.causal_conv(u, taps[:, 3:]), u * taps[:, 3])
    assert abs(float(pf.softplus(torch.tensor(50.0, dtype=F64))) - 50.0) < 1e-12
    assert abs(float(pf.softplus(torch.tensor(0.0, dtype=F64))) - math.log(2.0)) < 1e-12


def test_plain_choice_in_groups_and_the_corrections_role():
    s = torch.tensor([[0.05, 0.30, 0.10, 0.05, 0.20, 0.22, 0.04, 0.04]], dtype=F64)
    zero = torch.zeros(8, dtype=F64)
    ids, w, _ = pf.choose(s, zero, 2, 1, 1)
    assert ids.tolist() == [[1, 5]] and torch.allclose(w, torch.tensor([[0.30, 0.22]], dtype=F64) / 0.52)
    # four groups of two, one kept: the group of the largest score, and the second choice comes from it too
    ids, w, _ = pf.choose(s, zero, 2, 4, 1)
    assert ids.tolist() == [[1, 0]] and torch.allclose(w.sum(), torch.tensor(1.0, dtype=F64))
    # two groups kept: the groups of 0.30 and 0.22
    assert pf.choose(s, zero, 3, 4, 2)[0].tolist() == [[1, 5, 4]]
    # the correction moves the choice (of groups and of experts) but not the weights
    c = torch.tensor([0, 0, 0, 0, 0, 0, 0.5, 0], dtype=F64)
    ids, w, _ = pf.choose(s, c, 2, 4, 1)
    assert ids.tolist() == [[6, 7]] and torch.allclose(w, torch.tensor([[0.5, 0.5]], dtype=F64))
    # corrected scores may be negative: a group that is out counts as minus infinity, not as zero
    ids, _, _ = pf.choose(s, torch.full((8,), -1.0, dtype=F64), 2, 4, 1)
    assert ids.tolist() == [[1, 0]]


def test_plain_experts_identity_shared_and_clamps():
    torch.manual_seed(4)
    W = 6
    mlp = {"expert": {"ff": 5, "limit": 0.7}, "router": {"experts": 2, "identity": 2, "top": 2}, "shared": {"ff": 3, "limit": 0.4}}
    t = {"router": torch.randn(4, W) * 2, "correction": torch.zeros(4), "shared.gate": torch.randn(3, W), "shared.up": torch.randn(3, W),
         "shared.down": torch.randn(W, 3), "shared.sg": torch.randn(1, W)}
    for e in range(2):
        t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"] = torch.randn(5, W), torch.randn(5, W), torch.randn(W, 5)
    t = {k: v.double() for k, v in t.items()}
    h = torch.randn(9, W, dtype=F64)

    def expert(x, pre, limit):
        g = torch.minimum(x @ t[pre + "gate"].T, torch.tensor(limit, dtype=F64))
        u = torch.clamp(x @ t[pre + "up"].T, -limit, limit)
        return (g / (1 + torch.exp(-1.702 * g)) * (u + 1)) @ t[pre + "down"].T

    s = torch.softmax(h @ t["router"].T, -1)
    want = torch.zeros_like(h)
    for r in range(9):
        top = torch.topk(s[r], 2)
        for e, sc in zip(top.indices.tolist(), top.values):
            want[r] += sc / top.values.sum() * (expert(h[r], f"e{e}.", 0.7) if e < 2 else h[r])
    want = want + expert(h, "shared.", 0.4) * torch.sigmoid(h @ t["shared.sg"].T)
    assert torch.allclose(pf.moe_ff(h, t, "", mlp), want, atol=1e-12)
    assert (torch.topk(s, 2).indices >= 2).any() and (torch.topk(s, 2).indices < 2).any()      # both kinds were chosen
    assert ((h @ t["e0.gate"].T) > 0.7).any() and ((h @ t["e0.up"].T) < -0.7).any()                # and the clamps bit
    x = torch.tensor([[-1.0, 0.5, 2.0]], dtype=F64)
    assert torch.allclose(pf.dense_ff(x, {"up": torch.eye(3, dtype=F64), "down": torch.eye(3, dtype=F64)}, ""),
                          torch.tensor([[0.0, 0.25, 4.0]], dtype=F64))
    assert abs(float(pf.gelu_tanh(torch.tensor(1.0, dtype=F64))) - 0.8411919906082768) < 1e-12


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
        assert worst[0] <= TOL_OF.get(name, TOL32), worst
        assert eng.cache.n_live == 0
        eng.cache.check()
    # several requests at a time with pages for the live ones only: pages and state slots are used again
    steps, peak = H.mixed_trace(reqs, max_live=3, seed=4)
    eng = engine_for(cfg, w, max_requests=3, max_tokens=peak, graphs=True)
    got = FM.run_trace(eng, steps)
    worst = FM.worst_error(name, cfg, w64, reqs, got)
    assert worst[0] <= TOL_OF.get(name, TOL32), worst
    eng.cache.check()


def test_a_used_state_slot_starts_from_zero():
    cfg, w, w64 = model("B")
    eng = engine_for(cfg, w, max_requests=1)
    ids_a, ids_b = H.random_ids(cfg["vocab"], 30, 1), H.random_ids(cfg["vocab"], 9, 2)
    FM.run_trace(eng, H.whole_trace({"a": ids_a}))
    assert any(t[0].abs().max() > 0 for t in eng.cache.states.values())     # the first request left its state in the only slot
    got = FM.run_trace(eng, H.portions_trace({"b": ids_b}, sizes=(2, 3)))
    assert FM.worst_error("B", cfg, w64, {"b": ids_b}, got)[0] <= TOL32


def needle_case(name, at, distance, side="left", chunk=None, seed=60):
    """A sequence in which the probe token, `distance` after the needle at `at`, looks for it in the first layer (whose
    chunk is set to `chunk` if given); and how far the probe's logits move when the needle is replaced."""
    cfg, w, _ = model(name)
    cfg = copy.deepcopy(cfg)
    if chunk is not None:
        cfg["layers"][0]["mixer"]["left"]["mask"] = {"size": chunk}
    needle, probe = 3, 7
    w = FM.sharpen(cfg, w, needle, probe, side)
    w64 = FM.as_f64(w)
    ids = [t if t not in (needle, probe) else 11 for t in H.random_ids(cfg["vocab"], at + distance + 4, seed + at)]
    ids[at], ids[at + distance] = needle, probe
    without = list(ids)
    without[at] = 11
    key = (name, "sharp", side, chunk)
    want = FM.plain_logits(key, cfg, w64, ids)[at + distance]
    moved = FM.relative_error(pf.forward(cfg, w64, without)[at + distance], want)
    return key, cfg, w, w64, ids, moved


def run_three_ways(key, cfg, w, w64, ids, tail=6):
    eng = engine_for(cfg, w)
    for steps in (H.whole_trace({"s": ids}), H.tail_decode_trace({"s": ids}, tail=tail),
                  H.portions_trace({"s": ids}, sizes=(5, 2, 11))):
        got = FM.run_trace(eng, steps)
        worst = FM.worst_error(key, cfg, w64, {"s": ids}, got)
        assert worst[0] <= TOL32, worst


@pytest.mark.parametrize("name,distance,side,chunk", [("A", 1, "left", None), ("C", 300, "left", 400), ("C", 150, "right", None),
                                                      ("B", 60, "right", None)])
def test_a_token_that_stands_out(name, distance, side, chunk):
    """The probe looks for a needle right before it or hundreds of tokens back (through attention's pages or the
    delta rule's state), with the needle on both sides of a page's border; whole, decoded alone and in portions."""
    for at in (15, 16):
        key, cfg, w, w64, ids, moved = needle_case(name, at, distance, side, chunk)
        assert moved >= 0.01, moved              # losing that one key would show
        run_three_ways(key, cfg, w, w64, ids)


@pytest.mark.parametrize("chunk", [21, 32])
def test_keys_just_inside_and_just_outside_a_chunk(chunk):
    """A chunk that ends inside a page and one that ends at a page's border. The needle is the first position of a
    chunk and the probe the last of the same chunk (the farthest key a row ever sees), then the probe is the first
    position of the next chunk (the needle has just gone out of sight), then the needle is the last position of a chunk
    and the probe right after it. Seen: the logits rest on the needle; not seen: the left mixer's row does not change."""
    c0 = 2 * chunk
    for at, distance, seen in ((c0, chunk - 1, True), (c0, chunk, False), (c0 + chunk - 1, 1, False), (c0 + chunk - 2, 1, True)):
        key, cfg, w, w64, ids, moved = needle_case("A", at, distance, "left", chunk)
        if seen:
            assert moved >= 0.01, (at, distance, moved)
        else:
            without = list(ids)
            without[at] = 11
            rows = []
            for seq in (ids, without):
                x = w64["embed"][torch.tensor(seq)] * cfg["embedding"]["scale"]
                h = pf.rms_norm(x, w64["l0.norm1"], cfg["norm"]["eps"])
                rows.append(pf.left_mixer(h, w64, "l0.mix.left.", cfg["layers"][0]["mixer"]["left"], torch.arange(len(seq)))[at + distance])
            assert torch.equal(rows[0], rows[1])
        run_three_ways(key, cfg, w, w64, ids, tail=chunk + 3)      # decoding passes the chunk's edge too


def test_the_first_tokens_and_one_token_alone():
    for name in ("A", "B", "D"):
        cfg, w, w64 = model(name, seed=7)
        eng = engine_for(cfg, w)
        reqs = {"one": H.random_ids(cfg["vocab"], 1, 1), "two": H.random_ids(cfg["vocab"], 2, 2), "five": H.random_ids(cfg["vocab"], 5, 3)}
        for steps in (H.whole_trace(reqs), H.tail_decode_trace(reqs, tail=4)):
            got = FM.run_trace(eng, steps)
            assert FM.worst_error((name, 7), cfg, w64, reqs, got)[0] <= TOL_OF.get(name, TOL32)


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
    got = FM.run_trace(eng, steps)
    assert FM.worst_error(("A", 6), cfg, w64, reqs, got)[0] <= TOL32


def test_what_the_design_fixes_shows_in_the_logits():
    """Dropping the head mixture, normalising the weights over the keys, reading before the write in the delta rule, or
    counting a group that is out as zero instead of minus infinity moves the plain logits by far more than the engine's
    tolerance: the schedules above would catch any of them."""
    cfg, w, w64 = model("A")
    ids = H.random_ids(cfg["vocab"], 40, 9)
    want = FM.plain_logits("A", cfg, w64, ids)
    keep = pf.mix_heads, pf.sigmoid_weights, pf.delta_rule
    try:
        pf.mix_heads = lambda weights, talk: weights
        assert FM.relative_error(pf.forward(cfg, w64, ids)[20], want[20]) > 100 * TOL32
        pf.mix_heads = keep[0]
        pf.sigmoid_weights = lambda *a: (lambda p: p / p.sum(-1, keepdim=True))(keep[1](*a))
        assert FM.relative_error(pf.forward(cfg, w64, ids)[20], want[20]) > 100 * TOL32
        pf.sigmoid_weights = keep[1]

        def read_first(q, k, v, beta, decay):
            out = keep[2](q, k, v, beta, decay)
            return torch.cat((torch.zeros_like(out[:1]), out[:-1]))
        pf.delta_rule = read_first
        assert FM.relative_error(pf.forward(cfg, w64, ids)[20], want[20]) > 100 * TOL32
    finally:
        pf.mix_heads, pf.sigmoid_weights, pf.delta_rule = keep


def test_greedy_generation_through_the_scheduler():
    for name in ("A", "B"):
        cfg, w, w64 = model(name, seed=8)
        prompts = [H.random_ids(cfg["vocab"], n, 80 + i) for i, n in enumerate((13, 1, 30, 6))]
        want = [pf.greedy_generate(cfg, w64, p, 7) for p in prompts]
        eng = engine_for(cfg, w, max_requests=2, max_tokens=160, graphs=True)
        out, s = generate(eng, prompts, max_new_tokens=7, temperature=0.0, max_batch=2, token_budget=11,
                          return_scheduler=True)
        assert out == want
        assert s.peak_running == 2 and eng.cache.n_live == 0
        eng.cache.check()


def test_the_named_size_runs_with_random_weights(tmp_path):
    from tiny_inference_server_amd.__main__ import preset_names, size_config
    from tiny_inference_server_amd.weights import write_random_model
    assert "fesupel-small" in preset_names()
    cfg = size_config("fesupel-small")
    folder = write_random_model(cfg, 3, str(tmp_path / "m"))
    assert load_config(folder).to_dict() == cfg.to_dict()
    eng = Engine(folder, dtype="float32", max_tokens=64, max_requests=2, ops=TorchOps())
    out = eng.step([("a", [5, 9, 1, 300], [3]), ("b", [7], [0])]).logits
    assert out.shape == (2, cfg.vocab) and torch.isfinite(out).all()
