"""Small Rurorax configurations with random weights for the tests, and what the tests need around them.

The configurations differ in everything a layer has: the order and kinds of mixers, head counts, key/value heads (one,
some, as many as query heads), key and value sizes (equal and different), chunks from one position to longer than any
test sequence and none at all, rotated channels (all, some, none) with and without scaled frequencies, state sizes,
groups (one, some, as many as heads), convolution taps from 1 (no inputs kept) to 4, norm parts, dense and routed
feed-forwards with top from 1 to all experts, a layer without a feed-forward, a model without a cap on its logits, a
width that is no multiple of 8, and sizes of one wherever a size may be one.

Routing and bfloat16: an expert is chosen by comparing scores, and a bfloat16 engine may turn a close comparison the
other way; the plain implementation would then describe another model. So the engine's bfloat16 tests run the
configurations with every expert chosen (`all_chosen`): the weights still follow the router and still scale each
expert's input, no comparison decides anything. Routing itself is tested in 32-bit through the engine and kernel by
kernel in both types.
"""
from __future__ import annotations

import copy
import math
from typing import Dict, List

import torch

import plain_rurorax as pr
from fikevik_models import as_f64, relative_error, run_trace, write_folder  # noqa: F401  (the tests use them from here)


def attention(H, G, D, V, scale, chunk=None, dims=0, base=10000.0, factor=None):
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if dims is not None:
        m["rot"] = {"dims": dims, "base": base}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention", "mixer": m}


def ssm(H, P, N, G, taps, parts=None):
    m = {"heads": H, "vdim": P, "state": N, "groups": G, "conv": taps}
    if parts is not None:
        m["norm_groups"] = parts
    return {"type": "mamba2", "mixer": m}


def dense(entry, ff):
    e = copy.deepcopy(entry)
    e["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return e


def moe(entry, ff, experts, top):
    e = copy.deepcopy(entry)
    e["mlp"] = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    return e


def config(width, vocab, layers, cap=None, eps=1e-5):
    c = {"architecture": "Rurorax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if cap:
        c["logit_softcap"] = cap
    return c


def _configs():
    A = config(64, 211, [dense(attention(4, 2, 16, 24, 0.2, chunk=24, dims=8, factor=2.0), 40),
                         moe(ssm(4, 8, 12, 2, 4, parts=2), 24, 6, 2),
                         dense(attention(2, 2, 32, 32, 0.15, chunk=7), 0),
                         dense(ssm(3, 16, 8, 1, 2), 56)], cap=9.0)
    # a width that is no multiple of 8, no cap, chunks of one position (a row sees itself alone), every channel rotated
    # with unscaled frequencies, two heads a group, all experts chosen, a norm in three parts
    B = config(44, 97, [moe(ssm(6, 4, 5, 3, 3, parts=3), 20, 3, 3),
                        dense(attention(6, 1, 8, 8, 0.3, chunk=1, dims=8, base=50.0), 28),
                        moe(attention(3, 3, 12, 4, 0.25, chunk=33, dims=4, base=300.0, factor=1.5), 12, 5, 1)], eps=1e-6)
    # heads as wide as a served model's, keys and values of one size (the pages every attention kernel reads); prompts
    # of the tests are long enough for the scan to run in segments and for tiles of rows to cross chunks
    C = config(128, 300, [moe(attention(4, 1, 64, 64, 0.125, chunk=100, dims=32, base=1e5, factor=4.0), 64, 8, 2),
                          dense(ssm(4, 64, 64, 2, 4, parts=2), 96),
                          moe(attention(2, 2, 128, 128, 0.09, chunk=64, dims=64, base=1e6), 48, 4, 1),
                          moe(ssm(2, 32, 128, 1, 3, parts=1), 64, 8, 2)], cap=20.0)
    # the state-space mixer alone (no pages at all): one tap (nothing of the convolution to keep), as many groups as heads
    D = config(48, 77, [dense(ssm(2, 12, 16, 1, 4), 32), dense(ssm(4, 6, 4, 4, 1, parts=4), 0), moe(ssm(1, 20, 7, 1, 2), 16, 2, 1)],
               cap=5.0)
    # attention alone: no mask at all (with keys and values of different sizes and of one size), a chunk longer than any
    # sequence, keys wider and narrower than values, no rotation entry at all in one layer
    E = config(56, 150, [moe(attention(3, 3, 20, 36, 0.22, dims=None), 24, 7, 3),
                         dense(attention(2, 1, 40, 16, 0.16, chunk=4096, dims=10, base=1e4, factor=8.0), 48),
                         dense(attention(4, 2, 16, 16, 0.3, dims=2), 0)])
    # ones wherever a size may be one: a single head, one key/value head, one group, a state of one number per value
    # channel, values of one channel, one expert, one norm part per channel, chunks longer than a page and a single tap
    F = config(24, 61, [moe(ssm(1, 8, 1, 1, 2), 8, 1, 1), dense(attention(1, 1, 8, 8, 0.4, chunk=19, dims=8, base=100.0), 16),
                        dense(ssm(3, 1, 6, 1, 1, parts=3), 0), moe(attention(2, 1, 6, 1, 0.5, chunk=2), 4, 2, 1)], cap=3.0)
    return {"A": A, "B": B, "C": C, "D": D, "E": E, "F": F}


CONFIGS = _configs()


def tensor_shapes(cfg) -> Dict[str, tuple]:
    w = cfg["width"]
    out = {"embed": (cfg["vocab"], w), "final.norm": (w,), "final.norm.b": (w,), "final.norm.alpha": ()}
    for i, e in enumerate(cfg["layers"]):
        p, q, m = f"l{i}.", f"l{i}.mix.", e["mixer"]
        out.update({p + "norm1": (w,), p + "norm1.b": (w,), p + "norm1.alpha": (), p + "ls1": (w,)})
        if e["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({q + "q": (H * D, w), q + "q.b": (H * D,), q + "k": (G * D, w), q + "k.b": (G * D,), q + "v": (G * V, w),
                        q + "v.b": (G * V,), q + "q.norm": (H * D,), q + "k.norm": (G * D,), q + "o": (w, H * V), q + "o.b": (w,)})
        else:
            H, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            inner, C = H * P, H * P + 2 * G * N
            out.update({q + "in": (inner + C + H, w), q + "conv": (C, K), q + "conv.b": (C,), q + "dt_bias": (H,),
                        q + "A_log": (H,), q + "D": (H,), q + "norm": (inner,), q + "o": (w, inner)})
        mlp = e.get("mlp")
        if mlp is None:
            continue
        out[p + "ls2"] = (w,)
        f = p + "mlp."
        if mlp["kind"] == "dense":
            out.update({f + "gate": (mlp["ff"], w), f + "gate.b": (mlp["ff"],), f + "up": (mlp["ff"], w), f + "up.b": (mlp["ff"],),
                        f + "down": (w, mlp["ff"]), f + "down.b": (w,)})
        else:
            out[f + "router"] = (mlp["router"]["experts"], w)
            for k in range(mlp["router"]["experts"]):
                out.update({f"{f}e{k}.gate": (mlp["expert"]["ff"], w), f"{f}e{k}.up": (mlp["expert"]["ff"], w),
                            f"{f}e{k}.down": (w, mlp["expert"]["ff"])})
    return out


def random_weights(cfg, seed, storage=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/in); the table N(0, 1); gains and factors 1 +- 0.1; a norm's alpha around 0.7 (tanh bends but does
    not saturate); biases that differ from zero; a router strong enough for its scores to differ; step-size biases and
    decay rates that spread the heads' memories from a few tokens to hundreds."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        if name == "embed":
            t = torch.randn(shape, generator=g)
        elif name.endswith("alpha"):
            t = 0.5 + 0.4 * torch.rand(shape, generator=g)
        elif name.endswith("router"):
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith("mix.conv"):
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith("dt_bias"):
            t = -2.5 + 2.0 * torch.rand(shape, generator=g)
        elif name.endswith("A_log"):
            t = -2.0 + 2.5 * torch.rand(shape, generator=g)
        elif name.endswith(".D"):
            t = torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith(".b"):
            t = 0.3 * torch.randn(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(storage)
    return out


# ---- the plain implementation, kept per sequence ------------------------------------------------------------------

_plain: Dict[tuple, tuple] = {}


def plain(key, cfg, w64, ids):
    """(logits [T, vocab], the smallest routing margin of the sequence) from the plain implementation."""
    k = (key, tuple(ids))
    if k not in _plain:
        margins: List[float] = []
        _plain[k] = (pr.forward(cfg, w64, list(ids), margins=margins), min(margins, default=math.inf))
    return _plain[k]


def plain_logits(key, cfg, w64, ids):
    return plain(key, cfg, w64, ids)[0]


def routing_margin(key, cfg, w64, ids) -> float:
    return plain(key, cfg, w64, ids)[1]


def errors(key, cfg, w64, reqs: Dict[str, List[int]], got) -> list:
    """Sorted (error, place) over all places that came back: the difference of the logits with its mean taken off, root
    mean square over the vocabulary, over the spread of the plain logits of that request."""
    errs = []
    for rid, ids in reqs.items():
        want = plain_logits(key, cfg, w64, ids)
        scale = float(want.std())
        for p in range(len(ids)):
            if (rid, p) in got:
                d = got[(rid, p)].double() - want[p]
                e = float((d - d.mean()).pow(2).mean().sqrt()) / scale
                errs.append((e if e == e else math.inf, (rid, p)))
    return sorted(errs)


def worst_error(key, cfg, w64, reqs, got) -> tuple:
    return errors(key, cfg, w64, reqs, got)[-1]


TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def check(key, cfg, w64, reqs, got, dtype):
    """32-bit: every place within 3e-5 of the plain logits' spread. bfloat16: 98 of 100 places within 4 %, none beyond
    15 %."""
    errs = errors(key, cfg, w64, reqs, got)
    if dtype == "float32":
        assert errs[-1][0] <= TOL[dtype], errs[-1]
    else:
        assert errs[int(0.98 * (len(errs) - 1))][0] <= TOL[dtype], errs[int(0.98 * (len(errs) - 1))]
        assert errs[-1][0] <= 0.15, errs[-1]


# ---- weights that make one key stand out ----------------------------------------------------------------------------

def sharpen(cfg, tensors, needle: int, probe: int, strength: float = 8.0):
    """Make the token `probe` look for the token `needle` in the first layer's mixer, so that one score stands out among
    hundreds and a key wrongly seen or wrongly missed, or a state that was lost, moves the logits by far more than
    rounding does.

    Attention: the query matrix becomes the key matrix behind a map that sends the probe's normed embedding to the
    needle's, biases of queries and keys are cleared, the gains of the two norms are set to one and rotation is left to
    the configuration (the tests' first layers rotate few channels slowly); the query is scaled so that the needle's
    score is `strength` above the rest. State space: the needle writes a large step into the state (its dt row is
    lifted), the decay rates are made tiny so that the state still holds it hundreds of tokens later, and the probe's C
    becomes the needle's B."""
    t = {n: v.float().clone() for n, v in tensors.items()}

    def normed(tok):
        return pr.norm_of(t["embed"][tok].double(), {k: v.double() for k, v in t.items() if k.startswith("l0.norm1")},
                          "l0.norm1").float()

    hp, hn = normed(probe), normed(needle)

    def looking(wk):
        return wk + torch.outer(wk @ (hn - hp), hp) / (hp @ hp)

    e, m = cfg["layers"][0], cfg["layers"][0]["mixer"]
    if e["type"] == "attention":
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        k = looking(t["l0.mix.k"]).view(G, D, -1)
        t["l0.mix.q"] = k.repeat_interleave(H // G, dim=0).reshape(H * D, -1).clone()
        for n in ("q.b", "k.b"):
            t["l0.mix." + n].zero_()
        for n in ("q.norm", "k.norm"):
            t["l0.mix." + n].fill_(1.0)
        # after the whole-row norms a head's query and key have about D entries of size 1: a matching pair scores about
        # D * scale; the query's gain brings that to `strength`
        t["l0.mix.q.norm"].fill_(strength / (m["scale"] * D))
    else:
        H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
        inner = H * P
        b0, c0, d0 = 2 * inner, 2 * inner + G * N, 2 * inner + 2 * G * N
        w_in = t["l0.mix.in"]
        w_in[c0:c0 + G * N] = looking(w_in[b0:b0 + G * N]) * 3.0
        # the convolution passes the row itself alone for B and C, so that the probe's C is the needle's B whatever
        # came before either
        K = t["l0.mix.conv"].shape[1]
        t["l0.mix.conv"][inner:, :K - 1] = 0.0
        t["l0.mix.conv"][inner:, K - 1] = 1.0
        t["l0.mix.conv.b"][inner:] = 0.0
        t["l0.mix.A_log"].fill_(-9.0)
        # steps are small everywhere but at the needle
        w_in[d0:] = torch.outer(torch.full((H,), 6.0), hn - hp * (hn @ hp) / (hp @ hp)) / (hn @ hn)
        t["l0.mix.dt_bias"].fill_(-4.0)
    return {n: v.to(tensors[n].dtype) for n, v in t.items()}


def all_chosen(cfg):
    """The same configuration with every expert of every routed layer chosen for every row."""
    c = copy.deepcopy(cfg)
    for e in c["layers"]:
        if e.get("mlp") and e["mlp"]["kind"] == "moe":
            e["mlp"]["router"]["top"] = e["mlp"]["router"]["experts"]
    return c
