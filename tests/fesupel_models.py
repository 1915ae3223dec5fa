"""Small Fesupel configurations with random weights for the tests, and what the tests need around them.

The configurations differ in everything a layer has: head counts of both mixers (one, some, as many key/value heads as
heads), key and value sizes (equal and different), chunks from one position to longer than any test sequence and none,
rotated channels (all, some, none) with and without slowed long waves, a cap on the scores or none, taps from 1 (nothing
of the convolution to keep) to 4, the ranks of the two low-rank projections, dense and routed feed-forwards with and
without groups, identity experts, a shared expert, a layer without a feed-forward, a model without a token input, a width
that is no multiple of 8, and sizes of one wherever a size may be one.

Routing and bfloat16: an expert is chosen by comparing scores, and a bfloat16 engine may turn a close comparison the
other way; the plain implementation would then describe another model. So the engine's bfloat16 tests run the
configurations with every expert chosen (`all_chosen`): the weights still follow the router, no comparison decides
anything. Routing itself is tested in 32-bit through the engine and kernel by kernel in both types.
"""
from __future__ import annotations

import copy
import math
from typing import Dict, List

import torch

import plain_fesupel as pf
from fikevik_models import as_f64, relative_error, run_trace, write_folder  # noqa: F401  (the tests use them from here)


def left(H, G, D, V, scale, chunk=None, dims=0, base=10000.0, bands=None, cap=None):
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": scale}
    if chunk is not None:
        m["mask"] = {"size": chunk}
    if cap is not None:
        m["softcap"] = cap
    if dims is not None:
        m["rot"] = {"dims": dims, "base": base}
        if bands is not None:
            m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), bands))
    return m


def right(H, G, D, V, taps, ra=5, rg=3):
    return {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "conv": taps, "decay_rank": ra, "gate_rank": rg}


def layer(lm, rm, mlp=None):
    return {"type": "parallel", "mixer": {"left": lm, "right": rm}, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, limit, experts, top, identity=0, groups=None, shared=None):
    r = {"experts": experts, "top": top}
    if identity:
        r["identity"] = identity
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def config(width, vocab, layers, scale=None, side=None, eps=1e-5):
    c = {"architecture": "Fesupel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if scale is not None:
        c["embedding"] = {"scale": scale}
    if side:
        c["token_side"] = {"dim": side}
    return c


def _configs():
    A = config(64, 211, [
        layer(left(4, 2, 16, 24, 0.2, chunk=24, dims=8, bands=(2.0, 1.0, 3.0, 64), cap=20.0), right(4, 2, 12, 8, 4), dense(40)),
        layer(left(2, 2, 32, 32, 0.15, chunk=7, dims=32, base=500.0), right(6, 3, 8, 4, 2, ra=4, rg=6),
              moe(24, 1.5, 6, 2, identity=2, groups=(4, 2), shared=(16, 2.5))),
        layer(left(6, 1, 8, 8, 0.3, chunk=100, dims=4, cap=5.0), right(3, 3, 16, 16, 3), None),
        layer(left(3, 3, 12, 4, 0.25, dims=None), right(2, 1, 20, 6, 1, ra=2, rg=2), moe(20, 3.0, 5, 3, shared=(8, 1.0)))],
        scale=8.0, side=6)
    # a width that is no multiple of 8, no scale on the embedding, no token input, chunks of one position (a row sees
    # itself alone), every expert chosen, one group of all experts, identity experts beside one real expert
    B = config(44, 97, [
        layer(left(2, 1, 8, 8, 0.3, chunk=1, dims=8, base=50.0), right(4, 4, 5, 4, 3, ra=3), moe(20, 2.0, 3, 3)),
        layer(left(3, 3, 10, 6, 0.25, chunk=33, dims=4, base=300.0, bands=(8.0, 1.0, 4.0, 16), cap=50.0), right(4, 2, 6, 10, 2),
              moe(12, 1.0, 1, 2, identity=3, groups=(2, 2))),
        layer(left(4, 4, 6, 6, 0.4, dims=2), right(2, 2, 9, 3, 4), dense(28))], eps=1e-6)
    # heads as wide as a served model's; prompts of the tests are long enough to cross many pages and chunks
    C = config(128, 300, [
        layer(left(4, 1, 64, 64, 0.125, chunk=100, dims=32, base=1e5, bands=(4.0, 1.0, 4.0, 256), cap=30.0), right(4, 2, 64, 32, 4, ra=16, rg=8),
              moe(64, 1.5, 6, 2, identity=2, groups=(2, 1), shared=(48, 2.0))),
        layer(left(2, 2, 128, 128, 0.09, chunk=64, dims=64, base=1e6), right(2, 1, 128, 64, 3, ra=8, rg=8), dense(96))],
        scale=11.3, side=16)
    # ones wherever a size may be one: a single head on both sides, one channel a value, one key channel, a rank of
    # one, one expert that is an identity expert, a shared expert alone beside it, a token input of one number
    D = config(24, 61, [
        layer(left(1, 1, 8, 1, 0.4, chunk=19, dims=8, base=100.0), right(1, 1, 1, 8, 2, ra=1, rg=1), moe(8, 1.0, 0, 1, identity=1, shared=(4, 1.0))),
        layer(left(2, 1, 6, 8, 0.5, chunk=2, cap=1.0), right(3, 1, 6, 1, 1, ra=2, rg=1), moe(4, 0.5, 1, 1)),
        layer(left(1, 1, 2, 2, 1.0, dims=2), right(2, 2, 3, 2, 4), None)], scale=1.0, side=1)
    return {"A": A, "B": B, "C": C, "D": D}


CONFIGS = _configs()


def tensor_shapes(cfg) -> Dict[str, tuple]:
    w, side = cfg["width"], (cfg.get("token_side") or {}).get("dim", 0)
    out = {"embed": (cfg["vocab"], w), "head": (cfg["vocab"], w), "final.norm": (w,)}
    if side:
        out["side.embed"] = (cfg["vocab"], side * len(cfg["layers"]))
    for i, e in enumerate(cfg["layers"]):
        p = f"l{i}."
        out.update({p + "norm1": (w,), p + "norm1b": (w,)})
        m, q = e["mixer"]["left"], p + "mix.left."
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out.update({q + "q": (H * D, w), q + "q.b": (H * D,), q + "k": (G * D, w), q + "k.b": (G * D,), q + "v": (G * V, w),
                    q + "v.b": (G * V,), q + "talk": (H, H), q + "pb": (H,), q + "o": (w, H * V), q + "out": (w,)})
        m, q = e["mixer"]["right"], p + "mix.right."
        H, G, D, V, K, ra, rg = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], m["decay_rank"], m["gate_rank"]
        out.update({q + "q": (G * D, w), q + "q.conv": (G * D, K), q + "k": (G * D, w), q + "k.conv": (G * D, K),
                    q + "v": (H * V, w), q + "v.conv": (H * V, K), q + "b": (H, w), q + "A_log": (H,), q + "norm": (V,),
                    q + "a1": (ra, w), q + "a2": (H * D, ra), q + "dt_bias": (H * D,), q + "g1": (rg, w), q + "g2": (H * V, rg),
                    q + "o": (w, H * V), q + "out": (w,)})
        mlp = e.get("mlp")
        if mlp is not None:
            out.update({p + "norm2": (w,), p + "norm2b": (w,)})
            f = p + "mlp."
            if mlp["kind"] == "dense":
                out.update({f + "up": (mlp["ff"], w), f + "down": (w, mlp["ff"])})
            else:
                r = mlp["router"]
                n = r["experts"] + r.get("identity", 0)
                out.update({f + "router": (n, w), f + "correction": (n,)})
                for k in range(r["experts"]):
                    ff = mlp["expert"]["ff"]
                    out.update({f"{f}e{k}.gate": (ff, w), f"{f}e{k}.up": (ff, w), f"{f}e{k}.down": (w, ff)})
                if mlp.get("shared"):
                    ff = mlp["shared"]["ff"]
                    out.update({f + "shared.gate": (ff, w), f + "shared.up": (ff, w), f + "shared.down": (w, ff), f + "shared.sg": (1, w)})
        if side:
            out.update({p + "side.gate": (side, w), p + "side.proj": (w, side), p + "side.norm": (w,)})
    return out


def random_weights(cfg, seed, storage=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/in); tables N(0, 1); gains 1 +- 0.1; biases that differ from zero; head biases that keep a sigmoid
    weight small; a head mixture near the identity; a router strong enough for its scores to differ, with a correction
    of the scores' own size; step-size biases and decay rates that spread the memories from a few tokens to hundreds."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        if name in ("embed", "side.embed"):
            t = torch.randn(shape, generator=g)
        elif name.endswith("talk"):
            t = torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith(".pb"):
            t = -2.0 + torch.randn(shape, generator=g)
        elif name.endswith("router"):
            t = 2.0 * torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith("correction"):
            t = 0.3 * torch.randn(shape, generator=g) / shape[0]
        elif name.endswith(".conv"):
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith("dt_bias"):
            t = -2.5 + 2.0 * torch.rand(shape, generator=g)
        elif name.endswith("A_log"):
            t = -2.0 + 2.5 * torch.rand(shape, generator=g)
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
        _plain[k] = (pf.forward(cfg, w64, list(ids), margins=margins), min(margins, default=math.inf))
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
    25 % (the token input and the norm after a sublayer divide short or small vectors by their own size)."""
    errs = errors(key, cfg, w64, reqs, got)
    if dtype == "float32":
        assert errs[-1][0] <= TOL[dtype], errs[-1]
    else:
        assert errs[int(0.98 * (len(errs) - 1))][0] <= TOL[dtype], errs[int(0.98 * (len(errs) - 1))]
        assert errs[-1][0] <= 0.25, errs[-1]


# ---- weights that make one key stand out ----------------------------------------------------------------------------

def sharpen(cfg, tensors, needle: int, probe: int, side: str = "left", strength: float = 12.0):
    """Make the token `probe` look for the token `needle` in the first layer, so that one key stands out among hundreds
    and a key wrongly seen or wrongly missed, or a state that was lost, moves the logits by far more than rounding does.

    side "left": the query matrix becomes the key matrix behind a map that sends the probe's normed embedding to the
    needle's; biases of queries and keys are cleared; the head biases are set so low that a key weighs nothing unless its
    score is high, and the query is scaled so that the needle's score lifts its weight to about one half; the heads are
    not mixed (rotation is left to the configuration: the tests' first layers rotate few channels slowly). side
    "right": q and k pass the convolution alone (the row's own tap is 1), the probe's q becomes the needle's k, the decay
    is made so slow that the state still holds the needle hundreds of tokens later, and beta is large at the needle
    alone (every token's embedding gets one channel in common, which the beta projection reads as a low bias)."""
    t = {n: v.float().clone() for n, v in tensors.items()}
    scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
    eps = float(cfg["norm"]["eps"])

    def normed(tok):
        return pf.rms_norm(t["embed"][tok].double() * scale, t["l0.norm1"].double(), eps).float()

    hp, hn = normed(probe), normed(needle)

    def looking(wk):
        return wk + torch.outer(wk @ (hn - hp), hp) / (hp @ hp)

    if side == "left":
        m, p = cfg["layers"][0]["mixer"]["left"], "l0.mix.left."
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        q = looking(t[p + "k"]).view(G, D, -1).repeat_interleave(H // G, dim=0)          # [H, D, width]
        kn = (t[p + "k"] @ hn).view(G, D).repeat_interleave(H // G, dim=0)               # the needle's keys, [H, D]
        for h in range(H):
            q[h] *= strength / (m["scale"] * float(kn[h] @ kn[h]))
        t[p + "q"] = q.reshape(H * D, -1).clone()
        for n in ("q.b", "k.b"):
            t[p + n].zero_()
        t[p + "pb"].fill_(-strength)
        t[p + "talk"] = torch.eye(H)
    else:
        m, p = cfg["layers"][0]["mixer"]["right"], "l0.mix.right."
        for n in ("q.conv", "k.conv"):
            t[p + n].zero_()
            t[p + n][:, -1] = 1.0
        # every token's first channel is the same large number, which the row of Wb below turns into a low beta for
        # all tokens; the needle's own direction lifts its beta to about one
        t["embed"][:, 0] = 3.0
        hp, hn = normed(probe), normed(needle)
        t[p + "q"] = (t[p + "k"] + torch.outer(t[p + "k"] @ (hn - hp), hp) / (hp @ hp)) * 4.0
        t[p + "k"] = t[p + "k"] * 4.0                      # silu of a larger number is nearer to the number itself
        t[p + "A_log"].fill_(-9.0)
        first = torch.zeros_like(hn)
        first[0] = 1.0
        own = hn - first * hn[0]
        own = own - (hp - first * hp[0]) * (own @ hp) / ((hp - first * hp[0]) @ hp)
        t[p + "b"] = torch.outer(torch.ones(m["heads"]), -6.0 * first / hn[0] + 14.0 * own / (own @ hn))
    return {n: v.to(tensors[n].dtype) for n, v in t.items()}


def all_chosen(cfg):
    """The same configuration with every expert of every routed layer chosen for every row (and so no groups)."""
    c = copy.deepcopy(cfg)
    for e in c["layers"]:
        if e.get("mlp") and e["mlp"]["kind"] == "moe":
            r = e["mlp"]["router"]
            r["top"] = r["experts"] + r.get("identity", 0)
            r.pop("groups", None)
    return c
