"""The Fesupel decoder as a spec of parts.

Scaled token embedding into a 32-bit stream; blocks with an RMS norm before and after each sublayer,
x <- x + norm1b(mixer(norm1(x))), x <- x + norm2b(ff(norm2(x))), then a per-layer token input
x <- x + rmsnorm(proj(gelu_tanh(gate x) * side[token])); a closing RMS norm and an output table of its own. A layer's
mixer ("parallel") is two mixers side by side on the same rows, each result RMS-normed over the width and the two
averaged: attention inside chunks of positions with sigmoid weights that are mixed across the heads ("left"), and a
gated delta rule with a decay per key channel ("right"). The feed-forward is a dense layer with a squared relu, a
mixture of clamped gated experts with grouped choice, identity experts and a gated shared expert, or absent.

Tensor names: `embed`, `head`, `final.norm`, `side.embed`, and per layer i `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`,
`l<i>.norm2b`, `l<i>.mix.left.*` (`q`, `k`, `v` with `.b` each, `pb`, `talk`, `o`, `out`), `l<i>.mix.right.*` (`q`, `k`,
`v` with `.conv` each, `b`, `A_log`, `a1`, `a2`, `dt_bias`, `g1`, `g2`, `norm`, `o`, `out`), `l<i>.mlp.*` (`up`, `down`; or
`router`, `correction`, `e<k>.gate`, `e<k>.up`, `e<k>.down`, `shared.gate`, `shared.up`, `shared.down`, `shared.sg`) and
`l<i>.side.*` (`gate`, `proj`, `norm`).
"""
from __future__ import annotations

from ..config.fesupel_config import FesupelConfig
from ..config.model_config import ARCHITECTURES, Architecture
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec

NO_CONTEXT_LIMIT = 1 << 30      # nothing in the design bounds a sequence's length


def _norm(cfg, name):
    return PartSpec("norm", "rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps}, {"gain": name})


def _left(cfg, m, pre):
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    sc = rot.get("scaling")
    params = {"width": cfg.width, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"],
              "value_dim": m["vdim"], "scale": m["scale"], "softcap": m.get("softcap") or 0.0,
              "chunk": (m.get("mask") or {}).get("size", 0), "rot_dims": dims,
              "rot_base": rot.get("base", 10000.0) if dims else 1.0,
              "rot_bands": (sc["factor"], sc["low"], sc["high"], sc["original"]) if sc and dims else None}
    names = {k: pre + k for k in ("q", "k", "v", "o", "talk")}
    names.update(q_bias=pre + "q.b", k_bias=pre + "k.b", v_bias=pre + "v.b", head_bias=pre + "pb")
    return PartSpec("mixer", "sigmoid_mixed_attention", params, names)


def _right(cfg, m, pre):
    for k in ("decay_rank", "gate_rank"):
        if k not in m:
            raise ValueError(f"the right mixer's {k} is in no key: complete the configuration from the weight file's "
                             f"shapes (with_tensor_shapes) or give it in the mixer's entry")
    params = {"width": cfg.width, "n_heads": m["heads"], "qk_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"],
              "taps": m["conv"], "decay_rank": m["decay_rank"], "gate_rank": m["gate_rank"], "eps": cfg.norm_eps}
    names = {k: pre + k for k in ("q", "k", "v", "b", "a1", "a2", "dt_bias", "g1", "g2", "norm", "o")}
    names.update(q_conv=pre + "q.conv", k_conv=pre + "k.conv", v_conv=pre + "v.conv", a_log=pre + "A_log")
    return PartSpec("mixer", "gated_delta_rule", params, names)


def _feed_forward(cfg, mlp, pre):
    if mlp["kind"] == "dense":
        return PartSpec("feed_forward", "activated_dense", {"width": cfg.width, "hidden": mlp["ff"], "act": "relu2"},
                        {"up": pre + "up", "down": pre + "down"})
    r = mlp["router"]
    n, groups, shared = r["experts"], r.get("groups") or {}, mlp.get("shared")
    params = {"width": cfg.width, "hidden": mlp["expert"]["ff"] if n else 0, "limit": mlp["expert"]["limit"] if n else 0.0,
              "n_experts": n, "n_identity": r.get("identity", 0), "top": r["top"], "groups": groups.get("count", 1),
              "keep": groups.get("keep", groups.get("count", 1)), "shared_hidden": shared["ff"] if shared else 0,
              "shared_limit": shared["limit"] if shared else 0.0}
    names = {"router": pre + "router", "correction": pre + "correction"}
    for e in range(n):
        for k in ("gate", "up", "down"):
            names[f"{k}{e}"] = f"{pre}e{e}.{k}"
    if shared:
        names.update({"shared_" + k: f"{pre}shared.{k}" for k in ("gate", "up", "down", "sg")})
    return PartSpec("feed_forward", "grouped_choice_experts", params, names)


def _block(cfg, entry, i):
    pre = f"l{i}."
    m = entry["mixer"]
    parts = {"mixer_norm": _norm(cfg, pre + "norm1"), "mixer_post_norm": _norm(cfg, pre + "norm1b"),
             "left": _left(cfg, m["left"], pre + "mix.left."), "left_join": _norm(cfg, pre + "mix.left.out"),
             "right": _right(cfg, m["right"], pre + "mix.right."), "right_join": _norm(cfg, pre + "mix.right.out")}
    if entry.get("mlp") is not None:
        parts["feed_forward_norm"] = _norm(cfg, pre + "norm2")
        parts["feed_forward"] = _feed_forward(cfg, entry["mlp"], pre + "mlp.")
        parts["feed_forward_post_norm"] = _norm(cfg, pre + "norm2b")
    if cfg.side_dim:
        params = {"width": cfg.width, "dim": cfg.side_dim, "vocab": cfg.vocab, "table_width": cfg.side_width,
                  "offset": i * cfg.side_dim, "eps": cfg.norm_eps, "act": "gelu_tanh"}
        parts["token_input"] = PartSpec("token_input", "gated_token_table", params,
                                        {"table": "side.embed", "gate": pre + "side.gate", "proj": pre + "side.proj",
                                         "norm": pre + "side.norm"})
    return LayerSpec("sandwich_stream32", parts)


def build_spec(cfg: FesupelConfig) -> ModelSpec:
    layers = tuple(_block(cfg, entry, i) for i, entry in enumerate(cfg.layers))
    ignorable = []
    for i, entry in enumerate(cfg.layers):     # a layer without a feed-forward has no norms around one; a file may carry them
        if entry.get("mlp") is None:
            ignorable += [f"l{i}.norm2", f"l{i}.norm2b"]
    stage = StageSpec(name="trunk", lag=0,
                      input=PartSpec("stage_input", "scaled_token_embedding", {"scale": cfg.embedding_scale}),
                      calls=tuple(LayerCall(i) for i in range(len(layers))), out_norm=_norm(cfg, "final.norm"))
    return ModelSpec(d_model=cfg.width, vocab_size=cfg.vocab, max_context=NO_CONTEXT_LIMIT, layers=layers,
                     stages=(stage,), embedding="embed", lm_head="head", eos_token_id=-1, ignorable=tuple(ignorable))


ARCHITECTURES.register("Fesupel", Architecture("Fesupel", FesupelConfig, build_spec))
