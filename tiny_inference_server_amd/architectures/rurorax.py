"""The Rurorax decoder as a spec of parts.

Token embedding into a 32-bit stream; parallel blocks x <- x + s1 * mixer(h) + s2 * ff(h) in which both sublayers read
the same h = dyt(x) (dynamic tanh: tanh(alpha x) * gain + bias, element by element, without statistics of the row) and s1, s2 are factors per
channel; a closing dynamic tanh; the embedding table again as the output table; logits capped by cap * tanh(. / cap).
A layer's mixer is grouped-query attention inside chunks of positions ("attention": biased projections, an RMS norm over
the whole of a row's queries and of its keys, rotation of a head's first channels, paired half the rotated part apart, at frequencies divided by a factor) or a
selective state-space recurrence ("mamba2"). The feed-forward is a gated dense layer with biases and the tanh-form gelu,
a mixture of gated silu experts with a sigmoid router whose weight scales the expert's input, or absent.

Tensor names: `embed`, `final.norm` (+ `.alpha`, `.b`), and per layer i `l<i>.norm1` (+ `.alpha`, `.b`), `l<i>.ls1`,
`l<i>.ls2`, `l<i>.mix.*` and `l<i>.mlp.*` (`gate`, `up`, `down` with `.b` each; or `router` and `e<k>.gate`, `e<k>.up`,
`e<k>.down`).
"""
from __future__ import annotations

from ..config.model_config import ARCHITECTURES, Architecture
from ..config.rurorax_config import RuroraxConfig
from ..parts.spec import LayerCall, LayerSpec, ModelSpec, PartSpec, StageSpec

NO_CONTEXT_LIMIT = 1 << 30      # nothing in the design bounds a sequence's length


def _norm(cfg, name):
    return PartSpec("norm", "dynamic_tanh", {"width": cfg.width}, {"gain": name, "bias": name + ".b", "alpha": name + ".alpha"})


def _factor(cfg, name):
    return PartSpec("gate", "channel_factor", {"width": cfg.width}, {"factor": name})


def _attention(cfg, m, pre):
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    params = {"width": cfg.width, "n_heads": m["heads"], "n_kv_heads": m["kv_heads"], "key_dim": m["dim"],
              "value_dim": m["vdim"], "scale": m["scale"], "eps": cfg.norm_eps, "rot_dims": dims,
              "rot_base": rot.get("base", 10000.0) if dims else 1.0,
              "rot_factor": (rot.get("scaling") or {}).get("factor", 1.0),
              "chunk": (m.get("mask") or {}).get("size", 0)}
    names = {k: pre + k for k in ("q", "k", "v", "o")}
    names.update(q_bias=pre + "q.b", k_bias=pre + "k.b", v_bias=pre + "v.b", o_bias=pre + "o.b", q_norm=pre + "q.norm",
                 k_norm=pre + "k.norm")
    return PartSpec("mixer", "chunked_attention", params, names)


def _state_space(cfg, m, pre):
    params = {"width": cfg.width, "n_heads": m["heads"], "vdim": m["vdim"], "state": m["state"], "groups": m["groups"],
              "taps": m["conv"], "norm_groups": m.get("norm_groups", 1), "eps": cfg.norm_eps}
    names = {"in": pre + "in", "conv": pre + "conv", "conv_bias": pre + "conv.b", "dt_bias": pre + "dt_bias",
             "a_log": pre + "A_log", "skip": pre + "D", "norm": pre + "norm", "o": pre + "o"}
    return PartSpec("mixer", "selective_state_space", params, names)


_MIXERS = {"attention": _attention, "mamba2": _state_space}


def _feed_forward(cfg, mlp, pre):
    if mlp["kind"] == "dense":
        names = {k: pre + k for k in ("gate", "up", "down")}
        names.update(gate_bias=pre + "gate.b", up_bias=pre + "up.b", down_bias=pre + "down.b")
        return PartSpec("feed_forward", "gated_dense_biased", {"width": cfg.width, "hidden": mlp["ff"], "act": "gelu_tanh"},
                        names)
    n = mlp["router"]["experts"]
    params = {"width": cfg.width, "hidden": mlp["expert"]["ff"], "n_experts": n, "top": mlp["router"]["top"],
              "score": "sigmoid", "act": "silu"}
    names = {"router": pre + "router"}
    for e in range(n):
        for k in ("gate", "up", "down"):
            names[f"{k}{e}"] = f"{pre}e{e}.{k}"
    return PartSpec("feed_forward", "input_weighted_experts", params, names)


def _block(cfg, entry, i):
    pre = f"l{i}."
    parts = {"norm": _norm(cfg, pre + "norm1"), "mixer": _MIXERS[entry["type"]](cfg, entry["mixer"], pre + "mix."),
             "mixer_scale": _factor(cfg, pre + "ls1")}
    if entry.get("mlp") is not None:
        parts["feed_forward"] = _feed_forward(cfg, entry["mlp"], pre + "mlp.")
        parts["feed_forward_scale"] = _factor(cfg, pre + "ls2")
    return LayerSpec("parallel_scaled", parts)


def build_spec(cfg: RuroraxConfig) -> ModelSpec:
    layers = tuple(_block(cfg, entry, i) for i, entry in enumerate(cfg.layers))
    ignorable = [f"l{i}.ls2" for i, entry in enumerate(cfg.layers) if entry.get("mlp") is None]
    stage = StageSpec(name="trunk", lag=0, input=PartSpec("stage_input", "scaled_token_embedding", {"scale": 1.0}),
                      calls=tuple(LayerCall(i) for i in range(len(layers))), out_norm=_norm(cfg, "final.norm"))
    return ModelSpec(d_model=cfg.width, vocab_size=cfg.vocab, max_context=NO_CONTEXT_LIMIT, layers=layers,
                     stages=(stage,), embedding="embed", lm_head="embed", eos_token_id=-1, ignorable=tuple(ignorable),
                     logit_softcap=float(cfg.logit_softcap))


ARCHITECTURES.register("Rurorax", Architecture("Rurorax", RuroraxConfig, build_spec))
