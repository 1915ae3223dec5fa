"""Configuration of the Rurorax decoder, read from its config.json.

Keys: `vocab`, `width`, `norm.eps`, optionally `logit_softcap` (absent or 0: the logits stay as they are) and `layers`, a
list with one entry per layer: `type` ("attention" or "mamba2"), `mixer` (the mixer's sizes and constants) and `mlp`
({"kind": "dense", "ff": n}, {"kind": "moe", "expert": {"ff": n}, "router": {"experts", "top"}}, or null for a layer
without a feed-forward).

An "attention" mixer gives `heads`, `kv_heads`, `dim`, `vdim`, `scale`, and optionally `rot` ({"dims", "base",
"scaling": {"factor"}}; absent or dims 0: no rotation; no scaling: factor 1) and `mask` ({"size": n}: a row sees the
keys of its own chunk of n positions; absent: all earlier keys). A "mamba2" mixer gives `heads`, `vdim`, `state`,
`groups`, `conv` (taps) and optionally `norm_groups` (1).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Tuple

from .fikevik_config import _need, _number

MIXER_TYPES = ("attention", "mamba2")
MLP_KINDS = ("dense", "moe")


def _check_mixer(kind, m, where):
    _number(m, "heads", where, int, 1)
    _number(m, "vdim", where, int, 1)
    if kind == "attention":
        _number(m, "dim", where, int, 1)
        _number(m, "kv_heads", where, int, 1)
        _need(m["heads"] % m["kv_heads"] == 0, f"{where}: {m['heads']} heads over {m['kv_heads']} kv_heads")
        _number(m, "scale", where, float)
        rot = m.get("rot")
        if rot is not None:
            dims = _number(rot, "dims", where + ".rot", int, 0)
            _need(dims % 2 == 0 and dims <= m["dim"], f"{where}.rot.dims {dims}: an even number, at most dim {m['dim']}")
            if dims:
                _need(_number(rot, "base", where + ".rot", float) > 0, f"{where}.rot.base must be positive")
            if rot.get("scaling") is not None:
                _need(_number(rot["scaling"], "factor", where + ".rot.scaling", float) > 0,
                      f"{where}.rot.scaling.factor must be positive")
        if m.get("mask") is not None:
            _number(m["mask"], "size", where + ".mask", int, 1)
    else:
        state = _number(m, "state", where, int, 1)
        groups = _number(m, "groups", where, int, 1)
        _need(m["heads"] % groups == 0, f"{where}: {m['heads']} heads over {groups} groups")
        _number(m, "conv", where, int, 1)
        parts = _number(m, "norm_groups", where, int, 1) if "norm_groups" in m else 1
        _need((m["heads"] * m["vdim"]) % parts == 0, f"{where}.norm_groups {parts} does not divide {m['heads'] * m['vdim']}")
        _need(state >= 1, f"{where}.state must be at least 1")


def _check_layer(i, entry):
    where = f"layers[{i}]"
    _need(isinstance(entry, Mapping), f"{where} must be an object")
    _need(entry.get("type") in MIXER_TYPES, f"{where}.type {entry.get('type')!r}: known are {', '.join(MIXER_TYPES)}")
    _need(isinstance(entry.get("mixer"), Mapping), f"{where}.mixer must be an object")
    _check_mixer(entry["type"], entry["mixer"], where + ".mixer")
    mlp = entry.get("mlp")
    if mlp is None:
        return
    _need(isinstance(mlp, Mapping) and mlp.get("kind") in MLP_KINDS,
          f"{where}.mlp.kind {mlp.get('kind') if isinstance(mlp, Mapping) else mlp!r}: known are {', '.join(MLP_KINDS)}")
    if mlp["kind"] == "dense":
        _number(mlp, "ff", where + ".mlp", int, 1)
    else:
        n = _number(mlp.get("router"), "experts", where + ".mlp.router", int, 1)
        top = _number(mlp.get("router"), "top", where + ".mlp.router", int, 1)
        _need(top <= n, f"{where}.mlp.router.top {top} of {n} experts")
        _number(mlp.get("expert"), "ff", where + ".mlp.expert", int, 1)


@dataclass(frozen=True)
class RuroraxConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_softcap: float               # 0: none
    layers: Tuple[Dict[str, Any], ...]
    architecture: str = "Rurorax"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)

    def __post_init__(self):
        _need(self.vocab >= 1 and self.width >= 1, f"vocab {self.vocab} and width {self.width} must be at least 1")
        _need(self.norm_eps >= 0, f"norm.eps must not be negative, got {self.norm_eps}")
        _need(self.logit_softcap >= 0, f"logit_softcap must not be negative, got {self.logit_softcap}")
        _need(len(self.layers) >= 1, "layers must not be empty")
        for i, entry in enumerate(self.layers):
            _check_layer(i, entry)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "RuroraxConfig":
        _need(isinstance(raw.get("layers"), list), "config.json lacks 'layers' (a list)")
        used = {"architecture", "vocab", "width", "norm", "logit_softcap", "layers"}
        cap = raw.get("logit_softcap")
        return cls(vocab=_number(raw, "vocab", "config", int, 1), width=_number(raw, "width", "config", int, 1),
                   norm_eps=_number(raw.get("norm"), "eps", "norm", float),
                   logit_softcap=_number(raw, "logit_softcap", "config", float) if cap is not None else 0.0,
                   layers=tuple(copy.deepcopy(dict(e)) if isinstance(e, Mapping) else e for e in raw["layers"]),
                   architecture=str(raw.get("architecture", "Rurorax")),
                   extra={k: v for k, v in raw.items() if k not in used})

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": copy.deepcopy(list(self.layers))}
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        return out
