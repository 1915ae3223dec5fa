"""Configuration of the Fesupel decoder, read from its config.json.

Keys: `vocab`, `width`, `norm.eps`, optionally `embedding.scale` (1), `token_side.dim` (the width of a layer's slice of
the per-token side table; absent: no layer has a token input) and `layers`, a list with one entry per layer: `type`
("parallel"), `mixer` ({"left": ..., "right": ...}) and `mlp` ({"kind": "dense", "ff": n}, {"kind": "moe", ...} or null
for a layer without a feed-forward).

`mixer.left` (attention inside chunks with sigmoid weights mixed across heads) gives `heads`, `kv_heads`, `dim`, `vdim`,
`scale`, and optionally `softcap` (absent or 0: scores stay as they are), `mask` ({"size": n}; absent: all earlier
keys) and `rot` ({"dims", "base", "scaling": {"factor", "low", "high", "original"}}; absent or dims 0: no rotation; no
scaling: plain frequencies). `mixer.right` (a gated delta rule) gives `heads`, `kv_heads`, `dim`, `vdim`, `conv` (taps).
A "moe" feed-forward gives `expert` ({"ff", "limit"}), `router` ({"experts", "top", optionally "identity" (0) and
"groups": {"count", "keep"}}) and optionally `shared` ({"ff", "limit"}).

Two sizes are in no key: the ranks of the right mixer's two low-rank projections are the first dimensions of its
`a1` and `g1` tensors, and the side table may be wider than dim x layers. `with_tensor_shapes` completes the
configuration from the weight file's header (a config.json may also give them as `decay_rank` and `gate_rank` in the
right mixer's entry).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, Mapping, Tuple

from .fikevik_config import _need, _number

MIXER_TYPES = ("parallel",)
MLP_KINDS = ("dense", "moe")


def _check_left(m, where):
    for k in ("heads", "kv_heads", "dim", "vdim"):
        _number(m, k, where, int, 1)
    _need(m["heads"] % m["kv_heads"] == 0, f"{where}: {m['heads']} heads over {m['kv_heads']} kv_heads")
    _number(m, "scale", where, float)
    if m.get("softcap") is not None:
        _need(_number(m, "softcap", where, float) >= 0, f"{where}.softcap must not be negative")
    if m.get("mask") is not None:
        _number(m["mask"], "size", where + ".mask", int, 1)
    rot = m.get("rot")
    if rot is not None:
        dims = _number(rot, "dims", where + ".rot", int, 0)
        _need(dims % 2 == 0 and dims <= m["dim"], f"{where}.rot.dims {dims}: an even number, at most dim {m['dim']}")
        if dims:
            _need(_number(rot, "base", where + ".rot", float) > 0, f"{where}.rot.base must be positive")
        sc = rot.get("scaling")
        if sc is not None:
            w = where + ".rot.scaling"
            _need(_number(sc, "factor", w, float) > 0, f"{w}.factor must be positive")
            low, high = _number(sc, "low", w, float), _number(sc, "high", w, float)
            _need(_number(sc, "original", w, float) > 0 and low > 0 and high > 0, f"{w}: low, high and original must be positive")


def _check_right(m, where):
    for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
        _number(m, k, where, int, 1)
    _need(m["heads"] % m["kv_heads"] == 0, f"{where}: {m['heads']} heads over {m['kv_heads']} kv_heads")
    for k in ("decay_rank", "gate_rank"):
        if k in m:
            _number(m, k, where, int, 1)


def _check_gated(e, where):
    _number(e, "ff", where, int, 1)
    _need(_number(e, "limit", where, float) > 0, f"{where}.limit must be positive")


def _check_layer(i, entry):
    where = f"layers[{i}]"
    _need(isinstance(entry, Mapping), f"{where} must be an object")
    _need(entry.get("type") in MIXER_TYPES, f"{where}.type {entry.get('type')!r}: known are {', '.join(MIXER_TYPES)}")
    m = entry.get("mixer")
    _need(isinstance(m, Mapping) and isinstance(m.get("left"), Mapping) and isinstance(m.get("right"), Mapping),
          f"{where}.mixer needs 'left' and 'right'")
    _check_left(m["left"], where + ".mixer.left")
    _check_right(m["right"], where + ".mixer.right")
    mlp = entry.get("mlp")
    if mlp is None:
        return
    _need(isinstance(mlp, Mapping) and mlp.get("kind") in MLP_KINDS,
          f"{where}.mlp.kind {mlp.get('kind') if isinstance(mlp, Mapping) else mlp!r}: known are {', '.join(MLP_KINDS)}")
    if mlp["kind"] == "dense":
        _number(mlp, "ff", where + ".mlp", int, 1)
        return
    r, rw = mlp.get("router"), where + ".mlp.router"
    n = _number(r, "experts", rw, int, 0)
    ident = _number(r, "identity", rw, int, 0) if "identity" in r else 0
    top = _number(r, "top", rw, int, 1)
    _need(top <= n + ident, f"{rw}.top {top} of {n} + {ident} experts")
    g = r.get("groups")
    if g is not None:
        count, keep = _number(g, "count", rw + ".groups", int, 1), _number(g, "keep", rw + ".groups", int, 1)
        _need((n + ident) % count == 0 and keep <= count, f"{rw}.groups: {count} groups of {n} + {ident} experts, {keep} kept")
        _need(top <= keep * ((n + ident) // count), f"{rw}.top {top} of {keep} groups of {(n + ident) // count}")
    if n:
        _check_gated(mlp.get("expert"), where + ".mlp.expert")
    if mlp.get("shared") is not None:
        _check_gated(mlp["shared"], where + ".mlp.shared")


@dataclass(frozen=True)
class FesupelConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    side_dim: int                      # 0: no per-layer token input
    layers: Tuple[Dict[str, Any], ...]
    architecture: str = "Fesupel"
    extra: Dict[str, Any] = field(default_factory=dict, compare=False)
    side_table_width: int = 0          # columns of the side table; 0: side_dim * layers (a file's table may be wider)

    def __post_init__(self):
        _need(self.vocab >= 1 and self.width >= 1, f"vocab {self.vocab} and width {self.width} must be at least 1")
        _need(self.norm_eps >= 0, f"norm.eps must not be negative, got {self.norm_eps}")
        _need(self.side_dim >= 0, f"token_side.dim must not be negative, got {self.side_dim}")
        _need(len(self.layers) >= 1, "layers must not be empty")
        for i, entry in enumerate(self.layers):
            _check_layer(i, entry)

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FesupelConfig":
        _need(isinstance(raw.get("layers"), list), "config.json lacks 'layers' (a list)")
        used = {"architecture", "vocab", "width", "embedding", "norm", "token_side", "layers"}
        side, emb = raw.get("token_side"), raw.get("embedding")
        return cls(vocab=_number(raw, "vocab", "config", int, 1), width=_number(raw, "width", "config", int, 1),
                   embedding_scale=_number(emb, "scale", "embedding", float) if emb is not None else 1.0,
                   norm_eps=_number(raw.get("norm"), "eps", "norm", float),
                   side_dim=_number(side, "dim", "token_side", int, 0) if side is not None else 0,
                   layers=tuple(copy.deepcopy(dict(e)) if isinstance(e, Mapping) else e for e in raw["layers"]),
                   architecture=str(raw.get("architecture", "Fesupel")),
                   extra={k: v for k, v in raw.items() if k not in used})

    @property
    def side_width(self) -> int:
        return self.side_table_width or self.side_dim * len(self.layers)

    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "FesupelConfig":
        """The same configuration with every size that only a tensor's shape gives filled in: the ranks of the right
        mixer's low-rank projections and the side table's width."""
        layers = copy.deepcopy(list(self.layers))
        for i, entry in enumerate(layers):
            right = entry["mixer"]["right"]
            for key, name in (("decay_rank", f"l{i}.mix.right.a1"), ("gate_rank", f"l{i}.mix.right.g1")):
                if key not in right and name in shapes and len(shapes[name]) == 2:
                    right[key] = int(shapes[name][0])
        table, width = shapes.get("side.embed"), self.side_table_width
        if self.side_dim and table is not None and len(table) == 2 and table[1] >= self.side_dim * len(layers):
            width = int(table[1])
        return FesupelConfig(self.vocab, self.width, self.embedding_scale, self.norm_eps, self.side_dim, tuple(layers),
                             self.architecture, dict(self.extra), width)

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
               "layers": copy.deepcopy(list(self.layers))}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        return out
