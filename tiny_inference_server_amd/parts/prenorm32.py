"""Parts of pre-norm blocks over a residual stream that stays in 32-bit: x <- x + sub(norm(x)).

The stream travels as a `Stream32` whose 32-bit rows only sums and norms touch; a norm turns them into rows of the
compute type for the products. Every residual sum is one kernel that also does what follows it on the same row (the
next norm, a copy in the compute type), so a block of mixer, feed-forward and token input is three such kernels
beside its products.
"""
from __future__ import annotations

import torch

from .base import ARRANGEMENTS, NORMS, TOKEN_INPUTS, Arrangement, to_compute, to_gain
from .stream32 import Stream32


@NORMS.register("layernorm")
class LayerNorm:
    """y = (x - mean) / sqrt(var + eps) * gain + bias, var being the mean of the squared deviations, in 32-bit. Takes a
    32-bit stream (or plain 32-bit rows), gives rows in the compute type. params: width, eps. tensors: gain, bias
    (width,)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {"gain": (params["width"],), "bias": (params["width"],)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.eps = float(spec.params["eps"])
        self.gain = to_gain(ops, tensors.of(spec, "gain"))
        self.bias = to_gain(ops, tensors.of(spec, "bias"))

    def fused(self):
        """(kind, gain, bias, eps) for a residual sum that applies this norm to its result."""
        return "layer", self.gain, self.bias, self.eps

    def __call__(self, x):
        if isinstance(x, Stream32) and x.normed_by is self:
            return x.rows               # the block before has applied this norm in its last kernel
        return self.ops.layernorm32(x.full if isinstance(x, Stream32) else x, self.gain, self.bias, self.eps)


@TOKEN_INPUTS.register("gated_token_table")
class GatedTokenTable:
    """What a layer adds from a table with a short row per token: y = Wp . (act(Wg . x) * table[token]), RMS-normed with
    a gain before it joins the stream (the norm is left to the residual sum that follows). The table may be a slice of
    columns of a wider one that several layers share.

    params: width, dim, vocab, table_width, offset (first column of this layer's slice), eps, act. tensors: table
    (vocab, table_width), gate (dim, width), proj (width, dim), stored [out, in], norm (width,).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, d = params["width"], params["dim"]
        return {"table": (params["vocab"], params["table_width"]), "gate": (d, w), "proj": (w, d), "norm": (w,)}

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        off, dim = int(p.get("offset", 0)), int(p["dim"])
        self.table = to_compute(ops, tensors.of(spec, "table")[:, off:off + dim])
        self.w_gate = to_compute(ops, tensors.of(spec, "gate"))
        self.w_proj = to_compute(ops, tensors.of(spec, "proj"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.eps = float(p["eps"])
        self.act = str(p.get("act", "gelu_tanh"))

    def forward(self, x, tokens):
        ops = self.ops
        z = ops.linear(x, self.w_gate, out_dtype=torch.float32)
        g = ops.gate_table(z, self.table, tokens, self.act)
        return ops.linear(g, self.w_proj, out_dtype=torch.float32), (self.norm_gain, self.eps)


@ARRANGEMENTS.register("prenorm_stream32")
class PreNormStream32(Arrangement):
    """x <- x + mixer(norm_a(x));  x <- x + feed_forward(norm_f(x));  x <- x + token_input(x), on a 32-bit stream.

    The feed-forward and the token input are optional. Sublayers give their results in 32-bit (`forward32`); every sum
    is 32-bit. parts: mixer_norm, mixer, and optionally feed_forward_norm + feed_forward, token_input.
    """
    part_names = None

    def __init__(self, layer_spec, tensors, ops):
        super().__init__(layer_spec, tensors, ops)
        known = {"mixer_norm", "mixer", "feed_forward_norm", "feed_forward", "token_input"}
        if not {"mixer_norm", "mixer"} <= set(self.parts) or set(self.parts) - known:
            raise ValueError(f"a prenorm_stream32 block is made of {sorted(known)}, its spec brings {sorted(self.parts)}")
        self.norm_a, self.mixer = self.parts["mixer_norm"], self.parts["mixer"]
        self.ffn, self.norm_f = self.parts.get("feed_forward"), self.parts.get("feed_forward_norm")
        self.side = self.parts.get("token_input")
        self.first_norm = self.norm_a       # what reads this block's input first: the block before may apply it
        if (self.ffn is None) != (self.norm_f is None):
            raise ValueError("a prenorm_stream32 block has a feed-forward and its norm, or neither")

    @staticmethod
    def _fusable(norm):
        """Whether the residual sum's kernel can apply this norm (a layer norm or an RMS norm that offers its constants)."""
        return norm is not None and hasattr(norm, "fused") and norm.fused()[0] in ("layer", "rms")

    def _sum(self, x32, y, norm=None, copy=False, y_rms=None):
        """x32 + y with the norm that follows; a norm that cannot be fused is applied on its own."""
        fused = norm.fused() if self._fusable(norm) else None
        x32, cp, normed = self.ops.residual_norm(x32, y, y_rms=y_rms, copy=copy, norm=fused)
        if norm is not None and fused is None:
            normed = norm(x32)
        return x32, cp, normed

    def forward(self, x, ctx):
        x32 = x.full
        y = self.mixer.forward32(self.norm_a(x), ctx.of("mixer"))
        if self.ffn is not None:
            x32, _, h = self._sum(x32, y, norm=self.norm_f)
            # (a routed feed-forward leaves the sum over a row's chosen experts to the residual sum's kernel)
            y = self.ffn.forward32(h, combine=False) if getattr(self.ffn, "sums_in_residual", False) else self.ffn.forward32(h)
        # the block's last sum also applies the norm that reads its result next, where that norm can be fused
        after = ctx.next_norm if self._fusable(ctx.next_norm) else None
        if self.side is None:
            x32, _, normed = self._sum(x32, y, norm=after)
        else:
            x32, rows, _ = self._sum(x32, y, copy=True)
            y, y_rms = self.side.forward(rows, ctx.batch.tokens)
            x32, _, normed = self._sum(x32, y, y_rms=y_rms, norm=after)
        return Stream32(x32, normed, normed_by=after)
