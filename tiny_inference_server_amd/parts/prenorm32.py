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

    def _mixed(self, h, ctx):
        """(the mixer's result in 32-bit, the RMS norm (gain, eps) that it still needs before it joins the stream)."""
        return self.mixer.forward32(h, ctx.of("mixer")), None

    _ffn_rms = None     # the RMS norm (gain, eps) that the feed-forward's result still needs; None: it joins as it is

    def forward(self, x, ctx):
        x32 = x.full
        y, y_rms = self._mixed(self.norm_a(x), ctx)
        if self.ffn is not None:
            x32, _, h = self._sum(x32, y, y_rms=y_rms, norm=self.norm_f)
            # (a routed feed-forward leaves the sum over a row's chosen experts to the residual sum's kernel)
            y = self.ffn.forward32(h, combine=False) if getattr(self.ffn, "sums_in_residual", False) else self.ffn.forward32(h)
            y_rms = self._ffn_rms
        # the block's last sum also applies the norm that reads its result next, where that norm can be fused
        after = ctx.next_norm if self._fusable(ctx.next_norm) else None
        if self.side is None:
            x32, _, normed = self._sum(x32, y, y_rms=y_rms, norm=after)
        else:
            x32, rows, _ = self._sum(x32, y, y_rms=y_rms, copy=True)
            y, y_rms = self.side.forward(rows, ctx.batch.tokens)
            x32, _, normed = self._sum(x32, y, y_rms=y_rms, norm=after)
        return Stream32(x32, normed, normed_by=after)


@ARRANGEMENTS.register("sandwich_stream32")
class SandwichStream32(PreNormStream32):
    """x <- x + post_a(mix(norm_a(x)));  x <- x + post_f(feed_forward(norm_f(x)));  x <- x + token_input(x), on a 32-bit
    stream: an RMS norm before and after each sublayer. The norm after a sublayer is applied inside the residual sum.

    One mixer ("mixer"), or several side by side that read the same rows (any part whose role is "mixer", under any
    names): each mixer's result is then RMS-normed over the width with the gain `<name>_join` and the results are
    averaged. The mixers' input matrices are one product where every mixer offers `input_rows` and `forward_projected`.
    The feed-forward and the token input are optional.

    parts: mixer_norm, mixers, `<name>_join` (kind "rmsnorm") per mixer where there are several, mixer_post_norm, and
    optionally feed_forward_norm + feed_forward + feed_forward_post_norm, token_input.
    """
    part_names = None

    def __init__(self, layer_spec, tensors, ops):
        Arrangement.__init__(self, layer_spec, tensors, ops)
        names = [n for n, _ in layer_spec.mixers()]
        joins = {n + "_join" for n in names} if len(names) > 1 else set()
        known = {"mixer_norm", "mixer_post_norm", "feed_forward_norm", "feed_forward", "feed_forward_post_norm",
                 "token_input"} | set(names) | joins
        need = {"mixer_norm", "mixer_post_norm"} | joins
        if not names or not need <= set(self.parts) or set(self.parts) - known:
            raise ValueError(f"a sandwich_stream32 block is made of {sorted(known)}, its spec brings {sorted(self.parts)}")
        self.norm_a, self.post_a = self.parts["mixer_norm"], self.parts["mixer_post_norm"]
        self.ffn, self.norm_f = self.parts.get("feed_forward"), self.parts.get("feed_forward_norm")
        self.post_f = self.parts.get("feed_forward_post_norm")
        self.side = self.parts.get("token_input")
        self.first_norm = self.norm_a
        if len({self.ffn is None, self.norm_f is None, self.post_f is None}) != 1:
            raise ValueError("a sandwich_stream32 block has a feed-forward and both its norms, or none of the three")
        self._ffn_rms = (self.post_f.gain, self.post_f.eps) if self.post_f is not None else None
        self.mixers = [(n, self.parts[n], self.parts[n + "_join"] if joins else None) for n in names]
        self.mixer = self.mixers[0][1]
        # one input product for all mixers that read the block's normed rows, each starting at a multiple of 8 rows (the
        # 32-bit columns of every user then start 32 bytes apart)
        self.w_in, self.cols = None, []
        if all(hasattr(m, "input_rows") and hasattr(m, "forward_projected") for _, m, _ in self.mixers):
            blocks, at = [], 0
            for _, m, _ in self.mixers:
                rows = m.input_rows
                pad = -rows.shape[0] % 8
                blocks.append(rows)
                if pad:
                    blocks.append(torch.zeros(pad, rows.shape[1], dtype=rows.dtype, device=rows.device))
                self.cols.append((at, at + rows.shape[0]))
                at += rows.shape[0] + pad
            self.w_in = to_compute(ops, torch.cat(blocks, dim=0))

    def _mixed(self, h, ctx):
        post = (self.post_a.gain, self.post_a.eps)
        if self.w_in is not None:
            proj = self.ops.linear(h, self.w_in, out_dtype=torch.float32)
            results = [m.forward_projected(proj[:, c0:c1], ctx.of(n)) for (n, m, _), (c0, c1) in zip(self.mixers, self.cols)]
        else:
            results = [m.forward32(h, ctx.of(n)) for n, m, _ in self.mixers]
        if len(results) == 1:
            return results[0], post
        eps = {j.eps for _, _, j in self.mixers}
        if len(eps) != 1:
            raise ValueError("the norms that join a block's mixers differ in eps")
        return self.ops.normed_mean([(y, j.gain) for y, (_, _, j) in zip(results, self.mixers)], eps.pop()), post
