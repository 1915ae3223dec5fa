"""Parts of blocks whose residual stream stays in 32-bit whatever the compute type, with the norm after the sum.

The stream travels as a `Stream32`: the rows in 32-bit, which only the sums and norms touch, and the same rows in
the compute type, which the matrix products read (one tensor in a 32-bit engine). A stage input makes it, the block
arrangement below passes it on, and the closing norm turns it into plain rows for the output table.
"""
from __future__ import annotations

import torch

from .base import ARRANGEMENTS, FEED_FORWARDS, GATES, NORMS, STAGE_INPUTS, Arrangement, to_compute, to_gain


class Stream32:
    __slots__ = ("full", "rows", "normed_by")

    def __init__(self, full, rows, normed_by=None):
        self.full, self.rows = full, rows        # [rows, width] float32; the same in the compute type
        # a block that was told which norm reads its result next (CallContext.next_norm) may apply it in its last
        # kernel: `rows` then holds that norm's result, and the norm part named here hands it on instead of running
        self.normed_by = normed_by


@STAGE_INPUTS.register("scaled_token_embedding")
class ScaledTokenEmbedding:
    """x = E[token] * scale, as a 32-bit stream. params: scale."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {}

    @classmethod
    def state_need(cls, params):
        return None

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.scale = float(spec.params.get("scale", 1.0))

    def forward(self, batch, previous, shared, state):
        return Stream32(*self.ops.embed_scaled(shared["embedding"], batch.tokens, self.scale))


@NORMS.register("rmsnorm")
class RmsNorm:
    """y = x / sqrt(mean(x^2) + eps) * gain, eps under the root, computed in 32-bit. Takes a 32-bit stream (or plain
    32-bit rows) and gives rows in the compute type. params: width, eps. tensors: gain (width,)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {"gain": (params["width"],)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.gain = to_gain(ops, tensors.of(spec, "gain"))

    def fused(self):
        """(kind, gain, bias, eps) for a residual sum that applies this norm to its result."""
        return "rms", self.gain, None, self.eps

    def __call__(self, x):
        if isinstance(x, Stream32) and x.normed_by is self:
            return x.rows               # the block before has applied this norm in its last kernel
        return self.ops.rmsnorm32(x.full if isinstance(x, Stream32) else x, self.gain, self.eps)


@GATES.register("sigmoid_linear")
class SigmoidLinearGate:
    """A gate per channel on a sublayer's result: sigmoid(h . W^T + b), h being what the sublayer read.
    params: width. tensors: w (width, width) stored [out, in], b (width,)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d = params["width"]
        return {"w": (d, d), "b": (d,)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.input_rows = tensors.of(spec, "w")                 # as stored: a block may fuse it into a wider product
        self.bias = to_gain(ops, tensors.of(spec, "b"))
        self._w = None

    def pre_activation(self, rows):
        if self._w is None:
            self._w = to_compute(self.ops, self.input_rows)
        return self.ops.linear(rows, self._w, out_dtype=torch.float32)


@FEED_FORWARDS.register("gated_dense")
class GatedDense:
    """y = (silu(h . Wg^T) * (h . Wu^T)) . Wd^T. params: width, hidden. tensors: gate, up (hidden, width),
    down (width, hidden), stored [out, in]."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, f = params["width"], params["hidden"]
        return {"gate": (f, d), "up": (f, d), "down": (d, f)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        gate, up = tensors.of(spec, "gate"), tensors.of(spec, "up")
        # rows alternate gate_0, up_0, gate_1, ...: the product's kernel gates where its sums still sit in registers
        self.w_gate_up = to_compute(ops, torch.stack((gate, up), dim=1).reshape(2 * gate.shape[0], gate.shape[1]))
        self.w_down = to_compute(ops, tensors.of(spec, "down"))

    def hidden(self, rows):
        return self.ops.linear_swiglu(rows, self.w_gate_up)

    def forward(self, x, residual=None):
        return self.ops.linear(self.hidden(x), self.w_down, residual=residual)

    def forward32(self, rows):
        """The result in 32-bit, for a block that sums in 32-bit."""
        return self.ops.linear(self.hidden(rows), self.w_down, out_dtype=torch.float32)


@ARRANGEMENTS.register("postnorm_gated")
class PostNormGated(Arrangement):
    """x <- norm_a(alpha x + gate_a(x) * sum_m scale_m mixer_m(x));  x <- norm_f(alpha x + gate_f(x) * ff(x)).

    The sublayers read x itself; each norm comes after its sum; sums and norms are 32-bit. Every part whose role is
    "mixer" takes part in the first sum, with the factor the block's params give it (`scales`: part name -> factor,
    1 where absent). Without a "feed_forward" part the second half is left out. Gates are optional ("mixer_gate",
    "feed_forward_gate"). The mixers' input projections and the first gate read the same rows, so they are one
    product: a mixer offers `input_rows` (its stacked input matrices as stored) and
    `forward_projected(projections, ctx) -> 32-bit rows`.

    params: alpha, scales. parts: mixer_norm, feed_forward_norm (kind "rmsnorm"), mixers under any names,
    feed_forward, mixer_gate, feed_forward_gate.
    """
    part_names = None

    def __init__(self, layer_spec, tensors, ops):
        super().__init__(layer_spec, tensors, ops)
        p = layer_spec.params
        self.alpha = float(p.get("alpha", 1.0))
        scales = p.get("scales", {})
        self.norm_a = self.parts["mixer_norm"]
        self.gate_a = self.parts.get("mixer_gate")
        self.ffn = self.parts.get("feed_forward")
        self.norm_f = self.parts.get("feed_forward_norm")
        self.gate_f = self.parts.get("feed_forward_gate")
        if self.ffn is not None and self.norm_f is None:
            raise ValueError("a postnorm_gated block with a feed-forward needs a feed_forward_norm")
        names = [n for n, _ in layer_spec.mixers()]
        if not 1 <= len(names) <= 2:
            raise ValueError(f"a postnorm_gated block sums one or two mixers, its spec brings {len(names)}")
        # one input product for everything that reads the block's input: the mixers' matrices, then the gate's,
        # each starting at a multiple of 8 rows (the 32-bit columns of every user then start 32 bytes apart)
        blocks, self.mixers, at = [], [], 0

        def add(rows):
            nonlocal at
            first = at
            pad = -rows.shape[0] % 8
            blocks.append(rows)
            if pad:
                blocks.append(torch.zeros(pad, rows.shape[1], dtype=rows.dtype, device=rows.device))
            at += rows.shape[0] + pad
            return first, first + rows.shape[0]

        for n in names:
            m = self.parts[n]
            self.mixers.append((n, m, add(m.input_rows), float(scales.get(n, 1.0))))
        self.gate_cols = add(self.gate_a.input_rows) if self.gate_a is not None else None
        self.w_in = to_compute(ops, torch.cat(blocks, dim=0))

    def forward(self, x, ctx):
        ops = self.ops
        proj = ops.linear(x.rows, self.w_in, out_dtype=torch.float32)
        branches = [(m.forward_projected(proj[:, c0:c1], ctx.of(name)), scale) for name, m, (c0, c1), scale in self.mixers]
        gate = proj[:, self.gate_cols[0]:self.gate_cols[1]] if self.gate_cols else None
        full, rows = ops.gated_postnorm(x.full, branches, gate, self.gate_a.bias if gate is not None else None,
                                        self.alpha, self.norm_a.gain, self.norm_a.eps)
        if self.ffn is not None:
            y = self.ffn.forward32(rows)
            gate = self.gate_f.pre_activation(rows) if self.gate_f is not None else None
            full, rows = ops.gated_postnorm(full, [(y, 1.0)], gate, self.gate_f.bias if gate is not None else None,
                                            self.alpha, self.norm_f.gain, self.norm_f.eps)
        return Stream32(full, rows)
