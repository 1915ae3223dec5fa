"""Parts of parallel blocks over a residual stream that stays in 32-bit: x <- x + s_m * mixer(h) + s_f * ff(h), where
both sublayers read the same h = norm(x) and s_m, s_f are factors per channel.

The block's one sum is one kernel: it adds both branches with their factors and output biases, takes the sum over a
row's chosen experts where the feed-forward is routed, and applies the norm that reads the stream next (the following
block's, or the model's closing norm), so a block is that kernel beside its sublayers' products.
"""
from __future__ import annotations

from .base import ARRANGEMENTS, GATES, NORMS, Arrangement, to_gain
from .stream32 import Stream32


@NORMS.register("dynamic_tanh")
class DynamicTanh:
    """y = tanh(alpha * x) * gain + bias, element by element with one scalar alpha: a norm that computes no mean and no
    variance. Takes a 32-bit stream (or plain 32-bit rows), gives rows in the compute type. params: width. tensors:
    gain, bias (width,), alpha (a scalar)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {"gain": (params["width"],), "bias": (params["width"],), "alpha": ()}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.gain = to_gain(ops, tensors.of(spec, "gain"))
        self.bias = to_gain(ops, tensors.of(spec, "bias"))
        self.alpha = float(tensors.of(spec, "alpha").float().reshape(()).item())     # a constant of the launches

    def fused(self):
        """(kind, alpha, gain, bias) for a residual sum that applies this norm to its result."""
        return "dyt", self.alpha, self.gain, self.bias

    def __call__(self, x):
        if isinstance(x, Stream32) and x.normed_by is self:
            return x.rows               # the block before has applied this norm in its last kernel
        return self.ops.dyt32(x.full if isinstance(x, Stream32) else x, self.alpha, self.gain, self.bias)


@GATES.register("channel_factor")
class ChannelFactor:
    """A learned factor per channel on a sublayer's result (layer scale). params: width. tensors: factor (width,)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        return {"factor": (params["width"],)}

    def __init__(self, spec, tensors, ops):
        self.factor = to_gain(ops, tensors.of(spec, "factor"))


@ARRANGEMENTS.register("parallel_scaled")
class ParallelScaled(Arrangement):
    """h = norm(x);  x <- x + mixer_scale * mixer(h) + feed_forward_scale * feed_forward(h), on a 32-bit stream.

    There is one norm and both sublayers read its result. The feed-forward and the factors are optional. A sublayer
    gives its result in 32-bit as `forward_parts(h[, ctx]) -> (y, output bias | None)` (the bias is added inside the
    sum) or as `forward32(h[, ctx]) -> y`; a routed feed-forward may leave the sum over a row's choices to the block's
    sum (`sums_in_residual`). parts: norm, mixer, and optionally mixer_scale, feed_forward, feed_forward_scale.
    """
    part_names = None

    def __init__(self, layer_spec, tensors, ops):
        super().__init__(layer_spec, tensors, ops)
        known = {"norm", "mixer", "mixer_scale", "feed_forward", "feed_forward_scale"}
        if not {"norm", "mixer"} <= set(self.parts) or set(self.parts) - known:
            raise ValueError(f"a parallel_scaled block is made of {sorted(known)}, its spec brings {sorted(self.parts)}")
        self.norm, self.mixer, self.ffn = self.parts["norm"], self.parts["mixer"], self.parts.get("feed_forward")
        if "feed_forward_scale" in self.parts and self.ffn is None:
            raise ValueError("a parallel_scaled block has a factor for a feed-forward that it lacks")
        self.mixer_scale = self.parts["mixer_scale"].factor if "mixer_scale" in self.parts else None
        self.ffn_scale = self.parts["feed_forward_scale"].factor if "feed_forward_scale" in self.parts else None
        self.first_norm = self.norm         # what reads this block's input first: the block before may apply it

    @staticmethod
    def _result(part, *args):
        if hasattr(part, "forward_parts"):
            return part.forward_parts(*args)
        return part.forward32(*args), None

    def forward(self, x, ctx):
        h = self.norm(x)
        y, bias = self._result(self.mixer, h, ctx.of("mixer"))
        branches = [(y, self.mixer_scale, bias)]
        if self.ffn is not None:
            y, bias = self._result(self.ffn, h)
            branches.append((y, self.ffn_scale, bias))
        after = ctx.next_norm if getattr(ctx.next_norm, "fused", None) and ctx.next_norm.fused()[0] == "dyt" else None
        x32, normed = self.ops.scaled_sum(x.full, branches, norm=after.fused() if after is not None else None)
        return Stream32(x32, normed, normed_by=after)
