"""Feed-forward parts."""
from __future__ import annotations

import torch

from .base import FEED_FORWARDS, to_compute


@FEED_FORWARDS.register("swiglu")
class SwiGlu:
    """y = (silu(x.W1) * (x.W2)) . Wfc (+ residual), dense (reference main_models_new.py:44-60).

    params: d_model, hidden. tensors: gate (d_model, hidden), up (d_model, hidden), down (hidden, d_model),
    stored [in, out].
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, f = params["d_model"], params["hidden"]
        return {"gate": (d, f), "up": (d, f), "down": (f, d)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        # one projection for gate and up: rows of the [out, in] matrix alternate gate_0, up_0, gate_1, up_1, ...
        # so that the gating can be done where the product's results still sit in registers
        gate, up = tensors.of(spec, "gate"), tensors.of(spec, "up")
        self.w_gate_up = to_compute(ops, torch.stack((gate.t(), up.t()), dim=1).reshape(2 * gate.shape[1], gate.shape[0]))
        self.w_down = to_compute(ops, tensors.of(spec, "down").t())

    fuses_norm = True

    def forward(self, x, residual=None, norm=None, residual_is_spent=False):
        ops = self.ops
        if norm is not None and not hasattr(norm, "as_rms"):
            x, norm = norm(x), None
        hidden = ops.linear_swiglu(x, self.w_gate_up, rms=norm.as_rms() if norm is not None else None)
        return ops.linear(hidden, self.w_down, residual=residual, reuse_residual=residual_is_spent)


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts:
    """A mixture of small feed-forwards of which every row uses `top`.

    z = x.Wr^T (32-bit), s = softmax(z) over all router outputs; the `top` outputs with the largest s + correction are
    chosen; a chosen output's weight is s * scale (without the correction, not renormalised). Output e < n_experts is
    the expert Wdown[e] . act(Wup[e] . x) (no biases, act the erf-form gelu); the last n_identity outputs are identity
    experts without tensors whose result is x itself. y = the weighted sum of the chosen outputs, in 32-bit.

    params: width, hidden, n_experts, n_identity, top, scale. tensors, stored [out, in]: router
    (n_experts + n_identity, width), correction (n_experts + n_identity,), up<e> (hidden, width), down<e> (width, hidden).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, f, E, I = params["width"], params["hidden"], params["n_experts"], params.get("n_identity", 0)
        shapes = {"router": (E + I, w), "correction": (E + I,)}
        for e in range(E):
            shapes[f"up{e}"] = (f, w)
            shapes[f"down{e}"] = (w, f)
        return shapes

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.E, self.I, self.top = int(p["n_experts"]), int(p.get("n_identity", 0)), int(p["top"])
        if not 1 <= self.top <= self.E + self.I:
            raise ValueError(f"{self.top} of {self.E} + {self.I} experts")
        self.scale = float(p.get("scale", 1.0))
        self.w_router = to_compute(ops, tensors.of(spec, "router"))
        self.correction = to_gain(ops, tensors.of(spec, "correction"))
        self.w_up = self.w_down = None
        if self.E:
            self.w_up = to_compute(ops, torch.stack([tensors.of(spec, f"up{e}") for e in range(self.E)]))
            self.w_down = to_compute(ops, torch.stack([tensors.of(spec, f"down{e}") for e in range(self.E)]))

    def forward32(self, x, combine=True):
        """combine=False: the experts' results before the sum over a row's choices, for a residual sum that takes it
        (what `ops.routed_experts(..., combine=False)` gives)."""
        ops = self.ops
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.route_topk(z, self.correction, self.scale, self.top)
        return ops.routed_experts(x, ids, weights, self.w_up, self.w_down, "gelu_erf", combine=combine)

    sums_in_residual = True     # forward32(x, combine=False) is there

    def forward(self, x, residual=None):
        y = self.forward32(x)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)


@FEED_FORWARDS.register("gated_dense_biased")
class GatedDenseBiased:
    """y = Wd . (act(Wg . h + bg) * (Wu . h + bu)) + bd. params: width, hidden, act ("gelu_tanh" or "silu"). tensors,
    stored [out, in]: gate, up (hidden, width), down (width, hidden), gate_bias, up_bias (hidden,), down_bias (width,)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, f = params["width"], params["hidden"]
        return {"gate": (f, d), "up": (f, d), "down": (d, f), "gate_bias": (f,), "up_bias": (f,), "down_bias": (d,)}

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        self.ops = ops
        self.act = str(spec.params.get("act", "gelu_tanh"))
        self.hidden = int(spec.params["hidden"])
        # one product for both: the gate's rows, then the other factor's
        self.w_gate_up = to_compute(ops, torch.cat((tensors.of(spec, "gate"), tensors.of(spec, "up")), dim=0))
        self.w_down = to_compute(ops, tensors.of(spec, "down"))
        self.gate_bias, self.up_bias, self.down_bias = (to_gain(ops, tensors.of(spec, k))
                                                        for k in ("gate_bias", "up_bias", "down_bias"))

    def forward_parts(self, rows):
        """(the result without its output bias, 32-bit; the bias): for a block whose sum adds the bias."""
        ops = self.ops
        z = ops.linear(rows, self.w_gate_up, out_dtype=torch.float32)
        hidden = ops.gated_act(z, self.hidden, self.act, gate_bias=self.gate_bias, up_bias=self.up_bias)
        return ops.linear(hidden, self.w_down, out_dtype=torch.float32), self.down_bias

    def forward32(self, rows):
        y, bias = self.forward_parts(rows)
        return y + bias

    def forward(self, x, residual=None):
        y = self.forward32(x)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)


@FEED_FORWARDS.register("input_weighted_experts")
class InputWeightedExperts:
    """A mixture of gated experts in which a chosen expert's weight multiplies what the expert reads, not its result.

    z = Wr . h (32-bit), s = sigmoid(z) (score "sigmoid") or softmax(z); the `top` experts with the largest s are chosen;
    a chosen expert's weight is its s as it is (the chosen weights are not scaled to sum to one);
    y = sum over the chosen of expert_e(s_e * h) with expert(v) = Wd . (act(Wg . v) * (Wu . v)), no biases. Without
    biases Wg . (s h) = s (Wg . h), so the weight is applied to the first product's 32-bit results instead of to a
    rounded copy of the row.

    params: width, hidden, n_experts, top, score, act. tensors, stored [out, in]: router (n_experts, width),
    gate<e>, up<e> (hidden, width), down<e> (width, hidden).
    """
    graph_safe = True
    sums_in_residual = True     # forward_parts leaves the sum over a row's choices to the block's sum

    @classmethod
    def tensor_shapes(cls, params):
        w, f, E = params["width"], params["hidden"], params["n_experts"]
        shapes = {"router": (E, w)}
        for e in range(E):
            shapes[f"gate{e}"] = (f, w)
            shapes[f"up{e}"] = (f, w)
            shapes[f"down{e}"] = (w, f)
        return shapes

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.E, self.top = int(p["n_experts"]), int(p["top"])
        if not 1 <= self.top <= self.E:
            raise ValueError(f"{self.top} of {self.E} experts")
        self.score, self.act = str(p.get("score", "sigmoid")), str(p.get("act", "silu"))
        self.w_router = to_compute(ops, tensors.of(spec, "router"))
        self.w_gate_up = to_compute(ops, torch.stack([torch.cat((tensors.of(spec, f"gate{e}"), tensors.of(spec, f"up{e}")), dim=0)
                                                      for e in range(self.E)]))
        self.w_down = to_compute(ops, torch.stack([tensors.of(spec, f"down{e}") for e in range(self.E)]))

    def forward_parts(self, x):
        """(the experts' results line by (row, choice), for a sum that adds a row's lines; no bias)."""
        ops = self.ops
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.route_topk(z, None, 1.0, self.top, score=self.score)
        return ops.gated_experts(x, ids, weights, self.w_gate_up, self.w_down, self.act), None

    def forward32(self, x):
        chosen, _ = self.forward_parts(x)
        return chosen.results.view(x.shape[0], self.top, -1).sum(1)

    def forward(self, x, residual=None):
        y = self.forward32(x)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)


@FEED_FORWARDS.register("activated_dense")
class ActivatedDense:
    """y = Wd . act(Wu . h), no gate and no biases. params: width, hidden, act ("relu2": the square of relu, or
    "gelu_tanh", "silu"). tensors, stored [out, in]: up (hidden, width), down (width, hidden)."""
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, f = params["width"], params["hidden"]
        return {"up": (f, d), "down": (d, f)}

    def __init__(self, spec, tensors, ops):
        self.ops = ops
        self.act = str(spec.params.get("act", "relu2"))
        self.w_up = to_compute(ops, tensors.of(spec, "up"))
        self.w_down = to_compute(ops, tensors.of(spec, "down"))

    def forward32(self, rows):
        ops = self.ops
        hidden = ops.activate_rows(ops.linear(rows, self.w_up, out_dtype=torch.float32), self.act)
        return ops.linear(hidden, self.w_down, out_dtype=torch.float32)

    def forward(self, x, residual=None):
        y = self.forward32(x)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)


@FEED_FORWARDS.register("grouped_choice_experts")
class GroupedChoiceExperts:
    """A mixture of clamped gated experts whose router first narrows the choice to a few groups of neighbours, with
    identity experts and an optional shared expert behind a gate.

    z = Wr . h (32-bit), s = softmax(z) over all router outputs. The choice looks at s + correction: the outputs form
    `groups` equal runs of neighbours, a group's score is its largest s + correction, only outputs of the `keep` best
    groups can be chosen, and of those the `top` largest s + correction are. A chosen output's weight is its s (without
    the correction) divided by the sum of the chosen s (+ 1e-20). Output e < n_experts is the expert
    Wd[e] . (g sigmoid(1.702 g) (u + 1)) with g = min(Wg[e] . h, limit), u = clamp(Wu[e] . h, -limit, limit), no biases;
    the last n_identity outputs are identity experts without tensors whose result is h itself. A shared expert of the
    same form (sizes and limit of its own) runs for every row and is added times sigmoid(wsg . h), one number a row.
    y = the weighted sum of the chosen + the gated shared expert, in 32-bit.

    params: width, hidden, limit, n_experts, n_identity, top, groups, keep, shared_hidden (0: none), shared_limit.
    tensors, stored [out, in]: router (n_experts + n_identity, width), correction (n_experts + n_identity,), gate<e>,
    up<e> (hidden, width), down<e> (width, hidden), and with a shared expert shared_gate, shared_up (shared_hidden,
    width), shared_down (width, shared_hidden), shared_sg (1, width).
    """
    graph_safe = True
    sums_in_residual = True     # forward32(x, combine=False) is there

    @classmethod
    def tensor_shapes(cls, params):
        w, f, E, I = params["width"], params["hidden"], params["n_experts"], params.get("n_identity", 0)
        shapes = {"router": (E + I, w), "correction": (E + I,)}
        for e in range(E):
            shapes.update({f"gate{e}": (f, w), f"up{e}": (f, w), f"down{e}": (w, f)})
        fs = params.get("shared_hidden", 0)
        if fs:
            shapes.update({"shared_gate": (fs, w), "shared_up": (fs, w), "shared_down": (w, fs), "shared_sg": (1, w)})
        return shapes

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.E, self.I, self.top = int(p["n_experts"]), int(p.get("n_identity", 0)), int(p["top"])
        self.groups, self.keep = int(p.get("groups", 1)), int(p.get("keep", 1))
        n = self.E + self.I
        if not 1 <= self.top <= n or self.groups < 1 or n % self.groups or not 1 <= self.keep <= self.groups \
                or self.top > self.keep * (n // self.groups):
            raise ValueError(f"{self.top} of {self.E} + {self.I} experts in {self.groups} groups of which {self.keep} are kept")
        self.limit, self.F = float(p.get("limit", 0.0)), int(p.get("hidden", 0))
        self.w_router = to_compute(ops, tensors.of(spec, "router"))
        self.correction = to_gain(ops, tensors.of(spec, "correction"))
        self.w_gate_up = self.w_down = None
        if self.E:
            self.w_gate_up = to_compute(ops, torch.stack([torch.cat((tensors.of(spec, f"gate{e}"), tensors.of(spec, f"up{e}")), dim=0)
                                                          for e in range(self.E)]))
            self.w_down = to_compute(ops, torch.stack([tensors.of(spec, f"down{e}") for e in range(self.E)]))
        self.Fs = int(p.get("shared_hidden", 0))
        if self.Fs:
            self.shared_limit = float(p["shared_limit"])
            # one product for the shared expert's gate, its other factor, and the number that gates its result
            self.w_shared_in = to_compute(ops, torch.cat([tensors.of(spec, k) for k in ("shared_gate", "shared_up", "shared_sg")], dim=0))
            self.w_shared_down = to_compute(ops, tensors.of(spec, "shared_down"))

    def forward32(self, x, combine=True):
        """combine=False: the experts' results before the sum over a row's choices (and the shared expert's before its
        gate), as a `ChosenExperts` for a residual sum that takes the sum itself."""
        ops = self.ops
        z = ops.linear(x, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.route_topk(z, self.correction, 1.0, self.top, groups=(self.groups, self.keep), renorm=True)
        chosen = ops.gated_experts(x, ids, weights, self.w_gate_up, self.w_down, "clamped_swish", limit=self.limit,
                                   weigh="output", n_experts=self.E)
        if self.Fs:
            zs = ops.linear(x, self.w_shared_in, out_dtype=torch.float32)
            hidden = ops.gated_act(zs, self.Fs, "clamped_swish", limit=self.shared_limit)
            shared = ops.linear(hidden, self.w_shared_down, out_dtype=torch.float32)
            chosen = chosen._replace(extra=shared, extra_gate=zs[:, 2 * self.Fs:2 * self.Fs + 1])
        return chosen if not combine else ops.combine_experts(chosen)

    def forward(self, x, residual=None):
        y = self.forward32(x)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)
