"""Recurrent mixers: a matrix state per head and request, kept in 32-bit in the request's state slot."""
from __future__ import annotations

import torch

from .base import MIXERS, to_compute, to_gain
from .spec import StateNeed


def state_floats(kind: str, n_heads: int, dim: int, vdim: int) -> int:
    """32-bit floats of one request's state: S [heads, dim, vdim]; kind "gated_max" also keeps its normaliser
    n [dim] and running maximum per head, once per block of 16 value channels (a workgroup of the scan kernel)."""
    blocks = -(-vdim // 16)
    return n_heads * dim * vdim + (n_heads * blocks * (dim + 1) if kind == "gated_max" else 0)


class _MatrixStateMixer:
    """What the two mixers below share: stacked input matrices, the output matrix, the ways in."""
    graph_safe = True

    def _stack(self, spec, tensors, keys):
        """The input matrices under `keys`, stacked as stored; returns their first columns in the product."""
        mats = [tensors.of(spec, k) for k in keys]
        self.input_rows = torch.cat(mats, dim=0)
        offs, at = {}, 0
        for k, m in zip(keys, mats):
            offs[k] = at
            at += m.shape[0]
        self._w_in = None
        return offs

    def forward_projected(self, proj, ctx):
        """From this mixer's columns of a 32-bit input product to its result in 32-bit."""
        return self.ops.linear(self.core(proj, ctx), self.w_o, out_dtype=torch.float32)

    def forward(self, x, ctx, residual=None):
        if self._w_in is None:
            self._w_in = to_compute(self.ops, self.input_rows)
        proj = self.ops.linear(x, self._w_in, out_dtype=torch.float32)
        return self.ops.linear(self.core(proj, ctx), self.w_o, residual=residual)


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(_MatrixStateMixer):
    """Per head S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, with q = x.Wq^T / sqrt(dim), k = x.Wk^T,
    v = x.Wv^T and a decay per key channel a = sigmoid((x.Wa1^T).Wa2^T + b)^(1/tau). Each head's o is RMS-normed over
    its value channels (gain of vdim entries, shared by the heads), multiplied by silu(x.Wg^T) and projected by Wo.
    Decays, state and sums are 32-bit; the state starts at zero.

    params: width, n_heads, dim, vdim, tau, rank, eps. tensors, stored [out, in]: q, k (heads*dim, width), v, g
    (heads*vdim, width), o (width, heads*vdim), norm (vdim,), a1 (rank, width), a2 (heads*dim, rank), a2_bias.
    """

    @classmethod
    def tensor_shapes(cls, params):
        w, H, D, V, r = (params[k] for k in ("width", "n_heads", "dim", "vdim", "rank"))
        return {"q": (H * D, w), "k": (H * D, w), "v": (H * V, w), "g": (H * V, w), "o": (w, H * V), "norm": (V,),
                "a1": (r, w), "a2": (H * D, r), "a2_bias": (H * D,)}

    @classmethod
    def cache_need(cls, params):
        return StateNeed((state_floats("decay", params["n_heads"], params["dim"], params["vdim"]),), "float32")

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.H, self.D, self.V, self.rank = int(p["n_heads"]), int(p["dim"]), int(p["vdim"]), int(p["rank"])
        self.tau, self.eps = float(p["tau"]), float(p["eps"])
        self.at = self._stack(spec, tensors, ("q", "k", "v", "g", "a1"))
        self.w_a2 = to_gain(ops, tensors.of(spec, "a2"))
        self.a2_bias = to_gain(ops, tensors.of(spec, "a2_bias"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))

    def core(self, proj, ctx):
        ops, at, H, D, V = self.ops, self.at, self.H, self.D, self.V
        decay = ops.lowrank_decay(proj[:, at["a1"]:at["a1"] + self.rank], self.w_a2, self.a2_bias, self.tau)
        o = ops.state_scan("decay", proj, at["q"], at["k"], at["v"], D ** -0.5, ctx.state, ctx.batch, H, D, V,
                           decay=decay)
        return ops.head_norm_gate(o, proj[:, at["g"]:at["g"] + H * V], self.norm_gain, H, V, self.eps, "silu")


@MIXERS.register("matrix_memory")
class MatrixMemory(_MatrixStateMixer):
    """A matrix memory with exponential gating. Per head, with log gates i = cap tanh((x.Wi^T + bi) / cap) and
    f = log sigmoid(cap tanh((x.Wf^T + bf) / cap)) and a running maximum m (which starts at 0):
    m_t = max(f + m_(t-1), i); S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T; n_t alike with k alone;
    o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6), q = x.Wq^T / sqrt(dim). Each head's o is divided by its root
    mean square, the heads side by side are multiplied by a gain and by sigmoid(x.Wg^T), then projected by Wo.
    Gates, state and sums are 32-bit; S and n start at zero.

    params: width, n_heads, dim, vdim, gate_cap, eps. tensors, stored [out, in]: q, k (heads*dim, width), v, g
    (heads*vdim, width), o (width, heads*vdim), norm (heads*vdim,), i, f (heads, width), i_bias, f_bias (heads,).
    """

    @classmethod
    def tensor_shapes(cls, params):
        w, H, D, V = (params[k] for k in ("width", "n_heads", "dim", "vdim"))
        return {"q": (H * D, w), "k": (H * D, w), "v": (H * V, w), "g": (H * V, w), "o": (w, H * V), "norm": (H * V,),
                "i": (H, w), "f": (H, w), "i_bias": (H,), "f_bias": (H,)}

    @classmethod
    def cache_need(cls, params):
        return StateNeed((state_floats("gated_max", params["n_heads"], params["dim"], params["vdim"]),), "float32")

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.H, self.D, self.V = int(p["n_heads"]), int(p["dim"]), int(p["vdim"])
        self.cap, self.eps = float(p["gate_cap"]), float(p["eps"])
        self.at = self._stack(spec, tensors, ("q", "k", "v", "g", "i", "f"))
        self.i_bias = to_gain(ops, tensors.of(spec, "i_bias"))
        self.f_bias = to_gain(ops, tensors.of(spec, "f_bias"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))

    def core(self, proj, ctx):
        ops, at, H, D, V = self.ops, self.at, self.H, self.D, self.V
        o = ops.state_scan("gated_max", proj, at["q"], at["k"], at["v"], D ** -0.5, ctx.state, ctx.batch, H, D, V,
                           i_off=at["i"], f_off=at["f"], bias_i=self.i_bias, bias_f=self.f_bias, cap=self.cap)
        return ops.head_norm_gate(o, proj[:, at["g"]:at["g"] + H * V], self.norm_gain, H, V, self.eps, "sigmoid")


@MIXERS.register("lightning_attention")
class LightningAttention(_MatrixStateMixer):
    """Linear attention with one fixed decay per head: q = silu(x.Wq^T), k = silu(x.Wk^T), v = silu(x.Wv^T); per head
    S_t = decay[h] S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, with no other scale. The heads side by side are RMS-normed
    together with a gain, multiplied by sigmoid(x.Wg^T) and projected by Wo. State and sums are 32-bit; the state
    starts at zero.

    params: width, n_heads, dim, vdim, decay (one number per head), eps. tensors, stored [out, in]: q, k
    (heads*dim, width), v, g (heads*vdim, width), o (width, heads*vdim), norm (heads*vdim,).
    """

    @classmethod
    def tensor_shapes(cls, params):
        w, H, D, V = (params[k] for k in ("width", "n_heads", "dim", "vdim"))
        return {"q": (H * D, w), "k": (H * D, w), "v": (H * V, w), "g": (H * V, w), "o": (w, H * V), "norm": (H * V,)}

    @classmethod
    def cache_need(cls, params):
        return StateNeed((state_floats("decay", params["n_heads"], params["dim"], params["vdim"]),), "float32")

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.H, self.D, self.V = int(p["n_heads"]), int(p["dim"]), int(p["vdim"])
        self.eps = float(p["eps"])
        decay = [float(a) for a in p["decay"]]
        if len(decay) != self.H:
            raise ValueError(f"{len(decay)} decays for {self.H} heads")
        # the scan takes a decay per key channel and row: one line that every row reads
        self.decay = torch.tensor(decay, dtype=torch.float64).repeat_interleave(self.D).to(torch.float32).to(ops.device).view(1, -1)
        self.at = self._stack(spec, tensors, ("q", "k", "v", "g"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))

    def core(self, proj, ctx):
        ops, at, H, D, V = self.ops, self.at, self.H, self.D, self.V
        ops.activate32(proj[:, :at["g"]], "silu")           # q, k and v lie first, side by side
        o = ops.state_scan("decay", proj, at["q"], at["k"], at["v"], 1.0, ctx.state, ctx.batch, H, D, V,
                           decay=self.decay.expand(proj.shape[0], H * D))
        return ops.head_norm_gate(o, proj[:, at["g"]:at["g"] + H * V], self.norm_gain, 1, H * V, self.eps, "sigmoid")

    def forward32(self, x, ctx):
        if self._w_in is None:
            self._w_in = to_compute(self.ops, self.input_rows)
        return self.forward_projected(self.ops.linear(x, self._w_in, out_dtype=torch.float32), ctx)


@MIXERS.register("selective_state_space")
class SelectiveStateSpace:
    """A selective state-space mixer with a scalar decay per head.

    One input product, laid out [z: inner | x: inner | B: groups*state | C: groups*state | dt: heads] with
    inner = heads * vdim. The columns x, B and C go, channel by channel, through a short convolution over the
    row and the taps - 1 rows before it (a bias; nothing before a request's first row) and silu. dt = softplus(dt + dt_bias). Per head h, which
    reads the B and C of group h // (heads / groups), with the state S of state x vdim numbers:
    S_t = exp(-exp(a_log[h]) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + skip[h] x_t. The heads side by side are
    multiplied by silu(z), then RMS-normed in norm_groups equal parts (each by its own root mean square) with a gain,
    and projected by Wo. Everything between the convolution and the norm is 32-bit.

    A request's state line holds S [heads, state, vdim] and after it the convolution's last taps - 1 inputs
    [taps - 1, channels]; a line that is taken anew is all zeros.

    params: width, n_heads, vdim, state, groups, taps, norm_groups, eps. tensors: in (2 inner + 2 groups*state + heads,
    width) and o (width, inner), stored [out, in]; conv (inner + 2 groups*state, taps), conv_bias, dt_bias (heads,),
    a_log (heads,), skip (heads,), norm (inner,).
    """
    graph_safe = True

    @classmethod
    def _sizes(cls, params):
        H, P, N, G, K = (int(params[k]) for k in ("n_heads", "vdim", "state", "groups", "taps"))
        return H, P, N, G, K, H * P, H * P + 2 * G * N

    @classmethod
    def tensor_shapes(cls, params):
        H, P, N, G, K, inner, C = cls._sizes(params)
        w = params["width"]
        return {"in": (inner + C + H, w), "conv": (C, K), "conv_bias": (C,), "dt_bias": (H,), "a_log": (H,), "skip": (H,),
                "norm": (inner,), "o": (w, inner)}

    @classmethod
    def cache_need(cls, params):
        H, P, N, G, K, inner, C = cls._sizes(params)
        return StateNeed((state_floats("decay", H, N, P) + (K - 1) * C,), "float32")

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.H, self.P, self.N, self.G, self.K, self.inner, self.C = self._sizes(p)
        self.parts, self.eps = int(p.get("norm_groups", 1)), float(p["eps"])
        if self.H % self.G or self.inner % self.parts:
            raise ValueError(f"{self.H} heads over {self.G} groups, a norm of {self.inner} channels in {self.parts} parts")
        self.w_in = to_compute(ops, tensors.of(spec, "in"))
        self.taps = to_gain(ops, tensors.of(spec, "conv"))
        self.tap_bias = to_gain(ops, tensors.of(spec, "conv_bias"))
        self.dt_bias = to_gain(ops, tensors.of(spec, "dt_bias"))
        self.neg_a = -torch.exp(to_gain(ops, tensors.of(spec, "a_log")))          # the decay's rate per head, 32-bit
        self.skip = to_gain(ops, tensors.of(spec, "skip"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))
        self.conv_at = state_floats("decay", self.H, self.N, self.P)              # where the line's convolution inputs start

    def core(self, proj, ctx):
        ops, b = self.ops, ctx.batch
        H, P, N, G, inner, C = self.H, self.P, self.N, self.G, self.inner, self.C
        u = ops.conv_prepare(proj, inner, inner + C, self.taps, self.tap_bias, self.dt_bias, self.neg_a, ctx.state,
                             self.conv_at, b, H, P)
        ops.conv_state_update(proj, inner, C, self.K, ctx.state, self.conv_at, b)      # after the rows have read the line
        # the scan's keys are B, its queries C, its values x * dt, its decay exp(-exp(a_log) dt), one per head and row
        y = ops.state_scan("decay", u, inner + G * N, inner, C, 1.0, ctx.state, b, H, N, P, decay=u[:, C + inner:],
                           qk_group=H // G, decay_per_head=True)
        return ops.gated_group_norm(y, u[:, :inner], self.skip, P, proj[:, :inner], self.norm_gain, self.eps, self.parts)

    def forward32(self, x, ctx):
        proj = self.ops.linear(x, self.w_in, out_dtype=torch.float32)
        return self.ops.linear(self.core(proj, ctx), self.w_o, out_dtype=torch.float32)

    def forward(self, x, ctx, residual=None):
        proj = self.ops.linear(x, self.w_in, out_dtype=torch.float32)
        return self.ops.linear(self.core(proj, ctx), self.w_o, residual=residual)


def delta_state_floats(n_heads: int, dim: int, vdim: int) -> int:
    """32-bit floats of a delta rule's matrix state in a request's line: [heads, blocks of 16 value channels, dim, 16],
    the value channels rounded up to whole blocks (a block is what one workgroup of the walk owns: one run of memory)."""
    return n_heads * -(-vdim // 16) * dim * 16


@MIXERS.register("gated_delta_rule")
class GatedDeltaRule:
    """A matrix state per head that is corrected towards each new value instead of only added to, with a decay per key
    channel.

    q = x.Wq^T and k = x.Wk^T (qk_heads x dim), v = x.Wv^T (heads x vdim), no biases; head h reads the q and k of
    qk head h // (heads / qk_heads). q, k and v go, channel by channel, through a short convolution over the row and
    the taps - 1 rows before it (no bias; nothing before a request's first row) and silu. q and k are then made unit
    vectors per head, x / sqrt(sum x^2 + 1e-6), and q is multiplied by dim^(-1/2). beta = sigmoid(x.Wb^T), one per head.
    a = exp(-exp(a_log[h]) * softplus((x.Wa1^T).Wa2^T + dt_bias)), one per head and key channel. Per head and row:
    S <- diag(a) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q (the row reads what it has just written).
    Each head's o is divided by its root mean square over vdim (eps under the root), times a gain of vdim entries that
    the heads share, times sigmoid((x.Wg1^T).Wg2^T); then Wo. Everything between the convolution and the gate is 32-bit.

    A request's state line holds S as [heads, blocks of 16 value channels, dim, 16] (`delta_state_floats`) and after it
    the convolution's last taps - 1 inputs [taps - 1, channels]; a line that is taken anew is all zeros.

    params: width, n_heads, qk_heads, dim, vdim, taps, decay_rank, gate_rank, eps. tensors, stored [out, in]: q, k
    (qk_heads*dim, width), v (heads*vdim, width), q_conv, k_conv, v_conv ([channels, taps], the last column weighs the
    row itself), b (heads, width), a_log (heads,), a1 (decay_rank, width), a2 (heads*dim, decay_rank), dt_bias
    (heads*dim,), g1 (gate_rank, width), g2 (heads*vdim, gate_rank), norm (vdim,), o (width, heads*vdim).
    """
    graph_safe = True

    @classmethod
    def _sizes(cls, params):
        H, G, D, V, K = (int(params[k]) for k in ("n_heads", "qk_heads", "dim", "vdim", "taps"))
        return H, G, D, V, K, 2 * G * D + H * V

    @classmethod
    def tensor_shapes(cls, params):
        H, G, D, V, K, C = cls._sizes(params)
        w, ra, rg = params["width"], params["decay_rank"], params["gate_rank"]
        return {"q": (G * D, w), "k": (G * D, w), "v": (H * V, w), "q_conv": (G * D, K), "k_conv": (G * D, K),
                "v_conv": (H * V, K), "b": (H, w), "a_log": (H,), "a1": (ra, w), "a2": (H * D, ra), "dt_bias": (H * D,),
                "g1": (rg, w), "g2": (H * V, rg), "norm": (V,), "o": (w, H * V)}

    @classmethod
    def cache_need(cls, params):
        H, G, D, V, K, C = cls._sizes(params)
        floats = delta_state_floats(H, D, V) + (K - 1) * C
        return StateNeed((floats + -floats % 4,), "float32")        # (lines start 16 bytes aligned)

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.H, self.G, self.D, self.V, self.K, self.C = self._sizes(p)
        if self.H % self.G:
            raise ValueError(f"{self.H} heads are not a multiple of {self.G} query/key heads")
        self.eps = float(p["eps"])
        self.ra, self.rg = int(p["decay_rank"]), int(p["gate_rank"])
        keys = ("q", "k", "v", "b", "a1", "g1")
        mats = [tensors.of(spec, k) for k in keys]
        self.input_rows = torch.cat(mats, dim=0)        # as stored: a block may fuse them into a wider product
        self.at, at = {}, 0
        for k, m in zip(keys, mats):
            self.at[k] = at
            at += m.shape[0]
        self._w_in = None
        self.taps = to_gain(ops, torch.cat([tensors.of(spec, k) for k in ("q_conv", "k_conv", "v_conv")], dim=0))
        self.rate = torch.exp(to_gain(ops, tensors.of(spec, "a_log")))          # the decay's rate per head, 32-bit
        self.w_a2, self.dt_bias = to_gain(ops, tensors.of(spec, "a2")), to_gain(ops, tensors.of(spec, "dt_bias"))
        self.w_g2 = to_gain(ops, tensors.of(spec, "g2"))
        self.norm_gain = to_gain(ops, tensors.of(spec, "norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))
        self.conv_at = delta_state_floats(self.H, self.D, self.V)                # where the line's convolution inputs start

    def core(self, proj, ctx):
        ops, b, at = self.ops, ctx.batch, self.at
        H, G, D, V, C = self.H, self.G, self.D, self.V, self.C
        # u: the convolved q (unit, scaled), k (unit), v side by side, then beta
        u = ops.delta_prepare(proj, at["q"], at["b"], self.taps, ctx.state, self.conv_at, b, H, G, D, V)
        ops.conv_state_update(proj, at["q"], C, self.K, ctx.state, self.conv_at, b)      # after the rows have read the line
        decay = ops.lowrank_act(proj[:, at["a1"]:at["a1"] + self.ra], self.w_a2, self.dt_bias, "exp_softplus",
                                rate=self.rate, group=D)
        o = ops.delta_scan(u, 0, G * D, 2 * G * D, C, decay, ctx.state, b, H, G, D, V)
        gate = ops.lowrank_act(proj[:, at["g1"]:at["g1"] + self.rg], self.w_g2, None, "none")
        return ops.head_norm_gate(o, gate, self.norm_gain, H, V, self.eps, "sigmoid")

    def forward_projected(self, proj, ctx):
        """From this mixer's columns of a 32-bit input product to its result in 32-bit."""
        return self.ops.linear(self.core(proj, ctx), self.w_o, out_dtype=torch.float32)

    def forward32(self, x, ctx):
        if self._w_in is None:
            self._w_in = to_compute(self.ops, self.input_rows)
        return self.forward_projected(self.ops.linear(x, self._w_in, out_dtype=torch.float32), ctx)

    def forward(self, x, ctx, residual=None):
        y = self.forward32(x, ctx)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)
