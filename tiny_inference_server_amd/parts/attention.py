"""Attention mixers."""
from __future__ import annotations

import torch

from .base import MIXERS, build_part, to_compute
from .spec import PagedKvNeed


@MIXERS.register("gqa_attention")
class GqaAttention:
    """Grouped-query attention over a paged cache.

    q = x.Wq, [k|v] = x.Wkv, rotary on q and k, keys and values written into the call's cache plane before
    any row attends, then every row at position p attends the keys [0, p] (or the last `window`) of its
    own request, query head h using key/value head h // group_size; out = attn.Wo (+ residual)
    (reference main_models_new.py:96-136; paged_attention_kernels.py:49).

    params: d_model, n_heads, n_kv_heads, head_dim, window (0: all keys), position (a PartSpec).
    tensors: q (d_model, n_heads*head_dim), kv (d_model, 2*n_kv_heads*head_dim) with the key columns first,
    o (n_heads*head_dim, d_model); all stored [in, out] as the reference applies them (x @ W).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        d, nh, nkv, hd = params["d_model"], params["n_heads"], params["n_kv_heads"], params["head_dim"]
        return {"q": (d, nh * hd), "kv": (d, 2 * nkv * hd), "o": (nh * hd, d)}

    @classmethod
    def cache_need(cls, params):
        return PagedKvNeed(params["n_kv_heads"], params["head_dim"], int(params.get("window", 0)))

    def __init__(self, spec, tensors, ops):
        p = spec.params
        self.ops = ops
        self.n_heads, self.n_kv_heads, self.head_dim = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["head_dim"])
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{self.n_heads} query heads are not a multiple of {self.n_kv_heads} key/value heads")
        self.window = int(p.get("window", 0))
        self.scale = float(p.get("scale", self.head_dim ** -0.5))
        pos = p["position"]
        self.position = build_part(pos, tensors, ops)
        # a position encoding may work on the scores instead of (or beside) rotating queries and keys
        slopes = getattr(self.position, "score_slopes", None)
        self.slopes = slopes(self.n_heads) if slopes is not None else None
        # one projection for q, k and v: rows of the [out, in] matrix are q heads, then k heads, then v heads.
        # Inside every q and k head the rows are put in pair order (the two members of a rotary pair side by side),
        # so that the kernel that makes them can rotate them while they are still in its registers.
        w = torch.cat((tensors.of(spec, "q"), tensors.of(spec, "kv")), dim=1).t()
        _, interleaved = self.position.rotary()
        hd, half = self.head_dim, self.head_dim // 2
        if not interleaved:
            order = torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)
            rows = torch.arange(w.shape[0]).view(-1, hd)
            n_qk = self.n_heads + self.n_kv_heads
            rows[:n_qk] = rows[:n_qk][:, order]
            w = w[rows.reshape(-1)]
        self.w_qkv = to_compute(ops, w)
        self.w_o = to_compute(ops, tensors.of(spec, "o").t())
        self.q_width = self.n_heads * self.head_dim

    fuses_norm = True

    # work lists for the attention kernels are made on the host, once per step and attention shape
    def plan_key(self):
        if not hasattr(self.ops, "plan_attention"):
            return None
        return ("attention", self.n_heads, self.n_kv_heads, self.head_dim, self.window)

    def plan_mode(self, seq_rows):
        mode = getattr(self.ops, "plan_attention_mode", None)
        return mode(seq_rows, self.window) if mode is not None else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_attention(self.n_heads, self.n_kv_heads, self.head_dim, seq_rows, add, mode, self.window)

    def forward(self, x, ctx, residual=None, norm=None):
        ops, b = self.ops, ctx.batch
        rms = None
        if norm is not None:
            if hasattr(norm, "as_rms"):
                rms = norm.as_rms()
            else:
                x = norm(x)
        table, interleaved = self.position.rotary()
        page_size = ctx.plane.shape[3]
        q = ops.qkv_rope(x, self.w_qkv, rms, b.positions, b.write_slots[ctx.group], table, ctx.plane, self.n_heads,
                         self.n_kv_heads, self.head_dim, page_size, interleaved, ctx.writes_cache)
        extra = {"slopes": self.slopes} if self.slopes is not None else {}
        attn = ops.paged_attention(q, ctx.plane, b, ctx.group, self.n_heads, self.n_kv_heads,
                                   self.head_dim, self.window, self.scale, **extra)
        return ops.linear(attn, self.w_o, residual=residual, reuse_residual=ctx.residual_is_spent)


@MIXERS.register("windowed_qknorm_attention")
class WindowedQkNormAttention:
    """Grouped-query softmax attention over the last `window` positions (0: all), with keys and values of different
    sizes. q = x.Wq^T, k = x.Wk^T, v = x.Wv^T; queries and keys are RMS-normed per head (a gain of key_dim entries
    each, shared by the heads), then the first rot_dims channels of each head are rotated in interleaved pairs
    (2i, 2i+1) by position * base^(-2i/rot_dims); values are divided by their root mean square and cached so;
    score = q.k * scale * temp[head]; out = softmax-weighted values of all heads . Wo^T. Norms, angles, scores and
    the softmax are 32-bit.

    params: width, n_heads, n_kv_heads, key_dim, value_dim, window, rot_dims, rot_base, scale, eps. tensors, stored
    [out, in]: q (heads*key_dim, width), k (kv_heads*key_dim, width), v (kv_heads*value_dim, width), q_norm, k_norm
    (key_dim,), temp (heads,), o (width, heads*value_dim).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, H, G, kd, vd = (params[k] for k in ("width", "n_heads", "n_kv_heads", "key_dim", "value_dim"))
        return {"q": (H * kd, w), "k": (G * kd, w), "v": (G * vd, w), "q_norm": (kd,), "k_norm": (kd,), "temp": (H,),
                "o": (w, H * vd)}

    @classmethod
    def cache_need(cls, params):
        return PagedKvNeed(params["n_kv_heads"], params["key_dim"], int(params.get("window", 0)),
                           value_dim=params["value_dim"])

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.H, self.G, self.kd, self.vd = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["key_dim"]), int(p["value_dim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads are not a multiple of {self.G} key/value heads")
        self.window, self.scale, self.eps = int(p.get("window", 0)), float(p["scale"]), float(p["eps"])
        self.rot_dims = int(p.get("rot_dims", 0))
        if self.rot_dims % 2 or self.rot_dims > self.kd:
            raise ValueError(f"{self.rot_dims} rotated channels of a head of {self.kd}: an even number, at most the head")
        i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
        self.freqs = (float(p.get("rot_base", 10000.0)) ** (-2.0 * i / max(1, self.rot_dims))).to(torch.float32).to(ops.device)
        q, k, v = tensors.of(spec, "q"), tensors.of(spec, "k"), tensors.of(spec, "v")
        self.input_rows = torch.cat((q, k, v), dim=0)
        self.k_at, self.v_at = q.shape[0], q.shape[0] + k.shape[0]
        self._w_in = None
        self.q_gain, self.k_gain = to_gain(ops, tensors.of(spec, "q_norm")), to_gain(ops, tensors.of(spec, "k_norm"))
        self.temp = to_gain(ops, tensors.of(spec, "temp"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))
        self.same = self.kd == self.vd        # then the pages have the layout every attention kernel reads

    # the matrix-core kernels' work lists, where keys and values are of one size (see GqaAttention)
    def plan_key(self):
        if not self.same or not hasattr(self.ops, "plan_attention"):
            return None
        return ("attention", self.H, self.G, self.kd, self.window)

    def plan_mode(self, seq_rows):
        mode = getattr(self.ops, "plan_attention_mode", None)
        return mode(seq_rows, self.window) if mode is not None and self.same else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_attention(self.H, self.G, self.kd, seq_rows, add, mode, self.window)

    def core(self, proj, ctx):
        ops, b = self.ops, ctx.batch
        q = ops.attention_prepare(proj, 0, self.k_at, self.v_at, b.positions, b.write_slots[ctx.group], ctx.plane, self.H,
                                  self.G, self.kd, self.vd, ctx.page_size, self.q_gain, self.k_gain, self.temp,
                                  self.freqs, self.rot_dims, self.eps, ctx.writes_cache)
        if self.same:
            return ops.paged_attention(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.window, self.scale)
        return ops.paged_attention_kv(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.vd, ctx.page_size,
                                      self.window, self.scale)

    def forward_projected(self, proj, ctx):
        return self.ops.linear(self.core(proj, ctx), self.w_o, out_dtype=torch.float32)

    def forward(self, x, ctx, residual=None):
        if self._w_in is None:
            self._w_in = to_compute(self.ops, self.input_rows)
        proj = self.ops.linear(x, self._w_in, out_dtype=torch.float32)
        return self.ops.linear(self.core(proj, ctx), self.w_o, residual=residual)


def banded_frequencies(dims: int, base: float, bands=None):
    """base^(-2i/dims) for the pairs i < dims/2 in 64-bit. bands = (factor, low, high, original) slows the long waves:
    with wavelength l = 2 pi / f, a pair with l < original / high keeps f, one with l > original / low turns at
    f / factor, and between the two f is blended with f / factor by s = (original / l - low) / (high - low):
    (1 - s) f / factor + s f."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(1, dims))
    if bands is None:
        return f
    factor, low, high, original = (float(b) for b in bands)
    wave = 2.0 * math.pi / f
    if high == low:
        s = (wave < original / high).to(torch.float64)
    else:
        s = torch.clamp((original / wave - low) / (high - low), 0.0, 1.0)
    blended = (1.0 - s) * f / factor + s * f
    return torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor, blended))


def _rotary_frequencies(ops, dims: int, base: float, bands=None):
    """The rotation's frequencies on the device in 32-bit (computed in 64-bit)."""
    return banded_frequencies(dims, base, bands).to(torch.float32).to(ops.device)


@MIXERS.register("sink_gated_attention")
class SinkGatedAttention:
    """Grouped-query attention over all earlier positions with biased projections, no rotation, a query factor that
    grows with the position, a sink in the softmax and a gate per head.

    q = x.Wq^T + bq, k = x.Wk^T + bk, v = x.Wv^T + bv; the query at position p is multiplied by
    1 + temp_coef * ln(floor((p + 1) / temp_every) + 1); score = q.k * scale; the weights of a row are
    exp(s_j) / (1 + sum_j exp(s_j)) (a sink of score 0 without a value); head h's result is multiplied by
    sigmoid(x.Wg^T)[h]; out = heads . Wo^T. Factors, scores, weights and gates are 32-bit. Keys and values may differ in
    size.

    params: width, n_heads, n_kv_heads, key_dim, value_dim, scale, temp_coef, temp_every (temp_coef 0: no factor),
    sink (default true), head_gate (default true). tensors, stored [out, in]: q (heads*key_dim, width), k
    (kv_heads*key_dim, width), v (kv_heads*value_dim, width), q_bias, k_bias, v_bias, g (heads, width; with head_gate),
    o (width, heads*value_dim).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, H, G, kd, vd = (params[k] for k in ("width", "n_heads", "n_kv_heads", "key_dim", "value_dim"))
        shapes = {"q": (H * kd, w), "k": (G * kd, w), "v": (G * vd, w), "q_bias": (H * kd,), "k_bias": (G * kd,),
                  "v_bias": (G * vd,), "o": (w, H * vd)}
        if params.get("head_gate", True):
            shapes["g"] = (H, w)
        return shapes

    @classmethod
    def cache_need(cls, params):
        return PagedKvNeed(params["n_kv_heads"], params["key_dim"], 0, value_dim=params["value_dim"])

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.H, self.G, self.kd, self.vd = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["key_dim"]), int(p["value_dim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads are not a multiple of {self.G} key/value heads")
        self.scale = float(p["scale"])
        self.temp_coef, self.temp_every = float(p.get("temp_coef", 0.0)), int(p.get("temp_every", 1))
        self.sink, self.head_gate = bool(p.get("sink", True)), bool(p.get("head_gate", True))
        mats = [tensors.of(spec, k) for k in ("q", "k", "v")] + ([tensors.of(spec, "g")] if self.head_gate else [])
        self.k_at = mats[0].shape[0]
        self.v_at = self.k_at + mats[1].shape[0]
        self.g_at = self.v_at + mats[2].shape[0]
        self.w_in = to_compute(ops, torch.cat(mats, dim=0))
        self.q_bias, self.k_bias, self.v_bias = (to_gain(ops, tensors.of(spec, k)) for k in ("q_bias", "k_bias", "v_bias"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))
        self.same = self.kd == self.vd        # then the pages have the layout every attention kernel reads

    # the matrix-core kernels' work lists, where keys and values are of one size (see GqaAttention)
    def plan_key(self):
        if not self.same or not hasattr(self.ops, "plan_attention"):
            return None
        return ("attention", self.H, self.G, self.kd, 0)

    def plan_mode(self, seq_rows):
        mode = getattr(self.ops, "plan_attention_mode", None)
        return mode(seq_rows, 0) if mode is not None and self.same else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_attention(self.H, self.G, self.kd, seq_rows, add, mode, 0)

    def core(self, x, ctx):
        ops, b = self.ops, ctx.batch
        proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
        q = ops.attention_prepare(proj, 0, self.k_at, self.v_at, b.positions, b.write_slots[ctx.group], ctx.plane, self.H,
                                  self.G, self.kd, self.vd, ctx.page_size, write_cache=ctx.writes_cache, value_norm=False,
                                  q_bias=self.q_bias, k_bias=self.k_bias, v_bias=self.v_bias, temp_coef=self.temp_coef,
                                  temp_every=self.temp_every)
        gate = proj[:, self.g_at:self.g_at + self.H] if self.head_gate else None
        if self.same:
            return ops.paged_attention(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, 0, self.scale, sink=self.sink,
                                       gate=gate)
        return ops.paged_attention_kv(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.vd, ctx.page_size, 0,
                                      self.scale, sink=self.sink, gate=gate)

    def forward32(self, x, ctx):
        return self.ops.linear(self.core(x, ctx), self.w_o, out_dtype=torch.float32)

    def forward(self, x, ctx, residual=None):
        return self.ops.linear(self.core(x, ctx), self.w_o, residual=residual)


@MIXERS.register("latent_attention")
class LatentAttention:
    """Softmax attention whose keys and values are made from one low-rank latent per position.

    q = x.Wq^T, a head being [dim unrotated | rot_dim rotated] channels. x.Wdkv^T gives rank + rot_dim channels: the
    first rank, RMS-normed with a gain, are the latent c; the others are one rotated key part that all heads share.
    Head h's unrotated key is Wuk[h] c and its value Wuv[h] c; score = (q_plain . k_plain + q_rot . k_rot) * scale;
    rotation in interleaved pairs of the first rot_dims channels of the rotated parts by position * base^(-2i/rot_dims);
    causal softmax; out = heads . Wo^T.

    Only c and the rotated key part are kept, as one key of rank + rot_dim channels per position whose value is c
    again (transposed, as the attention kernels read values). The products with
    Wuk and Wuv are moved to the query's side of the sums: q_plain . (Wuk[h] c) = (Wuk[h]^T q_plain) . c, so a row's
    query becomes [Wuk[h]^T q_plain | q_rot] against the key [c | k_rot]; and sum_j p_j Wuv[h] c_j = Wuv[h] sum_j p_j c_j,
    so the attention's values are the latents themselves and Wuv[h] is applied to the result.

    params: width, n_heads, dim, rot_dim, value_dim, rank, rot_dims, rot_base, scale, eps. tensors, stored [out, in]:
    q (heads*(dim+rot_dim), width), dkv (rank+rot_dim, width), dkv_norm (rank,), uk (heads*dim, rank),
    uv (heads*value_dim, rank), o (width, heads*value_dim).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, H, D, R, V, C = (params[k] for k in ("width", "n_heads", "dim", "rot_dim", "value_dim", "rank"))
        return {"q": (H * (D + R), w), "dkv": (C + R, w), "dkv_norm": (C,), "uk": (H * D, C), "uv": (H * V, C),
                "o": (w, H * V)}

    @classmethod
    def cache_need(cls, params):
        return PagedKvNeed(1, params["rank"] + params["rot_dim"], 0, value_dim=params["rank"])

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.H, self.D, self.R, self.V, self.C = (int(p[k]) for k in ("n_heads", "dim", "rot_dim", "value_dim", "rank"))
        self.rot_dims = int(p.get("rot_dims", self.R))
        if self.rot_dims % 2 or self.rot_dims > self.R:
            raise ValueError(f"{self.rot_dims} rotated channels of a part of {self.R}: an even number, at most the part")
        self.scale, self.eps = float(p["scale"]), float(p["eps"])
        self.freqs = _rotary_frequencies(ops, self.rot_dims, float(p.get("rot_base", 10000.0)))
        wq, wdkv = tensors.of(spec, "q"), tensors.of(spec, "dkv")
        self.c_at = wq.shape[0]
        self.w_in = to_compute(ops, torch.cat((wq, wdkv), dim=0))
        self.c_gain = to_gain(ops, tensors.of(spec, "dkv_norm"))
        # [heads, rank, dim]: Wuk[h]^T, which takes a head's unrotated query into the latent's space
        self.w_uk_t = to_compute(ops, tensors.of(spec, "uk").view(self.H, self.D, self.C).transpose(1, 2))
        self.w_uv = to_compute(ops, tensors.of(spec, "uv").view(self.H, self.V, self.C))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))

    # the matrix-core kernel's items, where a step brings portions
    def plan_key(self):
        return ("latent", self.H) if hasattr(self.ops, "plan_latent") else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_latent(self.H, seq_rows, add)

    def core(self, x, ctx):
        ops, b = self.ops, ctx.batch
        H, D, R, V, C = self.H, self.D, self.R, self.V, self.C
        proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
        q, q_plain = ops.latent_prepare(proj, 0, self.c_at, b.positions, b.write_slots[ctx.group], ctx.plane, H, D, R, C,
                                        ctx.page_size, self.c_gain, self.freqs, self.rot_dims, self.eps, ctx.writes_cache)
        ops.heads_linear(q_plain, self.w_uk_t, q, C + R)
        mixed = ops.latent_attention(q, ctx.plane, b, ctx.group, H, C + R, C, ctx.page_size, self.scale)
        return ops.heads_linear(mixed, self.w_uv, ops.empty(mixed.shape[0], H * V), V)

    def forward32(self, x, ctx):
        return self.ops.linear(self.core(x, ctx), self.w_o, out_dtype=torch.float32)

    def forward(self, x, ctx, residual=None):
        return self.ops.linear(self.core(x, ctx), self.w_o, residual=residual)


@MIXERS.register("chunked_attention")
class ChunkedAttention:
    """Grouped-query softmax attention inside chunks of positions, with biased projections and keys and values of
    different sizes.

    q = x.Wq^T + bq, k = x.Wk^T + bk, v = x.Wv^T + bv. The whole of a row's queries (all heads side by side) is RMS-normed
    at once with a gain of heads * key_dim entries, and so is the whole of its keys, before rotation. The first rot_dims
    channels of every query and key head are rotated in the pairs (i, i + rot_dims / 2) by position * rot_base^(-2i /
    rot_dims) / rot_factor; the other channels pass. score = q.k * scale. The row at position p sees the keys j <= p
    with floor(j / chunk) = floor(p / chunk): a chunk's edges are multiples of `chunk` in the request, wherever a prompt
    was cut into portions (chunk 0: all j <= p).
    out = softmax-weighted values of all heads . Wo^T + bo. Norms, angles, scores and the softmax are 32-bit.

    params: width, n_heads, n_kv_heads, key_dim, value_dim, scale, eps, rot_dims, rot_base, rot_factor, chunk. tensors,
    stored [out, in]: q (heads*key_dim, width), k (kv_heads*key_dim, width), v (kv_heads*value_dim, width), q_bias,
    k_bias, v_bias, q_norm (heads*key_dim,), k_norm (kv_heads*key_dim,), o (width, heads*value_dim), o_bias (width,).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, H, G, kd, vd = (params[k] for k in ("width", "n_heads", "n_kv_heads", "key_dim", "value_dim"))
        return {"q": (H * kd, w), "k": (G * kd, w), "v": (G * vd, w), "q_bias": (H * kd,), "k_bias": (G * kd,),
                "v_bias": (G * vd,), "q_norm": (H * kd,), "k_norm": (G * kd,), "o": (w, H * vd), "o_bias": (w,)}

    @classmethod
    def cache_need(cls, params):
        # every key is kept: a chunk's keys are found through the same block table as any others
        return PagedKvNeed(params["n_kv_heads"], params["key_dim"], 0, value_dim=params["value_dim"])

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.H, self.G, self.kd, self.vd = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["key_dim"]), int(p["value_dim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads are not a multiple of {self.G} key/value heads")
        self.scale, self.eps, self.chunk = float(p["scale"]), float(p["eps"]), int(p.get("chunk", 0))
        self.rot_dims = int(p.get("rot_dims", 0))
        if self.rot_dims % 2 or self.rot_dims > self.kd or self.chunk < 0:
            raise ValueError(f"{self.rot_dims} rotated channels of a head of {self.kd} (an even number, at most the head), "
                             f"chunks of {self.chunk}")
        factor = float(p.get("rot_factor", 1.0))
        i = torch.arange(self.rot_dims // 2, dtype=torch.float64)
        freqs = float(p.get("rot_base", 10000.0)) ** (-2.0 * i / max(1, self.rot_dims)) / factor
        self.freqs = freqs.to(torch.float32).to(ops.device)
        mats = [tensors.of(spec, k) for k in ("q", "k", "v")]
        self.k_at = mats[0].shape[0]
        self.v_at = self.k_at + mats[1].shape[0]
        self.w_in = to_compute(ops, torch.cat(mats, dim=0))
        self.q_bias, self.k_bias, self.v_bias, self.o_bias = (to_gain(ops, tensors.of(spec, k))
                                                              for k in ("q_bias", "k_bias", "v_bias", "o_bias"))
        self.q_gain, self.k_gain = to_gain(ops, tensors.of(spec, "q_norm")), to_gain(ops, tensors.of(spec, "k_norm"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))
        self.same = self.kd == self.vd        # then the pages have the layout every attention kernel reads
        self.span = -self.chunk               # how the attention kernels for one size are told of chunks: a negative window

    # the matrix-core kernels' work lists, where keys and values are of one size (see GqaAttention)
    def plan_key(self):
        if not self.same or not hasattr(self.ops, "plan_attention"):
            return None
        return ("attention", self.H, self.G, self.kd, self.span)

    def plan_mode(self, seq_rows):
        mode = getattr(self.ops, "plan_attention_mode", None)
        return mode(seq_rows, self.span) if mode is not None and self.same else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_attention(self.H, self.G, self.kd, seq_rows, add, mode, self.span)

    def core(self, x, ctx):
        ops, b = self.ops, ctx.batch
        proj = ops.linear(x, self.w_in, out_dtype=torch.float32)
        q = ops.attention_prepare(proj, 0, self.k_at, self.v_at, b.positions, b.write_slots[ctx.group], ctx.plane, self.H,
                                  self.G, self.kd, self.vd, ctx.page_size, q_gain=self.q_gain, k_gain=self.k_gain,
                                  freqs=self.freqs, rot_dims=self.rot_dims, eps=self.eps, write_cache=ctx.writes_cache,
                                  value_norm=False, q_bias=self.q_bias, k_bias=self.k_bias, v_bias=self.v_bias,
                                  whole_norm=True, pair_half=True)
        if self.same:
            return ops.paged_attention(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.span, self.scale)
        return ops.paged_attention_kv(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.vd, ctx.page_size, 0,
                                      self.scale, chunk=self.chunk)

    def forward_parts(self, x, ctx):
        """(the result without its output bias, 32-bit; the bias): for a block whose sum adds the bias."""
        return self.ops.linear(self.core(x, ctx), self.w_o, out_dtype=torch.float32), self.o_bias

    def forward32(self, x, ctx):
        y, bias = self.forward_parts(x, ctx)
        return y + bias

    def forward(self, x, ctx, residual=None):
        y = self.forward32(x, ctx)
        if residual is not None:
            y = y + residual.to(torch.float32)
        return y.to(self.ops.dtype)


@MIXERS.register("sigmoid_mixed_attention")
class SigmoidMixedAttention:
    """Grouped-query attention inside chunks of positions whose weights are sigmoids, not a softmax, and are mixed across
    the heads before they meet the values.

    q = x.Wq^T + bq, k = x.Wk^T + bk, v = x.Wv^T + bv. The first rot_dims channels of every query and key head are
    rotated in the pairs (i, i + rot_dims / 2) by position * f_i (f from `banded_frequencies`); the other channels pass.
    s = q.k * scale, then s <- softcap * tanh(s / softcap) (softcap 0: as it is). The row at position p sees the keys
    j <= p with floor(j / chunk) = floor(p / chunk) (chunk 0: all j <= p); a seen key's weight for head g is
    w_g = sigmoid(s + head_bias[g]), each key on its own. Head h then uses sum_g talk[h, g] * w_g on the values of its
    own key/value head; out = heads . Wo^T. Angles, scores and weights are 32-bit.

    params: width, n_heads, n_kv_heads, key_dim, value_dim, scale, softcap, chunk, rot_dims, rot_base, rot_bands
    ((factor, low, high, original) or None). tensors, stored [out, in]: q (heads*key_dim, width), k (kv_heads*key_dim,
    width), v (kv_heads*value_dim, width), q_bias, k_bias, v_bias, head_bias (heads,), talk (heads, heads),
    o (width, heads*value_dim).
    """
    graph_safe = True

    @classmethod
    def tensor_shapes(cls, params):
        w, H, G, kd, vd = (params[k] for k in ("width", "n_heads", "n_kv_heads", "key_dim", "value_dim"))
        return {"q": (H * kd, w), "k": (G * kd, w), "v": (G * vd, w), "q_bias": (H * kd,), "k_bias": (G * kd,),
                "v_bias": (G * vd,), "head_bias": (H,), "talk": (H, H), "o": (w, H * vd)}

    @classmethod
    def cache_need(cls, params):
        # every key is kept: a chunk's keys are found through the same block table as any others
        return PagedKvNeed(params["n_kv_heads"], params["key_dim"], 0, value_dim=params["value_dim"])

    def __init__(self, spec, tensors, ops):
        from .base import to_gain
        p = spec.params
        self.ops = ops
        self.H, self.G, self.kd, self.vd = int(p["n_heads"]), int(p["n_kv_heads"]), int(p["key_dim"]), int(p["value_dim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads are not a multiple of {self.G} key/value heads")
        self.scale, self.softcap, self.chunk = float(p["scale"]), float(p.get("softcap", 0.0)), int(p.get("chunk", 0))
        self.rot_dims = int(p.get("rot_dims", 0))
        if self.rot_dims % 2 or self.rot_dims > self.kd or self.chunk < 0 or self.softcap < 0:
            raise ValueError(f"{self.rot_dims} rotated channels of a head of {self.kd} (an even number, at most the head), "
                             f"chunks of {self.chunk}, a cap of {self.softcap}")
        self.freqs = _rotary_frequencies(ops, self.rot_dims, float(p.get("rot_base", 10000.0)), p.get("rot_bands"))
        mats = [tensors.of(spec, k) for k in ("q", "k", "v")]
        self.input_rows = torch.cat(mats, dim=0)        # as stored: a block may fuse them into a wider product
        self.k_at = mats[0].shape[0]
        self.v_at = self.k_at + mats[1].shape[0]
        self._w_in = None
        self.q_bias, self.k_bias, self.v_bias = (to_gain(ops, tensors.of(spec, k)) for k in ("q_bias", "k_bias", "v_bias"))
        self.head_bias = to_gain(ops, tensors.of(spec, "head_bias"))
        self.talk = to_gain(ops, tensors.of(spec, "talk"))
        self.w_o = to_compute(ops, tensors.of(spec, "o"))

    # the matrix-core kernel's items (tiles of up to 16 rows of one request), where a step brings portions
    def plan_key(self):
        return ("row_tiles", 16) if hasattr(self.ops, "plan_row_tiles") else None

    def plan_rows(self, seq_rows, add, mode=None):
        return self.ops.plan_row_tiles(seq_rows, add)

    def core(self, proj, ctx):
        ops, b = self.ops, ctx.batch
        q = ops.attention_prepare(proj, 0, self.k_at, self.v_at, b.positions, b.write_slots[ctx.group], ctx.plane, self.H,
                                  self.G, self.kd, self.vd, ctx.page_size, freqs=self.freqs, rot_dims=self.rot_dims,
                                  write_cache=ctx.writes_cache, value_norm=False, q_bias=self.q_bias, k_bias=self.k_bias,
                                  v_bias=self.v_bias, pair_half=True)
        return ops.mixed_sigmoid_attention(q, ctx.plane, b, ctx.group, self.H, self.G, self.kd, self.vd, ctx.page_size,
                                           self.chunk, self.scale, self.softcap, self.head_bias, self.talk)

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
