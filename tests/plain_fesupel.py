"""The Fesupel decoder written out plainly: float64, whole sequences, one function per mechanism.

Nothing here is shared with the engine: no cache, no pages, no state slots, no kernels. A sequence goes in as a list of
token ids, logits for every position come out (and, if asked, the stream after every layer). Tests compare the engine
with this.

The design: x = E[token] * scale; every layer x <- x + N1b(mixer(N1(x))), x <- x + N2b(ff(N2(x))) with RMS norms before
and after each sublayer, then x <- x + rms(Wp (gelu_tanh(Wg x) * side[token])) * gain from the layer's columns of a side
table. The mixer is two mixers on the same rows whose results are RMS-normed and averaged: attention inside chunks of
positions whose weights are sigmoids (no softmax) mixed across heads, and a gated delta rule with a decay per key
channel. The feed-forward is W2 relu(W1 h)^2, or a mixture of clamped gated experts with grouped choice, identity
experts and a gated shared expert, or absent. logits = head N(x).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, gain, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ---- rotation ---------------------------------------------------------------------------------------------------------

def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims); with `scaling` (factor, low, high, original) long waves are slowed: a wave longer than
    original/low turns `factor` times slower, one shorter than original/high is kept, between them the two are blended
    by how far original/wavelength lies between low and high."""
    f = base ** (-2.0 * torch.arange(dims // 2, dtype=F64) / dims)
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for i in range(f.numel()):
        wave = 2.0 * math.pi / float(f[i])
        if wave < orig / high:
            continue
        if wave > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wave - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def rotate_half(x, positions, dims, freqs):
    """x: [T, heads, D]. Channel i < dims/2 is paired with channel i + dims/2; channels from dims on stay."""
    if not dims:
        return x
    half = dims // 2
    ang = positions.to(F64).view(-1, 1, 1) * freqs.view(1, 1, half)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat((u * c - v * s, v * c + u * s, x[..., dims:]), dim=-1)


# ---- the left mixer: attention with sigmoid weights mixed across heads ----------------------------------------------

def chunk_mask(T, size):
    """[T, T] booleans: row i sees column j if j <= i and both lie in the same chunk of `size` positions (0: any)."""
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    seen = j <= i
    if size:
        seen = seen & (i // size == j // size)
    return seen


def sigmoid_weights(q, k, scale, softcap, head_bias, mask):
    """q [T, H, D], k [T, G, D] -> weights [H, T, T]: sigmoid(cap(q.k * scale) + bias[h]) where seen, 0 elsewhere."""
    H, G = q.shape[1], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    if softcap:
        s = softcap * torch.tanh(s / softcap)
    w = torch.sigmoid(s + head_bias.view(-1, 1, 1))
    return w * mask.to(F64)


def mix_heads(weights, talk):
    """weights [H, T, T], talk [H, H]: head h's new weights are sum_g talk[h, g] * weights[g]."""
    return torch.einsum("hg,gij->hij", talk, weights)


def left_mixer(h, w, pre, m, positions):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].t() + w[pre + "q.b"]).view(T, H, D)
    k = (h @ w[pre + "k"].t() + w[pre + "k.b"]).view(T, G, D)
    v = (h @ w[pre + "v"].t() + w[pre + "v.b"]).view(T, G, V)
    rot = m.get("rot") or {}
    dims = int(rot.get("dims", 0))
    if dims:
        f = rotary_frequencies(dims, float(rot["base"]), rot.get("scaling"))
        q, k = rotate_half(q, positions, dims, f), rotate_half(k, positions, dims, f)
    mask = chunk_mask(T, int((m.get("mask") or {}).get("size", 0)))
    p = sigmoid_weights(q, k, float(m["scale"]), float(m.get("softcap", 0.0)), w[pre + "pb"], mask)
    p = mix_heads(p, w[pre + "talk"])
    vv = v.repeat_interleave(H // G, dim=1)                  # head h reads the values of its own key/value head
    o = torch.einsum("hij,jhv->ihv", p, vv).reshape(T, H * V)
    return o @ w[pre + "o"].t()


# ---- the right mixer: a gated delta rule ------------------------------------------------------------------------------

def causal_conv(x, taps):
    """x [T, C], taps [C, K]: y_t = sum_j taps[:, K-1-j] * x_(t-j), nothing before the first row."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        y[j:] += x[:T - j] * taps[:, K - 1 - j] if j else x * taps[:, K - 1]
    return y


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """q, k, decay [T, H, D], v [T, H, V], beta [T, H]. Per head, token by token:
    S <- decay * S (row by row); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, D = q.shape
    V = v.shape[2]
    S = torch.zeros(H, D, V, dtype=F64)
    out = torch.zeros(T, H, V, dtype=F64)
    for t in range(T):
        S = S * decay[t].unsqueeze(-1)
        u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t].unsqueeze(-1) * u.unsqueeze(1)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def right_mixer(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ w[pre + "q"].t(), w[pre + "q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ w[pre + "k"].t(), w[pre + "k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ w[pre + "v"].t(), w[pre + "v.conv"])).view(T, H, V)
    q, k = unit(q) * D ** -0.5, unit(k)
    q, k = q.repeat_interleave(H // G, dim=1), k.repeat_interleave(H // G, dim=1)
    beta = torch.sigmoid(h @ w[pre + "b"].t())
    step = softplus((h @ w[pre + "a1"].t()) @ w[pre + "a2"].t() + w[pre + "dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w[pre + "A_log"]).view(1, H, 1) * step)
    o = delta_rule(q, k, v, beta, decay)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[pre + "norm"]
    gate = torch.sigmoid((h @ w[pre + "g1"].t()) @ w[pre + "g2"].t()).view(T, H, V)
    return (o * gate).reshape(T, H * V) @ w[pre + "o"].t()


def parallel_mixer(h, w, pre, m, eps, positions):
    left = left_mixer(h, w, pre + "left.", m["left"], positions)
    right = right_mixer(h, w, pre + "right.", m["right"], eps)
    return 0.5 * (rms_norm(left, w[pre + "left.out"], eps) + rms_norm(right, w[pre + "right.out"], eps))


# ---- feed-forwards ----------------------------------------------------------------------------------------------------

def dense_ff(h, w, pre):
    return torch.relu(h @ w[pre + "up"].t()) ** 2 @ w[pre + "down"].t()


def clamped_expert(h, w, pre, limit):
    g = torch.clamp(h @ w[pre + "gate"].t(), max=limit)
    u = torch.clamp(h @ w[pre + "up"].t(), min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].t()


def choose(scores, correction, top, n_groups, keep):
    """scores [T, N] -> (ids [T, top], weights [T, top], margins): the `top` largest of scores + correction among the
    `keep` groups (of `n_groups` equal runs of neighbours) whose largest corrected score is largest; the weights are the
    plain scores of the chosen, divided by their sum."""
    T, N = scores.shape
    c = scores + correction
    margins = []
    if n_groups > 1 and keep < n_groups:
        per = N // n_groups
        best = c.view(T, n_groups, per).max(-1).values
        order = torch.sort(best, dim=-1, descending=True, stable=True)
        margins += [float(x) for x in (order.values[:, keep - 1] - order.values[:, keep])]
        kept = torch.zeros(T, n_groups, dtype=torch.bool)
        kept.scatter_(1, order.indices[:, :keep], True)
        c = torch.where(kept.repeat_interleave(per, dim=1), c, torch.full_like(c, -math.inf))
    order = torch.sort(c, dim=-1, descending=True, stable=True)
    if top < N:
        margins += [float(x) for x in (order.values[:, top - 1] - order.values[:, top]) if math.isfinite(float(x))]
    ids = order.indices[:, :top]
    s = torch.gather(scores, 1, ids)
    return ids, s / (s.sum(-1, keepdim=True) + 1e-20), margins


def moe_ff(h, w, pre, mlp, margins=None):
    r = mlp["router"]
    E, I, top = r["experts"], r.get("identity", 0), r["top"]
    groups = r.get("groups") or {}
    scores = torch.softmax(h @ w[pre + "router"].t(), dim=-1)
    ids, weights, mg = choose(scores, w[pre + "correction"], top, int(groups.get("count", 1)), int(groups.get("keep", 1)))
    if margins is not None:
        margins += mg
    limit = float(mlp["expert"]["limit"]) if E else 0.0
    y = torch.zeros_like(h)
    for e in range(E + I):
        share = (weights * (ids == e)).sum(-1, keepdim=True)          # this output's weight per row, 0 where not chosen
        rows = share[:, 0] != 0
        if rows.any():
            y[rows] += share[rows] * (clamped_expert(h[rows], w, f"{pre}e{e}.", limit) if e < E else h[rows])
    if mlp.get("shared"):
        shared = clamped_expert(h, w, pre + "shared.", float(mlp["shared"]["limit"]))
        y = y + shared * torch.sigmoid(h @ w[pre + "shared.sg"].t())
    return y


def token_side(x, w, pre, table, tokens, layer, dim, eps):
    e = table[tokens][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w[pre + "gate"].t()) * e) @ w[pre + "proj"].t()
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w[pre + "norm"]


# ---- the model --------------------------------------------------------------------------------------------------------

def forward(cfg, w, ids, layers_out=None, margins=None):
    """logits [T, vocab] in float64. w: {tensor name: float64 tensor}. layers_out: a list that receives the stream after
    every layer. margins: a list that receives how far every routing choice was from going the other way."""
    eps = float(cfg["norm"]["eps"])
    tokens = torch.tensor(list(ids), dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][tokens] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    side = int((cfg.get("token_side") or {}).get("dim", 0))
    for i, entry in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = parallel_mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", entry["mixer"], eps, positions)
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        mlp = entry.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            y = dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, w, p + "mlp.", mlp, margins)
            x = x + rms_norm(y, w[p + "norm2b"], eps)
        if side:
            x = x + token_side(x, w, p + "side.", w["side.embed"], tokens, i, side, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].t()


def greedy_generate(cfg, w, prompt, n_new):
    """The n_new tokens that follow `prompt` when the largest logit is taken every time (the whole sequence is run again
    for every token: plain, not fast)."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
