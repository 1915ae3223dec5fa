"""The Rurorax decoder written out plainly: float64, whole sequences, one function per mechanism.

Nothing here is shared with the engine: no cache, no pages, no state slots, no kernels. A sequence goes in as a list of
token ids, logits for every position come out (and, if asked, the stream after every layer). Tests compare the engine
with this.

The design: x = E[token]; every layer x <- x + s1 * mixer(h) + s2 * ff(h) with one h = dyt(x) for both sublayers
(dyt(x) = tanh(a x) * g + b, a scalar a), s1 and s2 a factor per channel; the mixer is chunk-local grouped-query
attention or a selective state-space recurrence; the feed-forward is a gated dense layer with biases, a mixture of
experts whose router weight scales the expert's input, or absent; logits = cap * tanh(E dyt(x) / cap).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def w64(tensors, name):
    return tensors[name].to(F64)


def dynamic_tanh(x, alpha, gain, bias):
    return torch.tanh(alpha * x) * gain + bias


def rms_norm(x, gain, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rotary_frequencies(dims, base, factor=1.0):
    i = torch.arange(dims // 2, dtype=F64)
    return base ** (-2.0 * i / dims) / factor


def rotate_half(x, positions, dims, base, factor=1.0):
    """x: [T, heads, D]. Channel i < dims/2 is paired with channel i + dims/2; channels from dims on stay."""
    if not dims:
        return x
    half = dims // 2
    ang = positions.to(F64).view(-1, 1, 1) * rotary_frequencies(dims, base, factor).view(1, 1, half)
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat((u * c - v * s, v * c + u * s, x[..., dims:]), dim=-1)


def chunk_visible(T, size):
    """visible[i, j]: j <= i and both in the same chunk of `size` positions counted from 0 (size 0: plain causal)."""
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    vis = j <= i
    if size:
        vis = vis & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))
    return vis


def chunked_attention(h, t, pre, m, eps):
    """Grouped-query attention inside chunks of positions: biased projections, an RMS norm over the whole of q and the
    whole of k (all heads at once), rotation of a head's first channels, paired half the rotated part apart, at frequencies divided by a factor."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w64(t, pre + "q").T + w64(t, pre + "q.b")
    k = h @ w64(t, pre + "k").T + w64(t, pre + "k.b")
    v = (h @ w64(t, pre + "v").T + w64(t, pre + "v.b")).view(T, G, V)
    q = rms_norm(q, w64(t, pre + "q.norm"), eps).view(T, H, D)
    k = rms_norm(k, w64(t, pre + "k.norm"), eps).view(T, G, D)
    rot = m.get("rot") or {}
    dims = rot.get("dims", 0)
    if dims:
        factor = (rot.get("scaling") or {}).get("factor", 1.0)
        pos = torch.arange(T)
        q = rotate_half(q, pos, dims, rot["base"], factor)
        k = rotate_half(k, pos, dims, rot["base"], factor)
    vis = chunk_visible(T, (m.get("mask") or {}).get("size", 0))
    out = torch.zeros(T, H, V, dtype=F64)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T * m["scale"]).masked_fill(~vis, -math.inf)
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    return out.reshape(T, H * V) @ w64(t, pre + "o").T + w64(t, pre + "o.b")


def causal_conv(x, taps, bias):
    """x: [T, C]; taps: [C, K], the last column weighs the current row; zeros before the first row."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat((torch.zeros(K - 1, C, dtype=x.dtype), x), dim=0)
    y = bias.expand(T, C).clone()
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return y


def selective_scan(x, B, C, dt, a, D):
    """x: [T, H, P]; B, C: [T, H, N] (already spread from groups to heads); dt: [T, H]; a = -exp(A_log): [H]; D: [H].
    S_t = exp(a dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t."""
    T, H, P = x.shape
    N = B.shape[-1]
    S = torch.zeros(H, N, P, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    for i in range(T):
        S = torch.exp(a * dt[i]).view(H, 1, 1) * S + dt[i].view(H, 1, 1) * B[i].unsqueeze(-1) * x[i].unsqueeze(-2)
        y[i] = torch.einsum("hnp,hn->hp", S, C[i]) + D.view(H, 1) * x[i]
    return y


def state_space(h, t, pre, m, eps):
    """The selective state-space mixer: one input product laid out [z | x | B | C | dt], a short causal convolution
    with silu over x, B and C, the scan, the gate silu(z) before a norm in equal parts, the output product."""
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    p = h @ w64(t, pre + "in").T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w64(t, pre + "conv"), w64(t, pre + "conv.b")))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    dt = softplus(dt + w64(t, pre + "dt_bias"))
    y = selective_scan(x, B, C, dt, -torch.exp(w64(t, pre + "A_log")), w64(t, pre + "D")).reshape(T, inner)
    y = y * silu(z)
    parts = m.get("norm_groups", 1)
    y = rms_norm(y.view(T, parts, inner // parts), torch.ones((), dtype=F64), eps).reshape(T, inner) * w64(t, pre + "norm")
    return y @ w64(t, pre + "o").T


def dense_ff(h, t, pre):
    g = h @ w64(t, pre + "gate").T + w64(t, pre + "gate.b")
    u = h @ w64(t, pre + "up").T + w64(t, pre + "up.b")
    return (gelu_tanh(g) * u) @ w64(t, pre + "down").T + w64(t, pre + "down.b")


def route(h, t, pre, top, margins=None):
    """(ids [T, top], weights [T, top]): the experts with the largest sigmoid scores, and those scores. margins: a list
    that receives, per row, how far the last chosen logit lies above the first one left out."""
    z = h @ w64(t, pre + "router").T
    s = torch.sigmoid(z)
    w, ids = torch.topk(s, top, dim=-1)
    if margins is not None and top < z.shape[-1]:
        ranked = torch.sort(z, dim=-1, descending=True).values
        margins.extend((ranked[:, top - 1] - ranked[:, top]).tolist())
    return ids, w


def expert_ff(h, t, pre):
    return (silu(h @ w64(t, pre + "gate").T) * (h @ w64(t, pre + "up").T)) @ w64(t, pre + "down").T


def moe_ff(h, t, pre, mlp, choose=None, margins=None):
    """sum over a row's chosen experts of expert(weight * h). choose(h) -> (ids, weights) replaces the router's choice."""
    ids, w = choose(h) if choose is not None else route(h, t, pre, mlp["router"]["top"], margins)
    y = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for e, we in zip(ids[r].tolist(), w[r]):
            y[r] += expert_ff((we * h[r]).unsqueeze(0), t, f"{pre}e{e}.")[0]
    return y


def norm_of(x, t, name):
    return dynamic_tanh(x, w64(t, name + ".alpha"), w64(t, name), w64(t, name + ".b"))


def layer(x, t, i, entry, eps, choose=None, margins=None):
    pre = f"l{i}."
    h = norm_of(x, t, pre + "norm1")
    if entry["type"] == "attention":
        y = chunked_attention(h, t, pre + "mix.", entry["mixer"], eps)
    elif entry["type"] == "mamba2":
        y = state_space(h, t, pre + "mix.", entry["mixer"], eps)
    else:
        raise ValueError(entry["type"])
    out = x + y * w64(t, pre + "ls1")
    mlp = entry.get("mlp")
    if mlp is not None:
        f = dense_ff(h, t, pre + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, t, pre + "mlp.", mlp, choose, margins)
        out = out + f * w64(t, pre + "ls2")
    return out


def forward(config, tensors, tokens, streams=None, choose=None, margins=None):
    """Logits [T, vocab] in float64. streams: a list that receives the stream after every layer. margins: a list that
    receives every routed row's margin (see route)."""
    eps = config["norm"]["eps"]
    x = w64(tensors, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    for i, entry in enumerate(config["layers"]):
        x = layer(x, tensors, i, entry, eps, choose, margins)
        if streams is not None:
            streams.append(x.clone())
    logits = norm_of(x, tensors, "final.norm") @ w64(tensors, "embed").T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy_generate(config, tensors, prompt, n_new):
    """n_new tokens, each the largest logit of the whole sequence so far run again from its start."""
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(forward(config, tensors, ids)[-1].argmax()))
    return ids[len(prompt):]
