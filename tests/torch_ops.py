"""Plain torch versions of the engine's operations, one function per kernel, with the kernels' signatures.

Two uses, both in tests only: as the reference that each HIP kernel is compared with, and as a stand-in
for the kernels so that the step function, the cache and the scheduler can be run on a machine without a
GPU. The engine never imports this file and has no CPU path of its own.
"""
from __future__ import annotations

import math

import torch


class TorchOps:
    def __init__(self, device="cpu", dtype=torch.float32, graphs=False):
        """graphs: let the engine keep steps in fixed buffers and "replay" them as it does with captured graphs on
        the GPU, only that a replay here is the same calls made again: the host side of that path without a device."""
        self.device = torch.device(device)
        self.dtype = dtype
        self.supports_graphs = self.emulates_graphs = bool(graphs)

    def empty(self, *shape, dtype=None):
        return torch.zeros(*shape, dtype=dtype or self.dtype, device=self.device)

    # ---- row-wise ---------------------------------------------------------------------------------------
    def embedding(self, table, tokens, out=None):
        r = table[tokens.long()]
        if out is not None:
            out[:tokens.numel()] = r
            return out
        return r

    def rmsnorm(self, x, gain, eps, out=None):
        xf = x.float()
        y = (xf * math.sqrt(x.shape[-1]) / (torch.linalg.vector_norm(xf, dim=-1, keepdim=True) + eps) * gain).to(x.dtype)
        if out is not None:
            out[:x.shape[0]] = y
            return out
        return y

    def embedding_rmsnorm(self, table, tokens, gain, eps, out=None):
        return self.rmsnorm(table[tokens.long()], gain, eps, out=out)

    def gather_rows(self, src, state, index, out=None):
        ix = index.long()
        rows = torch.zeros(ix.numel(), src.shape[1], dtype=src.dtype, device=src.device)
        from_src = ix >= 0
        rows[from_src] = src[ix[from_src]]
        rows[~from_src] = state[-ix[~from_src] - 1]
        if out is not None:
            out[:ix.numel()] = rows
            return out
        return rows

    def copy_rows(self, src, src_index, dst, dst_index):
        dst[dst_index.long()] = src[src_index.long()]

    def swiglu(self, gu, out=None):
        g, u = gu[:, 0::2].float(), gu[:, 1::2].float()      # gate and up columns come interleaved
        y = (g * torch.sigmoid(g) * u).to(gu.dtype)
        if out is not None:
            out.copy_(y)
            return out
        return y

    def linear(self, x, w, residual=None, out_dtype=None, rms=None, reuse_residual=False):
        if rms is not None:
            x = self.rmsnorm(x, rms[0], rms[1])
        y = x.float() @ w.float().t()
        if residual is not None:
            y = y + residual.float()
        return y.to(out_dtype or self.dtype)

    def linear_swiglu(self, x, w, rms=None):
        return self.swiglu(self.linear(x, w, rms=rms))

    # ---- rotary + cache write ---------------------------------------------------------------------------
    def qkv_rope(self, x, w, rms, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                 interleaved=False, write_cache=True):
        qkv = self.linear(x, w, rms=rms)
        q = torch.zeros(x.shape[0], n_heads * head_dim, dtype=qkv.dtype, device=qkv.device)
        self.rope_write_kv(qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                           interleaved, write_cache, paired=True, q_out=q)
        return q

    def rope_write_kv(self, qkv, positions, write_slots, table, plane, n_heads, n_kv_heads, head_dim, page_size,
                      interleaved=False, write_cache=True, paired=False, q_out=None):
        n = qkv.shape[0]
        if n == 0:
            return
        qkv = qkv if not paired else qkv.clone()
        x = qkv.view(n, n_heads + 2 * n_kv_heads, head_dim)
        if paired:
            # pair j sits at columns 2j, 2j+1 of every q and k head: put the heads back in natural order first
            qk_p = x[:, :n_heads + n_kv_heads]
            first, second = qk_p[..., 0::2], qk_p[..., 1::2]
            nat = torch.stack((first, second), dim=-1).flatten(-2) if interleaved else torch.cat((first, second), dim=-1)
            x[:, :n_heads + n_kv_heads] = nat
        qk = x[:, :n_heads + n_kv_heads].float()
        if table is not None:
            cs = table[positions.long()]                     # [n, hd/2, 2]
            c, s = cs[..., 0].unsqueeze(1), cs[..., 1].unsqueeze(1)
            if interleaved:
                a, b = qk[..., 0::2], qk[..., 1::2]
                rot = torch.stack((a * c - b * s, b * c + a * s), dim=-1).flatten(-2)
            else:
                h = head_dim // 2
                a, b = qk[..., :h], qk[..., h:]
                rot = torch.cat((a * c - b * s, b * c + a * s), dim=-1)
            x[:, :n_heads + n_kv_heads] = rot.to(qkv.dtype)
        if q_out is not None:
            q_out.copy_(x[:, :n_heads].reshape(n, n_heads * head_dim))
        if write_cache:
            slots = write_slots.long()
            page, off = slots // page_size, slots % page_size
            # a page holds keys as [kv head][slot][head_dim] and values transposed, [kv head][head_dim][slot]
            plane[page, 0, :, off] = x[:, n_heads:n_heads + n_kv_heads]
            vt = plane[:, 1].reshape(plane.shape[0], n_kv_heads, head_dim, page_size)
            vt[page, :, :, off] = x[:, n_heads + n_kv_heads:]
            plane[:, 1] = vt.reshape(plane.shape[0], n_kv_heads, page_size, head_dim)

    # ---- attention over the paged cache -----------------------------------------------------------------
    def paged_attention(self, q, plane, batch, group, n_heads, n_kv_heads, head_dim, window=0, scale=None, slopes=None,
                        sink=False, gate=None):
        n = q.shape[0]
        page_size = plane.shape[3]
        scale = scale if scale is not None else head_dim ** -0.5
        tables = batch.block_tables[group]
        g = n_heads // n_kv_heads
        out = torch.zeros(n, n_heads * head_dim, dtype=torch.float32, device=q.device)
        pos = batch.positions.tolist()
        seq = batch.row_seq.tolist()
        for r in range(n):
            p = pos[r]
            # window > 0: the last `window` keys; window < 0: the row's own chunk of -window positions; 0: all
            first = max(0, p - window + 1) if window > 0 else p - p % (-window) if window < 0 else 0
            js = torch.arange(first, p + 1)
            pages = tables[seq[r]].long()[js // page_size]
            k = plane[pages, 0, :, js % page_size].float()       # [keys, kvh, hd]
            vt = plane[:, 1].reshape(plane.shape[0], n_kv_heads, head_dim, page_size)
            v = vt[pages, :, :, js % page_size].float()
            qr = q[r].float().view(n_heads, head_dim)
            for h in range(n_heads):
                s = (k[:, h // g] @ qr[h]) * scale
                if slopes is not None:
                    s = s + float(slopes[h]) * (js - p).float()
                w = torch.softmax(torch.cat((s, s.new_zeros(1))), dim=0)[:-1] if sink else torch.softmax(s, dim=0)
                o = w @ v[:, h // g]
                if gate is not None:
                    o = o * torch.sigmoid(gate[r, h].float())
                out[r, h * head_dim:(h + 1) * head_dim] = o
        return out.to(q.dtype)

    def head_gate(self, x, gate, n_heads, vdim):
        y = x.float().view(x.shape[0], n_heads, vdim) * torch.sigmoid(gate.float())[:, :, None]
        x.copy_(y.view(x.shape[0], n_heads * vdim).to(x.dtype))
        return x

    # ---- a residual stream in 32-bit, norm after the sum ---------------------------------------------------
    def embed_scaled(self, table, tokens, scale):
        x32 = table[tokens.long()].float() * scale
        return x32, (x32 if self.dtype == torch.float32 else x32.to(self.dtype))

    def gated_postnorm(self, x32, branches, gate, gate_bias, alpha, gain, eps):
        y = sum(float(s) * b.float()[:, :x32.shape[1]] for b, s in branches)
        if gate is not None:
            y = y * torch.sigmoid(gate.float() + (gate_bias if gate_bias is not None else 0.0))
        r = alpha * x32 + y
        out = r / torch.sqrt((r * r).mean(-1, keepdim=True) + eps) * gain
        return out, (out if self.dtype == torch.float32 else out.to(self.dtype))

    def rmsnorm32(self, x32, gain, eps):
        return (x32 / torch.sqrt((x32 * x32).mean(-1, keepdim=True) + eps) * gain).to(self.dtype)

    def head_norm_gate(self, o32, gate, gain, n_heads, vdim, eps, act):
        n = o32.shape[0]
        o = o32.view(n, n_heads, vdim)
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps)
        o = o * (gain.view(n_heads, vdim) if gain.numel() == n_heads * vdim else gain)
        g = gate.float().reshape(n, n_heads, vdim)
        a = g * torch.sigmoid(g) if act == "silu" else torch.sigmoid(g)
        return (o * a).reshape(n, n_heads * vdim).to(self.dtype)

    def lowrank_decay(self, low, w2, bias, tau):
        z = low.float() @ w2.t() + bias
        return torch.exp(torch.nn.functional.logsigmoid(z) / tau)

    def attention_prepare(self, proj, q_off, k_off, v_off, positions, write_slots, plane, n_heads, n_kv_heads, key_dim,
                          value_dim, page_size, q_gain=None, k_gain=None, q_factor=None, freqs=None, rot_dims=0, eps=0.0,
                          write_cache=True, value_norm=True, q_bias=None, k_bias=None, v_bias=None, temp_coef=0.0,
                          temp_every=1, whole_norm=False, pair_half=False):
        n = proj.shape[0]
        H, G, kd, vd = n_heads, n_kv_heads, key_dim, value_dim

        def normed(x, gain):
            if gain is None:
                return x
            if whole_norm and torch.is_tensor(gain):      # over all heads of the row at once
                flat = x.reshape(n, -1)
                return (flat / torch.sqrt((flat * flat).mean(-1, keepdim=True) + eps) * gain).reshape(x.shape)
            return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain

        def turned(x):
            if not rot_dims:
                return x
            ang = positions.float()[:, None] * freqs[None, :]
            c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            y = x.clone()
            if pair_half:
                half = rot_dims // 2
                a, b = x[..., :half], x[..., half:rot_dims]
                y[..., :half] = a * c - b * s
                y[..., half:rot_dims] = b * c + a * s
                return y
            a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
            y[..., 0:rot_dims:2] = a * c - b * s
            y[..., 1:rot_dims:2] = b * c + a * s
            return y

        def part(off, heads, dim, bias):
            x = proj[:, off:off + heads * dim].float()
            return (x + bias if bias is not None else x).reshape(n, heads, dim)

        q = turned(normed(part(q_off, H, kd, q_bias), q_gain))
        if q_factor is not None:
            q = q * q_factor[None, :, None]
        if temp_coef:
            p1 = torch.div(positions.long() + 1, temp_every, rounding_mode="floor").float()
            q = q * (1.0 + temp_coef * torch.log(p1 + 1.0))[:, None, None]
        if write_cache:
            k = turned(normed(part(k_off, G, kd, k_bias), k_gain)).to(plane.dtype)
            v = normed(part(v_off, G, vd, v_bias), 1.0 if value_norm else None).to(plane.dtype)
            pages = plane.view(plane.shape[0], -1)
            page, off = write_slots.long() // page_size, write_slots.long() % page_size
            keys = pages[:, :G * page_size * kd].view(-1, G, page_size, kd)
            vals = pages[:, G * page_size * kd:].view(-1, G, vd, page_size)
            keys[page, :, off] = k
            vals[page, :, :, off] = v
        return q.reshape(n, H * kd).to(self.dtype)

    def latent_prepare(self, proj, q_off, c_off, positions, write_slots, plane, n_heads, dim, rot_dim, rank, page_size,
                       gain, freqs, rot_dims, eps, write_cache=True):
        n, H, D, R, C = proj.shape[0], n_heads, dim, rot_dim, rank

        def turned(x):                    # [n, ..., R]
            if not rot_dims:
                return x
            ang = positions.float()[:, None] * freqs[None, :]
            shape = (n,) + (1,) * (x.dim() - 2) + (rot_dims // 2,)
            c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
            a, b = x[..., 0:rot_dims:2], x[..., 1:rot_dims:2]
            y = x.clone()
            y[..., 0:rot_dims:2] = a * c - b * s
            y[..., 1:rot_dims:2] = b * c + a * s
            return y

        qh = proj[:, q_off:q_off + H * (D + R)].float().view(n, H, D + R)
        q = torch.zeros(n, H, C + R, dtype=self.dtype, device=proj.device)
        q[..., C:] = turned(qh[..., D:]).to(self.dtype)
        q_plain = qh[..., :D].reshape(n, H * D).to(self.dtype)
        if D == 0:
            q_plain = torch.zeros(n, H, dtype=self.dtype, device=proj.device)
        if write_cache:
            c = proj[:, c_off:c_off + C].float()
            c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * gain
            key = torch.cat((c, turned(proj[:, c_off + C:c_off + C + R].float())), dim=-1).to(plane.dtype)
            pages = plane.view(plane.shape[0], -1)
            page, off = write_slots.long() // page_size, write_slots.long() % page_size
            pages[:, :page_size * (C + R)].view(-1, page_size, C + R)[page, off] = key
            pages[:, page_size * (C + R):].view(-1, C, page_size)[page, :, off] = key[:, :C]
        return q.view(n, H * (C + R)), q_plain

    def paged_attention_kv(self, q, plane, batch, group, n_heads, n_kv_heads, key_dim, value_dim, page_size, window=0,
                           scale=None, sink=False, gate=None, chunk=0):
        n = q.shape[0]
        H, G, kd, vd = n_heads, n_kv_heads, key_dim, value_dim
        scale = scale if scale is not None else kd ** -0.5
        tables = batch.block_tables[group]
        pages = plane.view(plane.shape[0], -1)
        keys = pages[:, :G * page_size * kd].view(-1, G, page_size, kd)
        vals = pages[:, G * page_size * kd:].view(-1, G, vd, page_size)
        out = torch.zeros(n, H * vd, dtype=torch.float32, device=q.device)
        pos, seq = batch.positions.tolist(), batch.row_seq.tolist()
        for r in range(n):
            p = pos[r]
            first = max(0, p - window + 1) if window > 0 else 0
            if chunk > 0:
                first = max(first, p - p % chunk)
            js = torch.arange(first, p + 1)
            pg = tables[seq[r]].long()[js // page_size]
            k = keys[pg, :, js % page_size].float()          # [keys, G, kd]
            v = vals[pg, :, :, js % page_size].float()       # [keys, G, vd]
            qr = q[r].float().view(H, kd)
            for h in range(H):
                sc = (k[:, h // (H // G)] @ qr[h]) * scale
                if sink:
                    w = torch.softmax(torch.cat((sc, sc.new_zeros(1))), dim=0)[:-1]
                else:
                    w = torch.softmax(sc, dim=0)
                o = w @ v[:, h // (H // G)]
                if gate is not None:
                    o = o * torch.sigmoid(gate[r, h].float())
                out[r, h * vd:(h + 1) * vd] = o
        return out.to(q.dtype)

    def latent_attention(self, q, plane, batch, group, n_heads, key_dim, value_dim, page_size, scale):
        return self.paged_attention_kv(q, plane, batch, group, n_heads, 1, key_dim, value_dim, page_size, 0, scale)

    # ---- a residual stream in 32-bit, norm before the sublayer ------------------------------------------------
    def layernorm32(self, x32, gain, bias, eps):
        mu = x32.mean(-1, keepdim=True)
        var = ((x32 - mu) ** 2).mean(-1, keepdim=True)
        y = (x32 - mu) / torch.sqrt(var + eps) * gain
        return (y + bias if bias is not None else y).to(self.dtype)

    def residual_norm(self, x32, y=None, y_rms=None, copy=False, norm=None):
        if isinstance(y, tuple) and hasattr(y, "n_experts"):           # the experts' results, not summed yet
            n, top = y.ids.shape
            parts = y.results.view(n, top, -1) if y.results is not None else torch.zeros(n, top, x32.shape[1])
            own = (y.ids >= y.n_experts)[:, :, None]
            extra = y.extra.float() * torch.sigmoid(y.extra_gate.float()) if y.extra is not None else 0.0
            y = (y.weights[:, :, None] * torch.where(own, y.rows.float()[:, None, :], parts)).sum(1) + extra
        if y is not None:
            y = y.float()[:, :x32.shape[1]]
            if y_rms is not None:
                y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + y_rms[1]) * y_rms[0]
            x32 += y
        normed = None
        if norm is not None:
            kind, gain, bias, eps = norm
            normed = self.layernorm32(x32, gain, bias, eps) if kind == "layer" else self.rmsnorm32(x32, gain, eps)
        cp = (x32 if self.dtype == torch.float32 else x32.to(self.dtype)) if copy else None
        return x32, cp, normed

    @staticmethod
    def _act(z, act):
        if act == "gelu_tanh":
            return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
        return z * torch.sigmoid(z) if act == "silu" else torch.sigmoid(z)

    def gate_table(self, z, table, tokens, act):
        return (self._act(z.float(), act) * table[tokens.long()].float()).to(self.dtype)

    def activate32(self, z, act):
        z.copy_(self._act(z, act))
        return z

    # ---- products in groups ----------------------------------------------------------------------------------
    def heads_linear(self, x, w, out, out_group, out_offset=0):
        H, N, K = w.shape
        y = torch.einsum("rhk,hnk->rhn", x.float().view(x.shape[0], H, K), w.float())
        for h in range(H):
            out[:, out_offset + h * out_group:out_offset + h * out_group + N] = y[:, h].to(out.dtype)
        return out

    def route_topk(self, z, correction, scale, top, score="softmax", groups=None, renorm=False):
        s = torch.sigmoid(z.float()) if score == "sigmoid" else torch.softmax(z.float(), dim=-1)
        choice = s + correction if correction is not None else s
        if groups is not None and groups[1] < groups[0]:
            count, keep = groups
            n, N = choice.shape
            best = choice.view(n, count, N // count).max(-1).values
            kept = torch.zeros(n, count, dtype=torch.bool)
            kept.scatter_(1, torch.sort(best, dim=-1, descending=True, stable=True).indices[:, :keep], True)
            choice = torch.where(kept.repeat_interleave(N // count, dim=1), choice, torch.full_like(choice, -math.inf))
        ids = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        w = torch.gather(s, 1, ids)
        if renorm:
            w = w / (w.sum(-1, keepdim=True) + 1e-20)
        return ids.to(torch.int32), w * scale

    def routed_experts(self, x, ids, weights, w_up, w_down, act="gelu_erf", combine=True):
        from tiny_inference_server_amd.ops.hip_ops import ChosenExperts
        E = w_up.shape[0] if w_up is not None else 0
        xf = x.float()
        n, top = ids.shape
        parts = torch.zeros(n * top, x.shape[1])
        for r in range(n):
            for k in range(top):
                e = int(ids[r, k])
                if e < E:
                    hid = torch.nn.functional.gelu(w_up[e].float() @ xf[r]).to(self.dtype).float()
                    parts[r * top + k] = w_down[e].float() @ hid
        if not combine:
            return ChosenExperts(parts if E else None, ids, weights, E, x)
        own = (ids >= E)[:, :, None]
        return (weights[:, :, None] * torch.where(own, xf[:, None, :], parts.view(n, top, -1))).sum(1)

    def gated_experts(self, x, ids, weights, w_gate_up, w_down, act="silu", limit=0.0, weigh="input", n_experts=None):
        from tiny_inference_server_amd.ops.hip_ops import ChosenExperts
        E = w_gate_up.shape[0] if w_gate_up is not None else 0
        n, top = ids.shape
        xf = x.float()
        parts = torch.zeros(n * top, x.shape[1])
        for r in range(n):
            for k in range(top):
                e = int(ids[r, k])
                if e >= E:
                    continue            # an identity expert: the sum takes the row itself
                z = (w_gate_up[e].float() @ xf[r])[None, :]
                scale = weights[r, k].reshape(1) if weigh == "input" else None
                hid = self.gated_act(z, w_gate_up.shape[1] // 2, act, row_scale=scale, limit=limit)[0].float()
                parts[r * top + k] = w_down[e].float() @ hid
        return ChosenExperts(parts if E else None, ids, None if weigh == "input" else weights, E, x)

    def combine_experts(self, chosen):
        n, D = chosen.rows.shape
        return self.residual_norm(torch.zeros(n, D, dtype=torch.float32), chosen)[0]

    # ---- blocks whose sublayers read one norm and are summed with a factor per channel ------------------------
    def dyt32(self, x32, alpha, gain, bias=None):
        y = torch.tanh(alpha * x32) * gain
        return (y + bias if bias is not None else y).to(self.dtype)

    def scaled_sum(self, x32, branches, norm=None):
        from tiny_inference_server_amd.ops.hip_ops import ChosenExperts
        n = x32.shape[0]
        total = x32.clone()
        for y, scale, bias in branches:
            if isinstance(y, ChosenExperts):
                top = y.ids.shape[1]
                w = y.weights[:, :, None] if y.weights is not None else 1.0
                y = (w * y.results.view(n, top, -1)).sum(1)
            y = y.float()
            if bias is not None:
                y = y + bias
            total = total + (y * scale if scale is not None else y)
        x32.copy_(total)
        normed = self.dyt32(x32, norm[1], norm[2], norm[3]) if norm is not None else None
        return x32, normed

    def gated_act(self, z, hidden, act, gate_bias=None, up_bias=None, row_scale=None, limit=0.0):
        g, u = z[:, :hidden].float(), z[:, hidden:2 * hidden].float()
        if gate_bias is not None:
            g = g + gate_bias
        if up_bias is not None:
            u = u + up_bias
        if row_scale is not None:
            g, u = g * row_scale[:, None], u * row_scale[:, None]
        if act == "clamped_swish":
            g, u = torch.clamp(g, max=limit), torch.clamp(u, min=-limit, max=limit)
            return (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(self.dtype)
        a = torch.nn.functional.gelu(g, approximate="tanh") if act == "gelu_tanh" else g * torch.sigmoid(g)
        return (a * u).to(self.dtype)

    def activate_rows(self, z, act):
        zf = z.float()
        return (torch.relu(zf) ** 2 if act == "relu2" else self._act(zf, act)).to(self.dtype)

    def normed_mean(self, branches, eps):
        total = 0.0
        for y, gain in branches:
            yf = y.float()
            total = total + yf / torch.sqrt((yf * yf).mean(-1, keepdim=True) + eps) * gain
        return total / len(branches)

    def lowrank_act(self, low, w2, bias, kind, rate=None, group=1, tau=1.0):
        z = low.float() @ w2.t()
        if bias is not None:
            z = z + bias
        if kind == "none":
            return z
        if kind == "sigmoid_root":
            return torch.exp(torch.nn.functional.logsigmoid(z) / tau)
        return torch.exp(-rate.repeat_interleave(group) * torch.nn.functional.softplus(z, threshold=20.0))

    # ---- a gated delta rule -------------------------------------------------------------------------------------
    def delta_prepare(self, proj, conv_off, beta_off, taps, state, conv_at, batch, n_heads, qk_heads, dim, vdim):
        n = proj.shape[0]
        C, K = taps.shape
        H, G, D, V = n_heads, qk_heads, dim, vdim
        u = torch.zeros(n, C + H, dtype=torch.float32)
        cu, slots = batch.cu_rows.tolist(), batch.seq_slots.tolist()
        for k in range(batch.n_seqs):
            first, rows = cu[k], cu[k + 1] - cu[k]
            if rows == 0:
                continue
            old = state[slots[k], conv_at:conv_at + (K - 1) * C].view(K - 1, C)
            seq = torch.cat((old, proj[first:first + rows, conv_off:conv_off + C].float()), dim=0)
            acc = torch.zeros(rows, C)
            for j in range(K):
                acc = acc + seq[j:j + rows] * taps[:, j]
            y = acc * torch.sigmoid(acc)
            qk = y[:, :2 * G * D].view(rows, 2 * G, D)
            qk = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
            qk[:, :G] *= D ** -0.5
            u[first:first + rows, :2 * G * D] = qk.reshape(rows, -1)
            u[first:first + rows, 2 * G * D:C] = y[:, 2 * G * D:]
            u[first:first + rows, C:] = torch.sigmoid(proj[first:first + rows, beta_off:beta_off + H].float())
        return u

    def delta_scan(self, u, q_off, k_off, v_off, beta_off, decay, state, batch, n_heads, qk_heads, dim, vdim):
        H, G, D, V = n_heads, qk_heads, dim, vdim
        n = u.shape[0]
        out = torch.zeros(n, H * V, dtype=torch.float32)
        cu, slots = batch.cu_rows.tolist(), batch.seq_slots.tolist()
        rep = H // G
        VB = -(-V // 16)
        for s in range(batch.n_seqs):
            if cu[s + 1] == cu[s]:
                continue
            # the line holds S as [heads, blocks of 16 value channels, dim, 16]
            line = state[slots[s], :H * VB * D * 16].view(H, VB, D, 16)
            S = line.permute(0, 2, 1, 3).reshape(H, D, VB * 16)[:, :, :V].clone()
            for r in range(cu[s], cu[s + 1]):
                q = u[r, q_off:q_off + G * D].view(G, D).repeat_interleave(rep, dim=0)
                k = u[r, k_off:k_off + G * D].view(G, D).repeat_interleave(rep, dim=0)
                v = u[r, v_off:v_off + H * V].view(H, V)
                beta = u[r, beta_off:beta_off + H]
                S.mul_(decay[r].view(H, D, 1))
                w = beta[:, None] * (v - torch.einsum("hdv,hd->hv", S, k))
                S.add_(k[:, :, None] * w[:, None, :])
                out[r] = torch.einsum("hdv,hd->hv", S, q).reshape(-1)
            full = torch.zeros(H, D, VB * 16)
            full[:, :, :V] = S
            line.copy_(full.view(H, D, VB, 16).permute(0, 2, 1, 3))
        return out

    # ---- attention whose weights are sigmoids mixed across the heads --------------------------------------------
    def mixed_sigmoid_attention(self, q, plane, batch, group, n_heads, n_kv_heads, key_dim, value_dim, page_size, chunk,
                                scale, softcap, head_bias, talk):
        n = q.shape[0]
        H, G, kd, vd = n_heads, n_kv_heads, key_dim, value_dim
        tables = batch.block_tables[group]
        pages = plane.view(plane.shape[0], -1)
        keys = pages[:, :G * page_size * kd].view(-1, G, page_size, kd)
        vals = pages[:, G * page_size * kd:].view(-1, G, vd, page_size)
        out = torch.zeros(n, H * vd, dtype=torch.float32, device=q.device)
        pos, seq = batch.positions.tolist(), batch.row_seq.tolist()
        for r in range(n):
            p = pos[r]
            first = p - p % chunk if chunk > 0 else 0
            js = torch.arange(first, p + 1)
            pg = tables[seq[r]].long()[js // page_size]
            k = keys[pg, :, js % page_size].float().repeat_interleave(H // G, dim=1)      # [keys, H, kd]
            v = vals[pg, :, :, js % page_size].float().repeat_interleave(H // G, dim=1)   # [keys, H, vd]
            sc = torch.einsum("jhd,hd->hj", k, q[r].float().view(H, kd)) * scale
            if softcap:
                sc = softcap * torch.tanh(sc / softcap)
            w = talk.float() @ torch.sigmoid(sc + head_bias[:, None])
            out[r] = torch.einsum("hj,jhv->hv", w, v).reshape(-1)
        return out.to(q.dtype)

    def softcap(self, z, cap):
        z.copy_(cap * torch.tanh(z / cap))
        return z

    # ---- around the scan of a selective state-space mixer ----------------------------------------------------
    def conv_prepare(self, proj, xbc_off, dt_off, taps, tap_bias, dt_bias, neg_a, state, conv_at, batch, n_heads, vdim):
        n = proj.shape[0]
        C, K = taps.shape
        inner = n_heads * vdim
        u = torch.zeros(n, C + inner + n_heads, dtype=torch.float32)
        cu, slots = batch.cu_rows.tolist(), batch.seq_slots.tolist()
        for k in range(batch.n_seqs):
            first, rows = cu[k], cu[k + 1] - cu[k]
            if rows == 0:
                continue
            old = state[slots[k], conv_at:conv_at + (K - 1) * C].view(K - 1, C)
            seq = torch.cat((old, proj[first:first + rows, xbc_off:xbc_off + C].float()), dim=0)
            acc = (tap_bias if tap_bias is not None else torch.zeros(C)).expand(rows, C).clone()
            for j in range(K):
                acc = acc + seq[j:j + rows] * taps[:, j]
            y = acc * torch.sigmoid(acc)
            dt = torch.nn.functional.softplus(proj[first:first + rows, dt_off:dt_off + n_heads].float() + dt_bias, threshold=20.0)
            u[first:first + rows, :C] = y
            u[first:first + rows, C:C + inner] = (y[:, :inner].view(rows, n_heads, vdim) * dt[:, :, None]).reshape(rows, inner)
            u[first:first + rows, C + inner:] = torch.exp(neg_a * dt)
        return u

    def conv_state_update(self, proj, xbc_off, channels, taps, state, conv_at, batch):
        if taps == 1:
            return
        cu, slots = batch.cu_rows.tolist(), batch.seq_slots.tolist()
        for k in range(batch.n_seqs):
            first, rows = cu[k], cu[k + 1] - cu[k]
            if rows == 0:
                continue
            line = state[slots[k], conv_at:conv_at + (taps - 1) * channels].view(taps - 1, channels)
            seq = torch.cat((line, proj[first:first + rows, xbc_off:xbc_off + channels].float()), dim=0)
            line.copy_(seq[-(taps - 1):])

    def gated_group_norm(self, y, x, skip, vdim, z, gain, eps, parts):
        n, W = y.shape
        v = y.float()
        if skip is not None:
            v = v + x.float() * skip.repeat_interleave(vdim)
        if z is not None:
            zf = z.float()
            v = v * zf * torch.sigmoid(zf)
        v = v.view(n, parts, W // parts)
        v = (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)).reshape(n, W) * gain
        return v.to(self.dtype)

    @staticmethod
    def state_scan_floats(kind, n_heads, dim, vdim):
        return n_heads * dim * vdim + (n_heads * -(-vdim // 16) * (dim + 1) if kind == "gated_max" else 0)

    def state_scan(self, kind, proj, q_off, k_off, v_off, q_scale, state, batch, n_heads, dim, vdim, decay=None,
                   i_off=0, f_off=0, bias_i=None, bias_f=None, cap=0.0, qk_group=1, decay_per_head=False):
        """The same line of state as the kernel keeps (n and m once per block of 16 value channels)."""
        n, H, D, V = proj.shape[0], n_heads, dim, vdim
        blocks = -(-V // 16)
        out = torch.zeros(n, H * V, dtype=torch.float32, device=proj.device)
        # (the step's device arrays, as the kernel reads them: a kept step's host copies are those of its first run)
        cu, slots = batch.cu_rows.tolist(), batch.seq_slots.tolist()
        for k in range(batch.n_seqs):
            first, rows = cu[k], cu[k + 1] - cu[k]
            if rows == 0:
                continue
            line = state[slots[k]]
            S = line[:H * D * V].view(H, D, V)
            nm = line[H * D * V:H * D * V + H * blocks * (D + 1)].view(H, blocks, D + 1) if kind == "gated_max" else None
            for r in range(first, first + rows):
                Hq = H // qk_group
                q = proj[r, q_off:q_off + Hq * D].float().view(Hq, D).repeat_interleave(qk_group, dim=0) * q_scale
                kk = proj[r, k_off:k_off + Hq * D].float().view(Hq, D).repeat_interleave(qk_group, dim=0)
                v = proj[r, v_off:v_off + H * V].float().view(H, V)
                if kind == "decay":
                    a = decay[r, :H].view(H, 1, 1) if decay_per_head else decay[r].view(H, D, 1)
                    S.copy_(a * S + kk[:, :, None] * v[:, None, :])
                    o = torch.einsum("hdv,hd->hv", S, q)
                else:
                    gi = cap * torch.tanh((proj[r, i_off:i_off + H].float() + bias_i) / cap)
                    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((proj[r, f_off:f_off + H].float() + bias_f) / cap))
                    m = nm[:, 0, D].clone()
                    m_new = torch.maximum(gf + m, gi)
                    keep, take = torch.exp(gf + m - m_new), torch.exp(gi - m_new)
                    S.copy_(keep[:, None, None] * S + take[:, None, None] * kk[:, :, None] * v[:, None, :])
                    nvec = keep[:, None] * nm[:, 0, :D] + take[:, None] * kk
                    nm[:, :, :D] = nvec[:, None, :]
                    nm[:, :, D] = m_new[:, None]
                    den = torch.maximum((nvec * q).sum(-1).abs(), torch.exp(-m_new)) + 1e-6
                    o = torch.einsum("hdv,hd->hv", S, q) / den[:, None]
                out[r] = o.reshape(-1)
        return out

    # ---- sampling ---------------------------------------------------------------------------------------
    def argmax(self, logits):
        return torch.argmax(logits, dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, rep_penalty, uniform, ctx_tokens=None, ctx_offsets=None,
               seen=None, seen_row=None):
        """The kernel's method: thresholds instead of a sort, inverse CDF in token order."""
        n, V = logits.shape
        out = torch.zeros(n, dtype=torch.int32)
        if seen is not None:
            # the byte-table form of the context: turn each row's line into a token list, mark the draw afterwards
            lists = [torch.nonzero(seen[int(seen_row[r])]).flatten().to(torch.int32) if int(seen_row[r]) >= 0
                     else torch.zeros(0, dtype=torch.int32) for r in range(n)]
            offs = torch.tensor([0] + list(torch.tensor([len(l) for l in lists]).cumsum(0)), dtype=torch.int32)
            flat = torch.cat(lists) if lists else torch.zeros(0, dtype=torch.int32)
            out = self.sample(logits, temperature, top_k, top_p, rep_penalty, uniform, flat, offs)
            for r in range(n):
                if int(seen_row[r]) >= 0:
                    seen[int(seen_row[r]), int(out[r])] = 1
            return out
        for r in range(n):
            l = logits[r].float().clone()
            t, k, p = float(temperature[r]), int(top_k[r]), float(top_p[r])
            pen = float(rep_penalty[r]) if rep_penalty is not None else 1.0
            greedy = t == 0.0 or k == 1
            inv_t = 1.0 if greedy else 1.0 / t
            x = l * inv_t
            if pen != 1.0 and ctx_tokens is not None:
                toks = ctx_tokens[int(ctx_offsets[r]):int(ctx_offsets[r + 1])].long().unique()
                lt = l[toks]
                x[toks] = torch.where(lt > 0, lt / pen, lt * pen) * inv_t
            if greedy:
                out[r] = int(torch.argmax(x))
                continue
            keep = torch.ones(V, dtype=torch.bool)
            if 0 < k < V:
                kth = torch.topk(x, k).values[-1]
                keep = x >= kth
            e = torch.where(keep, torch.exp(x - x.max()), torch.zeros_like(x))
            if 0.0 < p < 1.0:
                z = e.sum()
                order = torch.argsort(x, descending=True)
                before = torch.cumsum(e[order], 0) - e[order]
                ok = before <= p * z
                keep2 = torch.zeros(V, dtype=torch.bool)
                keep2[order[ok]] = True
                e = torch.where(keep2, e, torch.zeros_like(e))
            c = torch.cumsum(e.double(), 0)
            nz = torch.nonzero(c > float(uniform[r]) * float(c[-1]))
            out[r] = int(nz[0]) if len(nz) else int(torch.argmax(x))
        return out.to(logits.device)
