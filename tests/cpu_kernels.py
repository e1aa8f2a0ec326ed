"""A stand-in for the kernel library, written with torch operators on the CPU.

It exists only so that tests without a GPU can drive the engine's own code
(step function, cache, block tables, generation loop) and compare with the plain
implementation.  The package never imports it; on the product path there is no
CPU fallback.  Same method names and argument meanings as `HipKernels`.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from longbow_quarrel_amd.kernels.dry import query


class CpuKernels:
    name = "cpu-test-standin"

    def __init__(self) -> None:
        self.force_generic = False
        self.calls = []

    def use_stream(self, stream) -> None:
        pass

    def embed(self, table, tokens, out, scale=1.0):
        t = tokens[: out.shape[0]].long()
        known = (t >= 0) & (t < table.shape[0])  # no row of the table: zeros, as the library does
        out.copy_(table[t.clamp(0, table.shape[0] - 1)].float() * known[:, None] * scale)

    @staticmethod
    def _whole(delta, like):
        d = delta.float()
        return d.sum(0) if d.dim() == like.dim() + 1 else d

    @query
    def linear_pieces(self, dtype, m, n, k):
        return 1

    @query
    def linear_fused_parts(self, dtype, m, n, k):
        return 0

    def rmsnorm(self, x, weight, eps, out, delta=None):
        if delta is not None:
            x += self._whole(delta, x)
        ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
        out.copy_((x / torch.sqrt(ms + eps) * weight).to(out.dtype))

    def add(self, x, delta):
        x += self._whole(delta, x)

    def cast(self, src, out):
        out.copy_(src.to(out.dtype))

    def linear(self, x, w, out):
        assert x.dtype == w.dtype
        out.copy_((x.float() @ w.float().t()).to(out.dtype))

    def swiglu(self, gate_up, out):
        inner = out.shape[1]
        g = gate_up[:, :inner].float()
        u = gate_up[:, inner:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def gather_rows(self, x, rows, out, delta=None):
        idx = rows[: out.shape[0]].long()
        v = x[idx]
        if delta is not None:
            v = v + self._whole(delta, x)[idx]
        out.copy_(v)

    @staticmethod
    def _rotate(x, heads, hd, freqs, pos):
        rows = x.shape[0]
        v = x[:, : heads * hd].float().reshape(rows, heads, hd).double()
        ang = pos[:rows].double()[:, None] * freqs[None, :]
        c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
        half = hd // 2
        a, b = v[..., :half].float(), v[..., half:].float()
        return torch.cat([a * c - b * s, a * s + b * c], dim=-1).reshape(rows, heads * hd)

    def rope_table(self, freqs, row_pos, table):
        ang = row_pos[: table.shape[0]].double()[:, None] * freqs.double()[None, :]
        table[:, :, 0] = torch.cos(ang).float()
        table[:, :, 1] = torch.sin(ang).float()

    def rope_store(self, q, k, v, heads, kv_heads, head_dim, freqs, row_pos, row_seq=None, seq_slot=None,
                   block_table=None, kcache=None, vcache=None, block_size=0, cos_sin=None, cu_rows=None):
        rows = q.shape[0]
        if freqs is not None:
            q[:, : heads * head_dim] = self._rotate(q, heads, head_dim, freqs, row_pos).to(q.dtype)
        if kcache is None:
            return
        kr = self._rotate(k, kv_heads, head_dim, freqs, row_pos) if freqs is not None \
            else k[:, : kv_heads * head_dim].float()
        kr = kr.to(q.dtype).reshape(rows, kv_heads, head_dim)
        vr = v[:, : kv_heads * head_dim].reshape(rows, kv_heads, head_dim)
        for r in range(rows):
            p = int(row_pos[r])
            slot = int(seq_slot[int(row_seq[r])])
            blk = int(block_table[slot, p // block_size])
            off = p % block_size
            kcache[blk, :, off, :] = kr[r]
            vcache[blk, :, :, off] = vr[r]

    @query
    def attention_workspace(self, dtype, rows, heads, kv_heads, head_dim, block_size, decode, max_len):
        return 0

    def attention(self, q, out, heads, kv_heads, head_dim, row_pos, row_seq, seq_slot, cu_rows, block_table,
                  kcache, vcache, block_size, scale, window=0, decode=False, max_len=0, workspace=None, uneven=False):
        rows = q.shape[0]
        group = heads // kv_heads
        for r in range(rows):
            p = int(row_pos[r])
            slot = int(seq_slot[int(row_seq[r])])
            lo = p - window + 1 if (window > 0 and p >= window) else 0
            ts = list(range(lo, p + 1))
            blks = [int(block_table[slot, t // block_size]) for t in ts]
            offs = [t % block_size for t in ts]
            kk = torch.stack([kcache[b, :, o, :] for b, o in zip(blks, offs)]).float()  # [T, kvh, hd]
            vv = torch.stack([vcache[b, :, :, o] for b, o in zip(blks, offs)]).float()
            for h in range(heads):
                g = h // group
                qv = q[r, h * head_dim : (h + 1) * head_dim].float()
                s = (kk[:, g] @ qv) * scale
                pr = torch.softmax(s, dim=0)
                out[r, h * head_dim : (h + 1) * head_dim] = (pr[:, None] * vv[:, g]).sum(0).to(out.dtype)

    # ---- the kernels of the recurrent mixers, the windowed attention with a sink and their norms ----
    def dynamic_tanh(self, x, weight, bias, alpha, out, delta=None, delta_scale=1.0):
        if delta is not None:
            x += self._whole(delta, x) * delta_scale
        out.copy_((torch.tanh(x * alpha) * weight + bias).to(out.dtype))

    def add_scaled(self, x, delta, scale):
        x += self._whole(delta, x) * scale

    @staticmethod
    def _act(g, activation):
        if activation == "relu":
            return torch.clamp(g, min=0)
        if activation == "silu":
            return g / (1 + torch.exp(-g))
        if activation == "gelu_tanh":
            return 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g * g * g)))
        if activation == "gelu":
            return 0.5 * g * (1 + torch.erf(g * math.sqrt(0.5)))
        raise ValueError(activation)

    def activation(self, x, out, activation):
        out.copy_(self._act(x.float(), activation).to(out.dtype))

    def glu(self, gate_up, out, activation, bias=None, tail=0, row_gate=None):
        inner = out.shape[1] - tail
        g, u = gate_up[:, :inner].float(), gate_up[:, inner:].float()
        if bias is not None:
            g, u = g + bias[:inner], u + bias[inner:]
        if activation == "gelu":
            raise ValueError(activation)
        a = self._act(g, activation)
        if row_gate is not None:
            a = a * torch.sigmoid(row_gate.float().reshape(-1, 1))
        out[:, :inner] = (a * u).to(out.dtype)
        if tail:
            out[:, inner:] = 0
            out[:, inner] = 1

    def kv_store(self, k, v, kv_heads, key_dim, value_dim, row_pos, row_seq, seq_slot, block_table, kcache, vcache,
                 block_size):
        for r in range(k.shape[0]):
            p = int(row_pos[r])
            blk = int(block_table[int(seq_slot[int(row_seq[r])]), p // block_size])
            kcache[blk, :, p % block_size, :] = k[r].reshape(kv_heads, key_dim)
            vcache[blk, :, :, p % block_size] = v[r].reshape(kv_heads, value_dim)

    def sink_attention(self, q, out, heads, kv_heads, key_dim, value_dim, row_pos, row_seq, seq_slot, block_table,
                       kcache, vcache, block_size, scale, window=0, keep_first=0, sink=True, gate=None, decode=False,
                       sink_values=None, maps=1):
        if maps > 1:  # a cached key row holds the keys of `maps` key heads side by side; they share the value head
            nb, g_heads, bs, wide = kcache.shape
            kcache = kcache.reshape(nb, g_heads, bs, maps, key_dim).permute(0, 1, 3, 2, 4).reshape(nb, kv_heads, bs, key_dim)
            vcache = vcache.repeat_interleave(maps, dim=1)
        for r in range(q.shape[0]):
            p = int(row_pos[r])
            slot = int(seq_slot[int(row_seq[r])])
            lo = p - window + 1 if (window > 0 and p >= window) else 0
            ts = [t for t in range(p + 1) if t >= lo or t < keep_first]
            kk = torch.stack([kcache[int(block_table[slot, t // block_size]), :, t % block_size, :] for t in ts]).float()
            vv = torch.stack([vcache[int(block_table[slot, t // block_size]), :, :, t % block_size] for t in ts]).float()
            for h in range(heads):
                g = h // (heads // kv_heads)
                s = (kk[:, g] @ q[r, h * key_dim : (h + 1) * key_dim].float()) * scale
                at = float(sink_values[h]) if sink_values is not None else 0.0
                m = torch.clamp(s.max(), min=at) if sink else s.max()
                e = torch.exp(s - m)
                denom = e.sum() + (torch.exp(at - m) if sink else 0.0)
                o = (e[:, None] * vv[:, g]).sum(0) / denom
                if gate is not None:
                    o = o * torch.sigmoid(gate[r, h].float())
                out[r, h * value_dim : (h + 1) * value_dim] = o.to(out.dtype)

    def causal_conv(self, x, weight, bias, state, out, row_pos, row_seq, seq_slot, seq_start, seq_len, cu_rows, batch,
                    activation="silu"):
        taps = weight.shape[1]
        for b in range(batch):
            r0, r1 = int(cu_rows[b]), int(cu_rows[b + 1])
            slot = int(seq_slot[b])
            hist = torch.cat([state[slot][: taps - 1], x[r0:r1].float()], 0) if taps > 1 else x[r0:r1].float()
            y = torch.zeros((r1 - r0, x.shape[1]))
            for j in range(taps):
                y += hist[j : j + (r1 - r0)] * weight[:, j]
            if bias is not None:
                y += bias
            if activation == "silu":
                y = y / (1 + torch.exp(-y))
            out[r0:r1] = y.to(out.dtype)
            if taps > 1:
                state[slot][: taps - 1] = hist[hist.shape[0] - (taps - 1) :]

    def ssd_scan(self, x, b_in, c_in, dt, dt_bias, a_log, d_skip, state, y, heads, head_dim, n_state, groups, seq_slot,
                 cu_rows, batch):
        for b in range(batch):
            r0, r1 = int(cu_rows[b]), int(cu_rows[b + 1])
            s = state[int(seq_slot[b])]  # [heads, head_dim, n_state]
            for r in range(r0, r1):
                step = torch.nn.functional.softplus(dt[r].float() + dt_bias, threshold=1e9)
                decay = torch.exp(-torch.exp(a_log) * step)
                xr = x[r].float().reshape(heads, head_dim)
                br = b_in[r].float().reshape(groups, n_state).repeat_interleave(heads // groups, 0)
                cr = c_in[r].float().reshape(groups, n_state).repeat_interleave(heads // groups, 0)
                s.mul_(decay[:, None, None]).add_(step[:, None, None] * xr[:, :, None] * br[:, None, :])
                y[r] = ((s * cr[:, None, :]).sum(-1) + d_skip[:, None] * xr).reshape(-1)

    def delta_scan(self, q, k, v, beta, a, dt_bias, a_log, state, out, heads, kv_heads, key_dim, value_dim, q_scale,
                   unit_eps, seq_slot, cu_rows, batch, channel_decay=False):
        rep = heads // kv_heads
        for b in range(batch):
            r0, r1 = int(cu_rows[b]), int(cu_rows[b + 1])
            s = state[int(seq_slot[b])]  # [heads, value_dim, key_dim]
            for r in range(r0, r1):
                qr = q[r].float().reshape(kv_heads, key_dim)
                kr = k[r].float().reshape(kv_heads, key_dim)
                qr = (qr / torch.sqrt((qr * qr).sum(-1, keepdim=True) + unit_eps) * q_scale).repeat_interleave(rep, 0)
                kr = (kr / torch.sqrt((kr * kr).sum(-1, keepdim=True) + unit_eps)).repeat_interleave(rep, 0)
                vr = v[r].float().reshape(heads, value_dim)
                bt = torch.sigmoid(beta[r].float())
                step = torch.nn.functional.softplus(a[r].float() + dt_bias, threshold=1e9)
                if channel_decay:
                    s.mul_(torch.exp(-torch.exp(a_log)[:, None] * step.reshape(heads, key_dim))[:, None, :])
                else:
                    s.mul_(torch.exp(-torch.exp(a_log) * step)[:, None, None])
                u = bt[:, None] * (vr - (s * kr[:, None, :]).sum(-1))
                s.add_(u[:, :, None] * kr[:, None, :])
                out[r] = (s * qr[:, None, :]).sum(-1).reshape(-1)

    def gated_rmsnorm(self, y, z, weight, eps, group, out, gate_first=True, gate="silu"):
        rows, n = y.shape
        zf = z.float()
        gate = torch.sigmoid(zf) if gate == "sigmoid" else zf / (1 + torch.exp(-zf))
        v = y.float() * gate if gate_first else y.float()
        v = v.reshape(rows, n // group, group)
        v = (v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)).reshape(rows, n)
        v = v * (weight if weight.numel() == n else weight.repeat(n // weight.numel()))
        out.copy_((v if gate_first else v * gate).to(out.dtype))

    def rmsnorm_mean(self, stack, weights, eps, out):
        acc = torch.zeros_like(out)
        for t, w in zip(stack, weights):
            acc += t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps) * w
        out.copy_(acc / len(weights))

    # greedy sampling and the upkeep of a decoding batch's arrays, so that the generation loop runs here too
    def argmax(self, logits, out, scratch=None, seq_slot=None, recent=None, recent_n=None):
        rows = logits.shape[0]
        best = logits.argmax(dim=-1).to(torch.int32)
        bad = ~torch.isfinite(logits).all(dim=-1)
        out[:rows] = torch.where(bad, torch.full_like(best, -1), best)

    def advance(self, row_pos, seq_start, seq_len, batch):
        for t in (row_pos, seq_start, seq_len):
            t[:batch] += 1

    # ---- the kernels of the bigram embedding, the norm on a sublayer's result, gated linear attention, attention
    # ---- through a latent and the mixture of experts ----
    def bigram_add(self, x, table, tokens, prev, buckets, mul_prev, mul_cur, vocab, row_pos, row_seq, seq_slot, cu_rows,
                   batch):
        for b in range(batch):
            r0, r1 = int(cu_rows[b]), int(cu_rows[b + 1])
            slot = int(seq_slot[b])
            for r in range(r0, r1):
                tok = int(tokens[r])
                before = int(tokens[r - 1]) if r > r0 else int(prev[slot, 0])
                if int(row_pos[r]) == 0:
                    x[r] += table[buckets].float()
                elif 0 <= tok < vocab and 0 <= before < vocab:
                    x[r] += table[(before * mul_prev + tok * mul_cur) % buckets].float()
            prev[slot, 0] = int(tokens[r1 - 1])

    def rmsnorm_residual(self, x, y, weight, eps, rounded=None):
        yf = y.float()
        x += yf / torch.sqrt((yf * yf).mean(-1, keepdim=True) + eps) * weight
        if rounded is not None:
            rounded.copy_(x.to(rounded.dtype))

    def rmsnorm_cols(self, src, weight, eps, out):
        v = src.float()
        out.copy_((v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * weight).to(out.dtype))

    def rotary(self, src, out, heads, size, out_head_stride, dims, interleaved, freqs, magnitude, row_pos):
        rows = src.shape[0]
        v = src.float().reshape(rows, heads, size).clone()
        ang = row_pos[:rows].double()[:, None] * freqs.double()[None, :]
        c = (torch.cos(ang) * magnitude).float()[:, None, :]
        s = (torch.sin(ang) * magnitude).float()[:, None, :]
        half = dims // 2
        if interleaved:
            a, b = v[..., 0:dims:2].clone(), v[..., 1:dims:2].clone()
            v[..., 0:dims:2], v[..., 1:dims:2] = a * c - b * s, b * c + a * s
        else:
            a, b = v[..., :half].clone(), v[..., half:dims].clone()
            v[..., :half], v[..., half:dims] = a * c - b * s, b * c + a * s
        for h in range(heads):
            out[:, h * out_head_stride : h * out_head_stride + size] = v[:, h].to(out.dtype)

    def diff_combine(self, both, out, heads, kv_heads, value_dim, lam, eps, gain):
        rows, group = both.shape[0], heads // kv_heads
        a = both.float().reshape(rows, kv_heads, 2, group, value_dim)
        o = (a[:, :, 0] - lam * a[:, :, 1]).reshape(rows, heads, value_dim)
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * gain
        out.copy_(o.reshape(rows, heads * value_dim).to(out.dtype))

    def rotary_qkv(self, src, q_out, k_out, v_out, heads, kv_heads, key_dim, value_dim, dims, interleaved, freqs,
                   magnitude, norm_eps, row_pos, value_width=0):
        rows = src.shape[0]
        n_rot = (heads + kv_heads) * key_dim
        turned = torch.empty((rows, n_rot), dtype=torch.float32)
        if dims:
            self.rotary(src[:, :n_rot], turned, heads + kv_heads, key_dim, key_dim, dims, interleaved, freqs, magnitude,
                        row_pos)
        else:
            turned.copy_(src[:, :n_rot].float())
        t = turned.reshape(rows, heads + kv_heads, key_dim)
        if norm_eps is not None:
            t = t / torch.sqrt((t * t).mean(-1, keepdim=True) + norm_eps)
        q_out.copy_(t[:, :heads].reshape(rows, -1).to(q_out.dtype))
        k_out.copy_(t[:, heads:].reshape(rows, -1).to(k_out.dtype))
        v_out.copy_(src[:, n_rot:].to(v_out.dtype))

    def postnorm_residual(self, x, y, scales, weight, eps, extra=None, next_weight=None, next_eps=0.0, h=None):
        pieces = y.float() if y.dim() == 3 else y.float()[None]
        total = pieces[0] * scales[0]
        for piece, sc in zip(pieces[1:], scales[1:]):
            total = total + piece * sc
        x += total / torch.sqrt((total * total).mean(-1, keepdim=True) + eps) * weight
        if extra is not None:
            x += extra
        if h is not None:
            h.copy_((x / torch.sqrt((x * x).mean(-1, keepdim=True) + next_eps) * next_weight).to(h.dtype))

    def scale(self, x, factor):
        x *= factor

    def linear_heads(self, x, w, out, heads, out_head_stride):
        n, k = w.shape[1], w.shape[2]
        for h in range(heads):
            out[:, h * out_head_stride : h * out_head_stride + n] = \
                (x[:, h * k : (h + 1) * k].float() @ w[h].float().t()).to(out.dtype)

    def gla_scan(self, q, k, v, z, bias, state, out, heads, key_dim, value_dim, q_scale, inv_tau, seq_slot, cu_rows,
                 batch):
        for b in range(batch):
            r0, r1 = int(cu_rows[b]), int(cu_rows[b + 1])
            s = state[int(seq_slot[b])]  # [heads, value_dim, key_dim]
            for r in range(r0, r1):
                decay = torch.exp(torch.nn.functional.logsigmoid(z[r].float() + bias) * inv_tau).reshape(heads, key_dim)
                qr = q[r].float().reshape(heads, key_dim) * q_scale
                kr = k[r].float().reshape(heads, key_dim)
                vr = v[r].float().reshape(heads, value_dim)
                s.mul_(decay[:, None, :]).add_(vr[:, :, None] * kr[:, None, :])
                out[r] = (s * qr[:, None, :]).sum(-1).reshape(-1)

    def moe_route(self, logits, route, top, renormalize=False, correction=None, groups=0, keep=0, scoring="sigmoid",
                  group_mark="top2", renormalize_eps=0.0, identity=None):
        s = torch.sigmoid(logits.float()) if scoring == "sigmoid" else torch.softmax(logits.float(), -1)
        c = s + correction if correction is not None else s
        experts = s.shape[1]
        real = route.shape[1]
        route.fill_(-1.0)
        if identity is not None:
            identity.fill_(-1.0)
        for r in range(s.shape[0]):
            allowed = list(range(experts))
            if groups > 1 and keep < groups:
                per = experts // groups
                best = 1 if group_mark == "max" else 2
                marks = [sum(sorted((float(c[r, e]) for e in range(g * per, (g + 1) * per)), reverse=True)[:best])
                         for g in range(groups)]
                kept = sorted(range(groups), key=lambda g: (-marks[g], g))[:keep]
                allowed = [e for e in allowed if e // per in kept]
            chosen = sorted(allowed, key=lambda e: (-float(c[r, e]), e))[:top]
            total = sum(float(s[r, e]) for e in chosen) + renormalize_eps if renormalize else 1.0
            for e in chosen:
                if e < real:
                    route[r, e] = s[r, e] / total
                else:
                    identity[r, e - real] = s[r, e] / total

    def moe_identity(self, h, weights, out):
        w = torch.clamp(weights.float(), min=0.0).sum(-1, keepdim=True)
        out += h.float() * w

    def moe_glu(self, gu, route, out, experts, ff, limit, weight_input=True, activation="clamped_swish"):
        rows = gu.shape[0]
        v = gu.float().reshape(rows, experts, 2, ff)
        w = route.float().reshape(rows, experts)[:, :, None]
        scale = w if weight_input else torch.ones_like(w)
        if activation == "silu":
            g = v[:, :, 0] * scale
            y = g * torch.sigmoid(g) * (v[:, :, 1] * scale)
        else:
            g = torch.clamp(v[:, :, 0] * scale, max=limit)
            u = torch.clamp(v[:, :, 1] * scale, -limit, limit)
            y = g * torch.sigmoid(1.702 * g) * (u + 1)
        if not weight_input:
            y = y * w
        y = torch.where(w >= 0, y, torch.zeros_like(y))
        out.copy_(y.reshape(rows, experts * ff).to(out.dtype))

    def moe_sort(self, route, counts, order, weight, place_of):
        rows, experts = route.shape
        place_of.fill_(-1)
        at = 0
        for e in range(experts):
            mine = [r for r in range(rows) if float(route[r, e]) >= 0]
            counts[e] = len(mine)
            for r in mine:
                order[at], weight.view(-1)[at], place_of[r, e] = r, route[r, e], at
                at += 1

    def moe_gather(self, src, order, dst, n):
        dst[:n] = src[order[:n].long()]

    def moe_scatter(self, ys, place_of, out):
        out.zero_()
        for e in range(place_of.shape[1]):
            at = place_of[:, e].long()
            out += torch.where((at >= 0)[:, None], ys[at.clamp(min=0)], torch.zeros_like(out))
