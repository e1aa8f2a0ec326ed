"""The Mifidra design, plain and slow: float64, whole sequences, no cache, one function per mechanism, written from
the design's equations and sharing nothing with the library.  `rounding=True` rounds activations to bfloat16 where a
bfloat16 run of the library does (what a matrix product reads), so that such a run can be held against it.

A layer:  x += N1b(mixer(N1(x)));  x += N2b(ffn(N2(x))), every N an RMS norm with a weight.
The mixer:  c_l * attention(h) + c_r * delta(h) on the same h.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rnd(t: torch.Tensor, rounding: bool) -> torch.Tensor:
    return t.to(torch.bfloat16).to(F) if rounding else t


def rms_norm(x: torch.Tensor, eps: float, w: Optional[torch.Tensor] = None) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1 + torch.exp(-z))


def rotary_table(rot: dict):
    """Frequencies of the rotated pairs and what cos and sin are multiplied by."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0

    def pair_at(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo, hi = max(math.floor(pair_at(sc["fast"])), 0), min(math.ceil(pair_at(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(fi / sc["factor"] * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """x [T, heads, dim]: entries (2i, 2i + 1), i < dims / 2, turned by position * f_i; the rest pass."""
    if not rot:
        return x
    f, mag = rotary_table(rot)
    dims = rot["dims"]
    ang = torch.arange(x.shape[0], dtype=F)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, rounding: bool) -> torch.Tensor:
    T, H, G, d, vd = h.shape[0], m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = rotate((h @ w[p + ".q"].T).view(T, H, d), m.get("rot"))
    k = rotate((h @ w[p + ".k"].T).view(T, G, d), m.get("rot"))
    q, k = rnd(rms_norm(q, eps), rounding), rnd(rms_norm(k, eps), rounding)
    v = rnd((h @ w[p + ".v"].T).view(T, G, vd), rounding)
    seen = torch.tril(torch.ones(T, T, dtype=torch.bool))
    out = torch.zeros(T, H, vd, dtype=F)
    for n in range(H):
        g = n // (H // G)
        score = (q[:, n] @ k[:, g].T) * m["scale"]
        out[:, n] = torch.softmax(score.masked_fill(~seen, -math.inf), -1) @ v[:, g]
    return rnd(out.reshape(T, H * vd), rounding) @ w[p + ".o"].T


def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y_t = silu(sum_j taps[:, j] x_{t - (n - 1) + j}), zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, C, dtype=F), x], 0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(n):
        y += padded[j : j + T] * taps[:, j]
    return silu(y)


def delta_rule(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, rounding: bool) -> torch.Tensor:
    T, H, G, d, vd = h.shape[0], m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = short_conv(h @ w[p + ".q"].T, w[p + ".q.conv"]).view(T, G, d)
    k = short_conv(h @ w[p + ".k"].T, w[p + ".k.conv"]).view(T, G, d)
    v = short_conv(h @ w[p + ".v"].T, w[p + ".v.conv"]).view(T, H, vd)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].T)
    step = torch.nn.functional.softplus(rnd(h @ w[p + ".a1"].T, rounding) @ w[p + ".a2"].T + w[p + ".dt_bias"],
                                        threshold=1e9).view(T, H, d)
    decay = torch.exp(-torch.exp(w[p + ".A_log"])[None, :, None] * step)
    gate = torch.sigmoid(rnd(h @ w[p + ".g1"].T, rounding) @ w[p + ".g2"].T).view(T, H, vd)
    o = torch.zeros(T, H, vd, dtype=F)
    for n in range(H):
        g = n // (H // G)
        S = torch.zeros(d, vd, dtype=F)
        for t in range(T):
            S = decay[t, n][:, None] * S
            u = beta[t, n] * (v[t, n] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, n] = S.T @ q[t, g]
    o = rms_norm(o, eps) * w[p + ".norm"] * gate
    return rnd(o.reshape(T, H * vd), rounding) @ w[p + ".o"].T


def mixer(h, m: dict, w, p: str, eps: float, rounding: bool) -> torch.Tensor:
    return m["left_scale"] * attention(h, m["left"], w, p + ".left", eps, rounding) \
        + m["right_scale"] * delta_rule(h, m["right"], w, p + ".right", eps, rounding)


def dense(h, w, p: str, rounding: bool) -> torch.Tensor:
    act = silu(h @ w[p + ".gate"].T + w[p + ".gate.b"]) * (h @ w[p + ".up"].T + w[p + ".up.b"])
    return rnd(act, rounding) @ w[p + ".down"].T + w[p + ".down.b"]


def expert(h, w, p: str, rounding: bool, weight=1.0) -> torch.Tensor:
    return rnd(weight * silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T), rounding) @ w[p + ".down"].T


def route(h, r: dict, w, p: str):
    """-> (scores [T, E], the chosen experts of every token)."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(h @ w[p + ".router"].T)
    choice = s + w[p + ".correction"]
    groups = r.get("groups")
    chosen = []
    for t in range(h.shape[0]):
        allowed = list(range(E))
        if groups and groups["count"] > 1:
            per = E // groups["count"]
            marks = [sum(sorted((float(choice[t, e]) for e in range(g * per, (g + 1) * per)), reverse=True)[:2])
                     for g in range(groups["count"])]
            kept = sorted(range(groups["count"]), key=lambda g: (-marks[g], g))[: groups["keep"]]
            allowed = [e for e in allowed if e // per in kept]
        chosen.append(sorted(allowed, key=lambda e: (-float(choice[t, e]), e))[:top])
    return s, chosen


def experts(h, mlp: dict, w, p: str, rounding: bool) -> torch.Tensor:
    s, chosen = route(h, mlp["router"], w, p)
    out = torch.zeros(h.shape[0], w[p + ".e0.down"].shape[0], dtype=F)
    for t, es in enumerate(chosen):
        for e in es:
            out[t] += expert(h[t : t + 1], w, f"{p}.e{e}", rounding, weight=s[t, e])[0]
    if mlp.get("shared"):
        out = out + expert(h, w, p + ".shared", rounding)
    return out


def run_order(cfg: dict):
    """(layer, whether the input is fed in again ahead of it), in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t > 0 and i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], rounding: bool = False,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; `layers_out` takes the stream after every layer run."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.tensor(tokens)]
    x = x0.clone()
    for i, again in run_order(cfg):
        if again:
            x = x + x0
        layer, p = cfg["layers"][i], f"l{i}"
        h = rnd(rms_norm(x, eps, w[p + ".norm1"]), rounding)
        x = x + rms_norm(mixer(h, layer["mixer"], w, p + ".mix", eps, rounding), eps, w[p + ".norm1b"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rnd(rms_norm(x, eps, w[p + ".norm2"]), rounding)
            y = dense(h, w, p + ".mlp", rounding) if mlp["kind"] == "dense" else experts(h, mlp, w, p + ".mlp", rounding)
            x = x + rms_norm(y, eps, w[p + ".norm2b"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rnd(rms_norm(x, eps, w["final.norm"]), rounding) @ w["embed"].T) * cfg.get("logit_scale", 1.0)
