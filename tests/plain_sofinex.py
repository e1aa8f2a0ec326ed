"""The Sofinex design, plain and slow: float64, whole sequences, no cache, one function per mechanism, written from
the design's equations and sharing nothing with the library.  `rounding=True` rounds activations to bfloat16 where a
bfloat16 run of the library does (what a matrix product reads, what the cache holds), so that such a run can be held
against it.

A layer:  x += mixer(N1(x));  x += ffn(N2(x)),  N(x) = x / sqrt(mean x^2 + eps) (1 + w).
An "attention" layer's mixer is differential attention under a sliding window; a "parallel" layer's mixer is the
half sum of windowed attention with a learned sink and the gated delta rule, each RMS-normed over the width.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rnd(t: torch.Tensor, rounding: bool) -> torch.Tensor:
    return t.to(torch.bfloat16).to(F) if rounding else t


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def one_plus_norm(x: torch.Tensor, eps: float, w: torch.Tensor) -> torch.Tensor:
    return rms(x, eps) * (1.0 + w)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1 + torch.exp(-z))


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2.0)))


def frequencies(rot: dict):
    """-> (frequency of every rotated pair, what cos and sin are multiplied by).  A scaling with `low` and `high`
    blends by wavelength; one with `fast` and `slow` ramps over the pairs' numbers and also stretches cos and sin."""
    dims, base = rot["dims"], rot["base"]
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0
    if "low" in sc:
        out = []
        for fi in f:
            wave = 2 * math.pi / fi
            if wave < sc["original"] / sc["high"]:
                out.append(fi)
            elif wave > sc["original"] / sc["low"]:
                out.append(fi / sc["factor"])
            else:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1 - s) * fi / sc["factor"] + s * fi)
        return torch.tensor(out, dtype=F), 1.0

    def pair_at(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo, hi = max(math.floor(pair_at(sc["fast"])), 0), min(math.ceil(pair_at(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(1.0, max(0.0, (i - lo) / max(hi - lo, 0.001)))
        out.append(fi / sc["factor"] * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(x: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """x [T, ..., dim]: entry i is paired with entry i + dims / 2 (i < dims / 2) and the pair turned by
    position * f_i; entries from dims on pass."""
    if not rot:
        return x
    f, mag = frequencies(rot)
    dims, half = rot["dims"], rot["dims"] // 2
    ang = torch.arange(x.shape[0], dtype=F)[:, None] * f[None, :]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (half,)
    c, s = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
    u, v = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def window_mask(T: int, size: Optional[int]) -> torch.Tensor:
    """[T, T] true where row i sees column j: 0 <= i - j < size (no size: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & (i - j < (T if size is None else size))


def window_of(m: dict) -> Optional[int]:
    return m["mask"]["size"] if m.get("mask") else None


def softmax_rows(score: torch.Tensor, seen: torch.Tensor, sink: Optional[float] = None) -> torch.Tensor:
    """Softmax over the seen columns of every row; with a sink the denominator has one more term exp(sink)."""
    score = score.masked_fill(~seen, -math.inf)
    top = score.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.clamp(top, min=sink)
    e = torch.exp(score - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink - top)
    return e / total


def sink_attention(h, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, rounding: bool) -> torch.Tensor:
    T, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rotate_half((h @ w[p + ".q"].T).view(T, H, d), m.get("rot"))
    k = rotate_half((h @ w[p + ".k"].T).view(T, G, d), m.get("rot"))
    q, k = rnd(rms(q, eps), rounding), rnd(rms(k, eps), rounding)
    v = rnd((h @ w[p + ".v"].T).view(T, G, vd), rounding)
    seen = window_mask(T, window_of(m))
    out = torch.zeros(T, H, vd, dtype=F)
    for n in range(H):
        g = n // (H // G)
        score = (q[:, n] @ k[:, g].T) * m["scale"]
        out[:, n] = softmax_rows(score, seen, float(w[p + ".sink"][n])) @ v[:, g]
    return rnd(out.reshape(T, H * vd), rounding) @ w[p + ".o"].T


def differential_lambda(w: Dict[str, torch.Tensor], p: str, diff: float) -> float:
    return float(torch.exp((w[p + ".lq1"] * w[p + ".lk1"]).sum()) - torch.exp((w[p + ".lq2"] * w[p + ".lk2"]).sum())
                 + diff)


def differential_attention(h, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, rounding: bool) -> torch.Tensor:
    """Two score maps a head, [map 1 | map 2] in q and k, over the same values: o = a1 - lambda a2, divided by its
    root mean square over the head's values, times (1 - diff)."""
    T, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rnd(rotate_half((h @ w[p + ".q"].T).view(T, H, 2, d), m.get("rot")), rounding)
    k = rnd(rotate_half((h @ w[p + ".k"].T).view(T, G, 2, d), m.get("rot")), rounding)
    v = rnd((h @ w[p + ".v"].T).view(T, G, vd), rounding)
    seen = window_mask(T, window_of(m))
    lam = differential_lambda(w, p, m["diff"])
    out = torch.zeros(T, H, vd, dtype=F)
    for n in range(H):
        g = n // (H // G)
        maps = [softmax_rows((q[:, n, j] @ k[:, g, j].T) * m["scale"], seen) @ v[:, g] for j in range(2)]
        out[:, n] = rms(maps[0] - lam * maps[1], eps) * (1.0 - m["diff"])
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


def delta_rule(h, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, rounding: bool) -> torch.Tensor:
    T, H, G, d, vd = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
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
    o = rms(o, eps) * w[p + ".norm"] * gate
    return rnd(o.reshape(T, H * vd), rounding) @ w[p + ".o"].T


def side_by_side(h, m: dict, w, p: str, eps: float, rounding: bool) -> torch.Tensor:
    left = sink_attention(h, m["left"], w, p + ".left", eps, rounding)
    right = delta_rule(h, m["right"], w, p + ".right", eps, rounding)
    return 0.5 * (rms(left, eps) * w[p + ".left.out"] + rms(right, eps) * w[p + ".right.out"])


def dense(h, w, p: str, rounding: bool) -> torch.Tensor:
    return rnd(gelu_erf(h @ w[p + ".up"].T), rounding) @ w[p + ".down"].T


def gated_expert(h, w, p: str, rounding: bool, weight=1.0) -> torch.Tensor:
    return rnd(weight * silu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T), rounding) @ w[p + ".down"].T


def route(h, r: dict, w, p: str):
    """-> (softmax scores [T, experts + identity], every token's chosen outputs of the router).  The choice is by
    score + correction, within the groups whose best choice score is highest; ties go to the lower number."""
    n_out, top = r["experts"] + r.get("identity", 0), r["top"]
    s = torch.softmax(h @ w[p + ".router"].T, -1)
    choice = s + w[p + ".correction"]
    groups = r.get("groups")
    chosen = []
    for t in range(h.shape[0]):
        allowed = list(range(n_out))
        if groups and groups["count"] > 1:
            per = n_out // groups["count"]
            marks = [max(float(choice[t, e]) for e in range(g * per, (g + 1) * per)) for g in range(groups["count"])]
            kept = sorted(range(groups["count"]), key=lambda g: (-marks[g], g))[: groups["keep"]]
            allowed = [e for e in allowed if e // per in kept]
        chosen.append(sorted(allowed, key=lambda e: (-float(choice[t, e]), e))[:top])
    return s, chosen


def experts(h, mlp: dict, w, p: str, rounding: bool) -> torch.Tensor:
    r = mlp["router"]
    s, chosen = route(h, r, w, p)
    out = torch.zeros(h.shape[0], w[p + ".e0.down"].shape[0], dtype=F)
    for t, es in enumerate(chosen):
        total = sum(s[t, e] for e in es) + 1e-20
        for e in es:
            share = s[t, e] / total
            if e >= r["experts"]:  # an identity expert: its input, weighted
                out[t] += share * h[t]
            else:
                out[t] += gated_expert(h[t : t + 1], w, f"{p}.e{e}", rounding, weight=share)[0]
    if mlp.get("shared"):
        open_ = torch.sigmoid(h @ w[p + ".shared.sg"].T)  # [T, 1]
        out = out + gated_expert(h, w, p + ".shared", rounding, weight=open_)
    return out


def run_order(cfg: dict) -> List[int]:
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(n))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] \
        + list(range(loop["stop"], n))


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], rounding: bool = False,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; `layers_out` takes the stream after every layer run."""
    w = {k: v.to(F) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    for i in run_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}"
        h = rnd(one_plus_norm(x, eps, w[p + ".norm1"]), rounding)
        if layer["type"] == "attention":
            x = x + differential_attention(h, layer["mixer"], w, p + ".mix", eps, rounding)
        else:
            x = x + side_by_side(h, layer["mixer"], w, p + ".mix", eps, rounding)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rnd(one_plus_norm(x, eps, w[p + ".norm2"]), rounding)
            x = x + (dense(h, w, p + ".mlp", rounding) if mlp["kind"] == "dense"
                     else experts(h, mlp, w, p + ".mlp", rounding))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rnd(one_plus_norm(x, eps, w["final.norm"]), rounding) @ w["head"].T
