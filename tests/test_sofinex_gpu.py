"""The Sofinex design on the GPU.  First every kernel that the design brought, or widened, alone against the plain
implementation's function of the same mechanism (float64), with inputs made so that a fault shows; then the engine
in float32 and in bfloat16 under every cutting and batching; then generation through the entry point, with captured
steps and direct ones, the command line and the trace replay."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import longbow_quarrel_amd as lq
import plain_sofinex as ps
import sofinex_cases as sc
from longbow_quarrel_amd.engine import StepEntry

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
TOL_F32 = 2e-5
F = torch.float64


@pytest.fixture(scope="module")
def kn():
    from longbow_quarrel_amd.kernels.hip import HipKernels
    return HipKernels()


def rnd(*shape, seed=0, std=1.0):
    return torch.empty(shape).normal_(0, std, generator=torch.Generator().manual_seed(seed))


def i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def dev(t, dtype=torch.float32):
    return t.to(dtype).to(DEV).contiguous()


def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, device=DEV, max_slots=8,
                          max_sequence_tokens=max_tokens)


class Paged:
    """A sequence's keys and values in a paged cache whose blocks lie in no particular order."""

    def __init__(self, length, kv_heads, key_dim, value_dim, dtype, bs=64, seed=0):
        n = (length + bs - 1) // bs
        order = torch.randperm(n + 3, generator=torch.Generator().manual_seed(seed)).tolist()
        self.table = torch.tensor([order[:n]], dtype=torch.int32, device=DEV)
        self.k = torch.zeros((n + 3, kv_heads, bs, key_dim), dtype=dtype, device=DEV)
        self.v = torch.zeros((n + 3, kv_heads, value_dim, bs), dtype=dtype, device=DEV)


def plain_maps(q, k, v, scale, window, sinks=None):
    """q [T, H, D], k [T, G, D], v [T, G', P] with G a multiple of G' (key heads that share a value head):
    windowed softmax attention of every query head over its key head, optionally with a sink score a head."""
    T, H, G, Gv = q.shape[0], q.shape[1], k.shape[1], v.shape[1]
    seen = ps.window_mask(T, window)
    out = torch.zeros(T, H, v.shape[2], dtype=F)
    for n in range(H):
        g = n // (H // G)
        p = ps.softmax_rows((q[:, n] @ k[:, g].T) * scale, seen, None if sinks is None else float(sinks[n]))
        out[:, n] = p @ v[:, g // (G // Gv)]
    return out


# ---- the kernels alone -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [
    # query heads, key heads, maps, key size, value size, window, learned sink, generic kernel
    (4, 2, 1, 32, 16, 7, True, False), (8, 4, 2, 16, 48, 70, False, False), (6, 2, 2, 48, 96, 64, False, False),
    (3, 1, 1, 16, 16, 65, True, False), (2, 2, 2, 24, 40, 9, False, False), (4, 4, 2, 64, 64, 0, False, False),
    (8, 4, 2, 16, 48, 70, False, True), (4, 2, 1, 32, 16, 7, True, True), (2, 2, 2, 10, 7, 63, False, False),
    (12, 4, 2, 32, 32, 130, False, False), (5, 5, 1, 20, 12, 1, True, False),
])
def test_windowed_attention_with_a_learned_sink_and_maps_that_share_values(kn, sizes, dtype):
    """Rows of a prompt and the same rows as single tokens.  Every eighth row's query is aimed at one key (its score
    stands out): the key just inside the window, just outside it, a key at a cache block's edge, in turn.  With
    `maps` the cached key row of a value head holds the keys of several key heads side by side; the result is 32-bit
    whatever the cache holds."""
    H, G, maps, D, P, window, sink, generic = sizes
    T = 200
    Gv = G // maps
    q, k, v = rnd(T, H, D, seed=1), rnd(T, G, D, seed=2), rnd(T, Gv, P, seed=3)
    sinks = rnd(H, seed=4, std=2.0) if sink else None
    w = window if window else T
    for n, i in enumerate(range(70, T, 8)):
        j = [i - w + 1, i - w, (i // 64) * 64, (i // 64) * 64 - 1][n % 4]
        if 0 <= j <= i:
            for h in range(H):
                q[i, h] = k[j, h // (H // G)] * 6.0 / k[j, h // (H // G)].norm()
    q, k, v = (t.to(dtype).double() for t in (q, k, v))  # what the kernel is given, exactly
    scale = 1.3 / math.sqrt(D)
    want = plain_maps(q, k, v, scale, w, None if sinks is None else sinks.double()).reshape(T, H * P)
    if sink:  # the sink takes weight: without it the result differs by much
        assert sc.err(plain_maps(q, k, v, scale, w).reshape(T, H * P), want) > 1e-2
    cache = Paged(T, Gv, maps * D, P, dtype, seed=5)
    pos, seq, slot = i32(range(T)), i32([0] * T), i32([0])
    kn.force_generic = generic
    try:
        # a position's keys of the key heads that share a value head are one cached row
        kn.kv_store(dev(k.reshape(T, -1), dtype), dev(v.reshape(T, -1), dtype), Gv, maps * D, P, pos, seq, slot,
                    cache.table, cache.k, cache.v, 64)
        qd = dev(q.reshape(T, -1), dtype)
        more = dict(window=window, keep_first=0, sink=sink, maps=maps)
        if sink:
            more["sink_values"] = dev(sinks)
        for out_dtype in {dtype, torch.float32}:
            out = torch.zeros((T, H * P), dtype=out_dtype, device=DEV)
            kn.sink_attention(qd, out, H, G, D, P, pos, seq, slot, cache.table, cache.k, cache.v, 64, scale, **more)
            tol = 1e-5 if dtype == torch.float32 else (1e-2 if out_dtype == torch.bfloat16 else 2e-5)
            # (a bfloat16 cache with 32-bit results: exact products of what the cache holds, 32-bit sums)
            assert sc.err(out, want) < tol, out_dtype
        for r in list(range(60, 76)) + [127, 128, 129, 191, 199]:  # single tokens, over block edges too
            one = torch.zeros((1, H * P), dtype=torch.float32, device=DEV)
            kn.sink_attention(qd[r : r + 1], one, H, G, D, P, i32([r]), i32([0]), slot, cache.table, cache.k, cache.v,
                              64, scale, decode=True, **more)
            assert sc.err(one[0], want[r]) < 2e-5, r
            if dtype == torch.float32 and not generic:
                assert torch.equal(one[0], out[r]), r  # the same sums in the same order
    finally:
        kn.force_generic = False


@pytest.mark.parametrize("sizes", [
    # query heads, key heads, maps, key size, value size, window, learned sink
    (4, 2, 1, 32, 48, 0, True), (4, 2, 1, 32, 48, 700, True), (8, 4, 2, 16, 80, 0, False), (6, 2, 2, 48, 96, 520, False),
])
def test_single_tokens_whose_keys_are_shared_out_over_workgroups(kn, sizes):
    """A bfloat16 step of single tokens over many cached keys: a tile's keys go to several workgroups and a second
    launch merges them.  The sink's term must count once (the first workgroup's first wavefront starts from it), and
    every workgroup must read its map's half of the cached key rows."""
    H, G, maps, D, P, window, sink = sizes
    T, dtype = 1500, torch.bfloat16
    Gv = G // maps
    q, k, v = rnd(T, H, D, seed=1), rnd(T, G, D, seed=2), rnd(T, Gv, P, seed=3)
    sinks = rnd(H, seed=4, std=1.0) + 3.0 if sink else None  # (a sink that takes a large share of the weight)
    q, k, v = (t.to(dtype).double() for t in (q, k, v))
    scale = 1.0 / math.sqrt(D)
    want = plain_maps(q, k, v, scale, window if window else T, None if sinks is None else sinks.double()).reshape(T, H * P)
    if sink:
        assert sc.err(plain_maps(q, k, v, scale, window if window else T).reshape(T, H * P), want) > 5e-2
    cache = Paged(T, Gv, maps * D, P, dtype, seed=5)
    pos, seq, slot = i32(range(T)), i32([0] * T), i32([0])
    kn.kv_store(dev(k.reshape(T, -1), dtype), dev(v.reshape(T, -1), dtype), Gv, maps * D, P, pos, seq, slot, cache.table,
                cache.k, cache.v, 64)
    qd = dev(q.reshape(T, -1), dtype)
    more = dict(window=window, keep_first=0, sink=sink, maps=maps)
    if sink:
        more["sink_values"] = dev(sinks)
    need = kn.sink_attention_workspace(dtype, 1, 1, H, G, D, P, 64, window, 0, T)
    assert need > 0
    scratch = torch.zeros(need, device=DEV)
    for r in (T - 1, 1100, 800, 767, 700):
        for out_dtype in (torch.float32, dtype):
            one = torch.zeros((1, H * P), dtype=out_dtype, device=DEV)
            kn.sink_attention(qd[r : r + 1], one, H, G, D, P, i32([r]), i32([0]), slot, cache.table, cache.k, cache.v, 64,
                              scale, decode=True, max_len=T, workspace=scratch, **more)
            assert sc.err(one[0], want[r]) < (2e-5 if out_dtype == torch.float32 else 1e-2), (r, out_dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 48), (3, 3, 7), (6, 1, 96), (2, 1, 130), (8, 4, 16)])
def test_difference_of_two_maps_and_its_norm(kn, sizes, dtype):
    """The maps' results lie (key/value head, map, query head of the group); lambda near one makes the difference
    small against both maps, and the norm brings it back to size."""
    H, G, P = sizes
    rows, group = 37, H // G
    a1 = rnd(rows, H, P, seed=1)
    a2 = a1 + 0.01 * rnd(rows, H, P, seed=2)
    both = torch.stack([a1.reshape(rows, G, group, P), a2.reshape(rows, G, group, P)], dim=2).reshape(rows, 2 * H * P)
    for lam, eps, gain in ((0.97, 1e-6, 0.4), (-0.3, 1e-3, 1.0), (1.0, 1e-5, 0.2)):
        o = a1.double() - lam * a2.double()
        want = (ps.rms(o, eps) * gain).reshape(rows, H * P)
        out = torch.zeros((rows, H * P), dtype=dtype, device=DEV)
        kn.diff_combine(dev(both), out, H, G, P, lam, eps, gain)
        assert sc.err(out, want) < (3e-5 if dtype == torch.float32 else 1e-2), (lam, eps)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(4, 2, 2, 24, 40, 16), (2, 1, 2, 10, 7, 6), (8, 2, 2, 64, 32, 64), (3, 3, 1, 8, 24, 8)])
def test_rotation_of_half_split_pairs_of_every_map(kn, dtype, sizes):
    """Every map of every head is a head to the rotation: entry i with entry i + dims / 2, the rest pass; the values
    of key heads that share a value head pass as they are; no norm unless asked for."""
    H, G, maps, D, P, dims = sizes
    rows = 50
    freqs = torch.tensor([777.0 ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    pos = torch.randint(0, 100000, (rows,), generator=torch.Generator().manual_seed(1))
    pos[0] = 0
    vw = G * P
    src = rnd(rows, (H + G) * maps * D + vw, seed=2)
    q = torch.zeros((rows, H * maps * D), dtype=dtype, device=DEV)
    k = torch.zeros((rows, G * maps * D), dtype=dtype, device=DEV)
    v = torch.zeros((rows, vw), dtype=dtype, device=DEV)
    for eps in (None, 1e-5):
        kn.rotary_qkv(dev(src), q, k, v, maps * H, maps * G, D, P, dims, False, freqs.to(DEV), 1.15, eps, i32(pos.tolist()),
                      value_width=vw)
        heads = src[:, : (H + G) * maps * D].double().reshape(rows, (H + G) * maps, D)
        ang = pos.double()[:, None] * freqs[None, :]
        c, s = (torch.cos(ang) * 1.15)[:, None, :], (torch.sin(ang) * 1.15)[:, None, :]
        want = heads.clone()
        a, b = heads[..., : dims // 2], heads[..., dims // 2 : dims]
        want[..., : dims // 2], want[..., dims // 2 : dims] = a * c - b * s, b * c + a * s
        if eps is not None:
            want = ps.rms(want, eps)
        tol = 2e-5 if dtype == torch.float32 else 1e-2
        assert sc.err(q, want[:, : H * maps].reshape(rows, -1)) < tol and sc.err(k, want[:, H * maps :].reshape(rows, -1)) < tol
        assert sc.err(v, src[:, (H + G) * maps * D :].double()) < tol


def test_exact_gelu_and_a_gate_a_row_on_a_gated_unit(kn):
    rows = 33
    for inner in (70, 72, 1024):  # (columns in fours go four a thread)
        x = rnd(rows, inner, seed=1, std=2.5)
        for dtype in (torch.float32, torch.bfloat16):
            out = torch.zeros((rows, inner), dtype=dtype, device=DEV)
            kn.activation(dev(x), out, "gelu")
            assert sc.err(out, ps.gelu_erf(x.double())) < (2e-6 if dtype == torch.float32 else 1e-2)
            wide = torch.full((rows, inner + 8), 7.0, dtype=dtype, device=DEV)  # rows with a stride of their own
            kn.activation(dev(torch.cat([x, x[:, :4]], 1))[:, :inner], wide[:, :inner], "silu")
            assert sc.err(wide[:, :inner], ps.silu(x.double())) < (2e-6 if dtype == torch.float32 else 1e-2)
            assert bool((wide[:, inner:] == 7.0).all())
    inner = 70
    # the tanh form is another function, further off than the kernel's limit above
    xd = x.double()
    tanh_form = 0.5 * xd * (1 + torch.tanh(math.sqrt(2 / math.pi) * (xd + 0.044715 * xd ** 3)))
    assert sc.err(ps.gelu_erf(xd), tanh_form) > 2e-5
    gu = rnd(rows, 2 * inner, seed=2, std=2.0)
    z = rnd(rows, 5, seed=3, std=2.0)  # the gate's logit is one column of a wider product
    out = torch.zeros((rows, inner), device=DEV)
    kn.glu(dev(gu), out, "silu", row_gate=dev(z)[:, 3:4])
    want = ps.silu(gu[:, :inner].double()) * gu[:, inner:].double() * torch.sigmoid(z[:, 3:4].double())
    assert sc.err(out, want) < 2e-6


def test_router_with_softmax_scores_identity_experts_and_the_best_groups_by_their_best_score(kn):
    """Against the plain router, row by row: softmax over all outputs, the choice by score plus correction
    (corrections large enough to turn the order over, and negative enough that choice scores below zero are common),
    a group's mark its best choice score, weights renormalised over the chosen, identity experts' weights apart."""
    rows = 200
    for E, ident, top, groups, keep in ((12, 4, 5, 4, 3), (4, 2, 2, 3, 2), (9, 3, 3, 4, 2), (8, 0, 8, 2, 2), (2, 2, 2, 4, 2),
                                        (8, 1, 3, 3, 1), (5, 2, 3, 0, 0), (1, 3, 2, 2, 1), (48, 16, 6, 8, 3)):
        N = E + ident
        z = rnd(rows, N, seed=N + top, std=2.0)
        corr = rnd(N, seed=N, std=0.2) - 0.2
        if groups:
            z[5, :] = -3.0
            z[5, 0], z[5, N // groups], z[5, N // groups + 1] = 1.0, 0.9, 0.9  # the best one against the best pair
        route = torch.zeros(rows, E, device=DEV)
        passed = torch.zeros(rows, max(ident, 1), device=DEV)
        kn.moe_route(dev(z), route, top, True, correction=dev(corr), groups=groups, keep=keep, scoring="softmax",
                     group_mark="max", renormalize_eps=1e-20, identity=passed[:, :ident] if ident else None)
        r = {"experts": E, "identity": ident, "top": top}
        if groups:
            r["groups"] = {"count": groups, "keep": keep}
        s, chosen = ps.route(z.double(), r, {"m.router": torch.eye(N, dtype=F), "m.correction": corr.double()}, "m")
        got = torch.cat([route.cpu(), passed.cpu()[:, :ident]], dim=1)
        close = 0
        for t in range(rows):
            mine = [e for e in range(N) if got[t, e] >= 0]
            if mine != sorted(chosen[t]):
                # only a call closer than 32-bit rounding may fall the other way
                c = (s[t] + corr.double()).tolist()
                diff = set(mine) ^ set(chosen[t])
                assert len(mine) == top and max(c[e] for e in diff) - min(c[e] for e in diff) < 1e-6, (E, t)
                close += 1
                continue
            total = sum(float(s[t, e]) for e in mine)
            for e in mine:
                assert float(got[t, e]) == pytest.approx(float(s[t, e]) / total, rel=3e-6, abs=1e-9)
        assert close <= 1
        assert bool(((got >= 0).sum(-1) == top).all())
        if ident:  # the identity experts' share: the input times their weights' sum
            h = rnd(rows, 50, seed=7)
            for dtype in (torch.float32, torch.bfloat16):
                out = dev(rnd(rows, 50, seed=8))
                kn.moe_identity(dev(h, dtype), passed[:, :ident], out)
                share = torch.clamp(passed.cpu()[:, :ident].double(), min=0).sum(-1, keepdim=True)
                assert sc.err(out, rnd(rows, 50, seed=8).double() + h.to(dtype).double() * share) < 2e-6


# ---- the engine ------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, dtype="float32", **kw):
        key = (name, dtype, tuple(sorted((k, str(v)) for k, v in kw.items())))
        if key not in made:
            made[key] = sc.Case(tmp_path_factory.mktemp("sofinex"), name, load, dtype=dtype,
                                rounding=dtype == "bfloat16", **kw)
        return made[key]

    return get


@pytest.mark.parametrize("name", ["diff", "sink", "delta", "dense", "moe", "loop"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    sc.whole_and_token_by_token(case, TOL_F32, lengths=(1, 2, 9, 70))
    sc.portions(case, TOL_F32, n=140)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_under_every_cutting_and_batching(cases, name):
    case = cases(name)
    sc.whole_and_token_by_token(case, TOL_F32)
    sc.portions(case, TOL_F32)
    sc.unequal_batches(case, TOL_F32)
    sc.slots_and_blocks_used_again(case, TOL_F32)


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("c", "float32"), ("c", "bfloat16")])
def test_prompt_rows_sorted_by_expert(cases, name, dtype, monkeypatch):
    """The same logits whether a prompt's rows run through all experts' columns or are sorted by expert."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    case = cases(name, dtype)
    t = sc.tokens(300, case.vocab, 12)
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 10 ** 9)
    every = case.run_cut(t, [300])
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    by_expert = case.run_cut(t, [200, 3, 90])
    if dtype == "float32":
        assert sc.err(by_expert, case.want(t)) < TOL_F32 and sc.err(by_expert, every) < TOL_F32
    else:
        sc.assert_close_bf16(by_expert, case.want(t), case.noise(t))


@pytest.mark.parametrize("seed", range(1, 13))
def test_configurations_drawn_from_a_seed(cases, seed):
    """Other sizes, head counts, windows, rotations, layer orders, loops, experts, groups and constants, in both
    dtypes."""
    case = cases(seed)
    t, u = sc.tokens(200, case.vocab, seed), sc.tokens(9, case.vocab, seed + 50)
    assert sc.err(case.run_cut(t, [150, 2, 1, 20]), case.want(t)) < TOL_F32
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:130], range(130))])
    assert sc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:130]])) < TOL_F32
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[130:131], [0])])
    assert sc.err(out, torch.stack([case.want(u)[8], case.want(t)[130]])) < TOL_F32
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()
    case16 = cases(seed, "bfloat16")
    sc.assert_close_bf16(case16.run_cut(t, [150, 2]), case16.want(t), case16.noise(t))


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(sc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 9
    for i, (g, w) in enumerate(zip(got, want)):
        assert sc.err(g, w) < TOL_F32, f"after layer run {i}"


@pytest.mark.parametrize("kind", ["diff", "sink"])
@pytest.mark.parametrize("window", [1, 2, 63, 64, 65, 130])
def test_keys_just_inside_and_just_outside_the_window(cases, kind, window):
    """Peaked attention under windows of one token, of a cache block less one, a block, a block and one, and two
    blocks and two: the last key a row sees and the first it does not, in a prompt, across portions and in
    decoding.  The plain implementation with a window one token off differs by much at these rows."""
    case = cases(f"{kind}-window-{window}", cfg=sc.windowed(kind, window), sharp=6.0)
    n = max(2 * window + 10, 80)
    t = sc.tokens(n, case.vocab, 40 + window)
    sc.a_window_off_by_one_would_show(case, t, kind, list(range(window, n)))
    want = case.want(t)
    assert sc.err(case.run_cut(t, [n]), want) < TOL_F32
    assert sc.err(case.run_cut(t, [window, 1, 1, 2, window - 1 or 1, 3]), want) < TOL_F32
    assert sc.err(case.run_cut(t, [max(1, window - 1)]), want) < TOL_F32  # decoding across the window's edge
    case.assert_idle()
    case16 = cases(f"{kind}-window-{window}", "bfloat16", cfg=sc.windowed(kind, window), sharp=6.0)
    sc.assert_close_bf16(case16.run_cut(t, [max(1, window - 1)]), case16.want(t), case16.noise(t))


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_bfloat16_whole_in_portions_and_in_batches(cases, name):
    case = cases(name, "bfloat16")
    t = sc.tokens(150, case.vocab, 3)
    want, noise = case.want(t), case.noise(t)
    sc.assert_close_bf16(case.run_cut(t, [150]), want, noise)
    sc.assert_close_bf16(case.run_cut(t, [64, 1, 63, 2, 3]), want, noise)
    u = sc.tokens(70, case.vocab, 4)
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, t[:100], range(100)), StepEntry(sb, u[:3], range(3))])
    sc.assert_close_bf16(out, torch.cat([want[:100], case.want(u)[:3]]), noise)
    got = []
    for i in range(20):
        got.append(eng.step([StepEntry(sb, [u[3 + i]], [0]), StepEntry(sa, [t[100 + i]], [0])]).clone())
    got = torch.cat(got)
    sc.assert_close_bf16(torch.cat([got[0::2], got[1::2]]), torch.cat([case.want(u)[3:23], want[100:120]]), noise)
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_bfloat16_decoding_over_long_contexts(cases):
    """Single tokens over several hundred positions (the windows long since full, their first blocks given back)
    against the same rows as parts of a prompt and against the plain implementation."""
    case = cases("c", "bfloat16")
    t, u = sc.tokens(640, case.vocab, 61), sc.tokens(330, case.vocab, 62)
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    whole = eng.step([StepEntry(sa, t, range(600, 640)), StepEntry(sb, u, range(290, 330))]).clone()
    eng.release(sa)
    eng.release(sb)
    sa, sb = eng.new_sequence(), eng.new_sequence()
    eng.step([StepEntry(sa, t[:600], []), StepEntry(sb, u[:290], [])])
    got = torch.cat([eng.step([StepEntry(sa, [t[600 + i]], [0]), StepEntry(sb, [u[290 + i]], [0])]).clone() for i in range(40)])
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()
    got = torch.cat([got[0::2], got[1::2]])
    want = torch.cat([case.want(t)[600:], case.want(u)[290:]])
    noise = max(case.noise(t), case.noise(u))
    sc.assert_close_bf16(got, want, noise)
    sc.assert_close_bf16(got, whole.double(), noise)


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    case = cases("delta", memory=7.0)
    t = sc.tokens(260, case.vocab, 31)
    want = case.want(t)
    other = case.want([(t[0] + 1) % case.vocab] + t[1:])
    assert sc.err(other[-1], want[-1]) > 1e-3  # the first token still matters at the end, far beyond the window
    assert sc.err(case.run_cut(t, [260]), want) < TOL_F32
    assert sc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL_F32


def test_the_first_tokens_see_zeros_ahead_of_the_sequence(cases):
    case = cases("a")
    eng = case.eng
    a, b = sc.tokens(150, case.vocab, 1), sc.tokens(6, case.vocab, 2)
    sa = eng.new_sequence()
    eng.step([StepEntry(sa, a, [])])
    eng.release(sa)
    for first in (1, 2, 3, 6):
        s = eng.new_sequence()
        assert s == sa
        out = eng.step([StepEntry(s, b[:first], range(first))])
        assert sc.err(out, case.want(b)[:first]) < TOL_F32
        if first < 6:
            out = eng.step([StepEntry(s, b[first:], range(6 - first))])
            assert sc.err(out, case.want(b)[first:]) < TOL_F32
        eng.release(s)
    case.assert_idle()


@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(cases, name):
    sc.long_decoding(cases(name), TOL_F32)


def test_float32_logits_do_not_depend_on_the_cutting_or_the_batch_by_more_than_rounding(cases):
    case = cases("a")
    t, u = sc.tokens(140, case.vocab, 7), sc.tokens(30, case.vocab, 8)
    whole = case.run_cut(t, [140]).double()
    assert sc.err(case.run_cut(t, [64, 1, 2, 70]), whole) < 2e-6 and sc.err(case.run_cut(t, [100]), whole) < 2e-6
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sb, u, []), StepEntry(sa, t[:90], range(90))])
    assert sc.err(out, whole[:90]) < 2e-6
    out = eng.step([StepEntry(sa, [t[90]], [0]), StepEntry(sb, [5], [])])
    assert sc.err(out[0], whole[90]) < 2e-6
    eng.release(sa)
    eng.release(sb)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(cases, graphs):
    case = cases("a")
    reqs, wants = sc.greedy(case, n_new=12, prompts=5)
    res = lq.generate(case.eng, reqs, max_new_tokens=12, max_batch=3, stop_ids=[], use_graphs=graphs)
    assert res.tokens == wants
    case.assert_idle()


def test_generation_in_bfloat16_captured_and_direct_steps_agree_and_stop_ids_end_requests(cases):
    case = cases("c", "bfloat16")
    assert case.eng.graph_safe
    reqs = [sc.tokens(n, case.vocab, 40 + n) for n in (3, 70, 9, 1, 130, 20)]
    direct = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[], use_graphs=False)
    stop = direct.tokens[1][7]
    a = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=False)
    b = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=True)
    assert a.tokens == b.tokens and a.finish == b.finish and "stop" in a.finish
    case.assert_idle()


def test_command_line_and_trace_replay(cases, tmp_path):
    case = cases("b")
    reqs, wants = sc.greedy(case, n_new=5, prompts=1)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quarrel"), "-model", case.folder, "-dtype", "float32",
                          "-prompt", " ".join(map(str, reqs[0])), "-n", "5", "-temp", "0", "-penalty", "1"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Architecture: Sofinex" in out.stdout
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in wants[0]]
    a, b = sc.tokens(70, case.vocab, 1), sc.tokens(9, case.vocab, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}, {"id": "b", "tokens": b[:7], "want": [6]}],
              "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [a[66]], "want": [0]}, {"id": "b", "tokens": [b[7]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [a[67]], "want": []}, {"id": "b", "tokens": [b[8]], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:], "want": [1]}], "end": ["a"]}]
    for dtype, check in (("float32", lambda g, w: sc.err(g, w) < TOL_F32), ("bfloat16", lambda g, w: sc.err(g, w) < 0.1)):
        folder = tmp_path / dtype
        folder.mkdir()
        proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", case.folder, "--dtype", dtype,
                                 "--out", str(folder), "--max-tokens", "79"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
                                stderr=subprocess.PIPE, text=True)
        try:
            for st in steps:
                proc.stdin.write(json.dumps(st) + "\n")
                proc.stdin.flush()
                assert proc.stdout.readline().strip() == f"done {st['step']}", proc.stderr.read()[-3000:]
            proc.stdin.close()
            assert proc.wait(timeout=120) == 0
        finally:
            if proc.poll() is None:
                proc.kill()
        read = lambda n: torch.from_numpy(np.fromfile(os.path.join(str(folder), f"{n}.f32"), dtype="<f4").reshape(-1, case.vocab).copy())
        wa, wb = case.want(a), case.want(b)
        assert check(read(0), torch.stack([wa[0], wa[65], wb[6]]))
        assert check(read(1), wa[66:67]) and check(read(2), wb[8:9]) and check(read(3), wa[69:70])
