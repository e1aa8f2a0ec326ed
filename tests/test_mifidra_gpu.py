"""The Mifidra design on the GPU.  First every kernel that the design brought, or widened, alone against the plain
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
import mifidra_cases as mc
import plain_mifidra as pm
from longbow_quarrel_amd.engine import StepEntry
from test_mifidra_cpu import far_attention_rows

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


# ---- kernels alone -------------------------------------------------------------------------------------------------
def plain_delta(q, k, v, beta, g):
    """The recurrence by itself, float64: q, k [T, G, D] (unit vectors, q scaled), v [T, H, P], beta [T, H], g [T, H,
    D]; -> o [T, H * P] and the last state [H, D, P]."""
    T, G, D = q.shape
    H, P = v.shape[1], v.shape[2]
    o = torch.zeros(T, H, P, dtype=F)
    last = torch.zeros(H, D, P, dtype=F)
    for n in range(H):
        j = n // (H // G)
        S = torch.zeros(D, P, dtype=F)
        for t in range(T):
            S = g[t, n][:, None] * S
            S = S + torch.outer(k[t, j], beta[t, n] * (v[t, n] - S.T @ k[t, j]))
            o[t, n] = S.T @ q[t, j]
        last[n] = S
    return o.reshape(T, H * P), last


@pytest.mark.parametrize("sizes", [(2, 2, 16, 8), (4, 2, 12, 20), (3, 1, 17, 9), (2, 1, 64, 64), (1, 1, 130, 70),
                                   (8, 4, 128, 128), (6, 3, 32, 64), (1, 1, 1, 1)])
def test_delta_rule_scan_with_a_decay_for_every_key_channel(kn, sizes):
    """Two sequences in unequal portions, their states in slots that are not in order.  The decays are near one in
    some channels and near zero in others, and differ between the channels of one head, so that a decay applied to
    the wrong axis of the state, a lost state and a wrong slot all show."""
    H, G, D, P = sizes
    lengths, slots = (45, 19), (3, 1)
    dt_bias = rnd(H * D, seed=6, std=3.0)
    a_log = rnd(H, seed=7, std=0.7)
    seqs, wants = [], []
    for i, T in enumerate(lengths):
        q, k, v = rnd(T, G, D, seed=10 + i), rnd(T, G, D, seed=20 + i), rnd(T, H, P, seed=30 + i)
        beta, a = rnd(T, H, seed=40 + i, std=2.0), rnd(T, H * D, seed=50 + i)
        qd, kd = q.double(), k.double()
        qn = qd / torch.sqrt((qd * qd).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        kn_ = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + 1e-6)
        step = torch.nn.functional.softplus(a.double() + dt_bias.double(), threshold=1e9).view(T, H, D)
        g = torch.exp(-torch.exp(a_log.double())[None, :, None] * step)
        if D > 1:
            assert float(g.max()) > 0.9 and float(g.min()) < 0.1
        seqs.append((q, k, v, beta, a))
        wants.append(plain_delta(qn, kn_, v.double(), torch.sigmoid(beta.double()), g))
    state = rnd(5, H, P, D, seed=3).to(DEV)  # what a slot's last sequence left
    state[list(slots)] = 0
    got = [[], []]
    at = [0, 0]
    for cut in ((1, 7), (1, 1), (2, 1), (30, 1), (1, 9), (10, 0)):  # (one token each: the kernel's form for single tokens)
        live = [i for i in (0, 1) if cut[i]]
        parts = [[t[at[i] : at[i] + cut[i]] for t in seqs[i]] for i in live]
        rows = sum(cut[i] for i in live)
        cat = [torch.cat([p[j].reshape(p[j].shape[0], -1) for p in parts]) for j in range(5)]
        o = torch.zeros((rows, H * P), device=DEV)
        cu = [0]
        for i in live:
            cu.append(cu[-1] + cut[i])
        kn.delta_scan(dev(cat[0]), dev(cat[1]), dev(cat[2]), dev(cat[3]), dev(cat[4]), dev(dt_bias), dev(a_log), state, o,
                      H, G, D, P, D ** -0.5, 1e-6, i32([slots[i] for i in live]), i32(cu), len(live), channel_decay=True)
        for j, i in enumerate(live):
            got[i].append(o[cu[j] : cu[j + 1]].cpu())
            at[i] += cut[i]
    for i in (0, 1):
        assert at[i] == lengths[i]
        assert mc.err(torch.cat(got[i]), wants[i][0]) < 5e-6, f"sequence {i}"
        assert mc.err(state[slots[i]].cpu().transpose(1, 2), wants[i][1]) < 5e-6, f"state of sequence {i}"
    # one decay a head still runs as before
    T = 12
    q, k, v, beta, a = rnd(T, G, D, seed=1), rnd(T, G, D, seed=2), rnd(T, H, P, seed=3), rnd(T, H, seed=4), rnd(T, H, seed=5)
    qd, kd = q.double(), k.double()
    qn = qd / torch.sqrt((qd * qd).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kn_ = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + 1e-6)
    g = torch.exp(-torch.exp(a_log.double()) * torch.nn.functional.softplus(a.double() + dt_bias[:H].double(), threshold=1e9))
    want = plain_delta(qn, kn_, v.double(), torch.sigmoid(beta.double()), g[:, :, None].expand(T, H, D))[0]
    state = torch.zeros((1, H, P, D), device=DEV)
    o = torch.zeros((T, H * P), device=DEV)
    kn.delta_scan(dev(q.reshape(T, -1)), dev(k.reshape(T, -1)), dev(v.reshape(T, -1)), dev(beta), dev(a), dev(dt_bias[:H]),
                  dev(a_log), state, o, H, G, D, P, D ** -0.5, 1e-6, i32([0]), i32([0, T]), 1)
    assert mc.err(o, want) < 5e-6


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_short_convolution_carries_its_last_inputs_between_steps(kn, taps):
    """Two sequences in portions of one, two and many tokens, in slots that another sequence has used."""
    C = 70
    lengths, slots = (23, 9), (2, 0)
    w = rnd(C, taps, seed=taps)
    xs = [rnd(n, C, seed=60 + i) for i, n in enumerate(lengths)]
    wants = [pm.short_conv(x.double(), w.double()) for x in xs]
    state = rnd(3, max(1, taps - 1), C, seed=4).to(DEV)
    state[list(slots)] = 0  # (the cache clears a slot when a sequence takes it)
    got, at = [[], []], [0, 0]
    for cut in ((1, 2), (1, 1), (2, 1), (14, 5), (5, 0)):
        live = [i for i in (0, 1) if cut[i]]
        x = torch.cat([xs[i][at[i] : at[i] + cut[i]] for i in live])
        cu, pos, seq = [0], [], []
        for j, i in enumerate(live):
            cu.append(cu[-1] + cut[i])
            pos += list(range(at[i], at[i] + cut[i]))
            seq += [j] * cut[i]
        out = torch.zeros((x.shape[0], C), device=DEV)
        kn.causal_conv(dev(x), dev(w), None, state, out, i32(pos), i32(seq), i32([slots[i] for i in live]),
                       i32([at[i] for i in live]), i32([cut[i] for i in live]), i32(cu), len(live), activation="silu")
        for j, i in enumerate(live):
            got[i].append(out[cu[j] : cu[j + 1]].cpu())
            at[i] += cut[i]
    for i in (0, 1):
        assert mc.err(torch.cat(got[i]), wants[i]) < 2e-6, f"sequence {i}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(6, 2, 24, 16, 16), (1, 1, 10, 7, 6), (8, 2, 64, 32, 64), (3, 3, 8, 24, 8),
                                   (2, 1, 128, 128, 64), (5, 5, 6, 10, 0), (4, 2, 192, 32, 190)])
def test_rotation_of_neighbouring_pairs_and_the_unit_root_mean_square(kn, dtype, sizes):
    """Queries, keys and values of one product: the first `dims` entries of every query and key head turn in pairs
    (2i, 2i + 1), the head is then divided by its root mean square, values pass; positions up to a hundred thousand,
    where a 32-bit angle is only as good as its 32-bit product."""
    H, G, d, vd, dims = sizes
    rows = 11
    pos = [0, 1, 2, 63, 64, 65, 1000, 4095, 4096, 50000, 99999]
    src = rnd(rows, (H + G) * d + G * vd, seed=d)
    rot = {"base": 30000.0, "dims": dims, "scaling": {"factor": 6.0, "original": 1024, "fast": 16.0, "slow": 2.0}}
    q, k = src[:, : H * d].double().view(rows, H, d), src[:, H * d : (H + G) * d].double().view(rows, G, d)
    if dims:
        f, mag = pm.rotary_table(rot)
        ang = torch.tensor(pos, dtype=F)[:, None] * f[None]
        c, s = (torch.cos(ang) * mag)[:, None], (torch.sin(ang) * mag)[:, None]

        def turn(x):
            y = x.clone()
            y[..., 0:dims:2] = x[..., 0:dims:2] * c - x[..., 1:dims:2] * s
            y[..., 1:dims:2] = x[..., 1:dims:2] * c + x[..., 0:dims:2] * s
            return y
        q, k = turn(q), turn(k)
    for eps in (1e-5, None):
        wq, wk = (q, k) if eps is None else (pm.rms_norm(q, eps), pm.rms_norm(k, eps))
        qo = torch.zeros((rows, H * d), dtype=dtype, device=DEV)
        ko = torch.zeros((rows, G * d), dtype=dtype, device=DEV)
        vo = torch.zeros((rows, G * vd), dtype=dtype, device=DEV)
        freqs = torch.tensor(f.tolist(), dtype=F, device=DEV) if dims else None
        kn.rotary_qkv(dev(src), qo, ko, vo, H, G, d, vd, dims, True, freqs, mag if dims else 1.0, eps, i32(pos))
        # an angle of 1e5 held in 32 bits is off by up to 4e-3: the rows far out are held to that, the others sharply
        tol = 8e-3 if dtype == torch.bfloat16 else 1e-6
        far = 8e-3 if dtype == torch.bfloat16 else 6e-3
        for got, want in ((qo, wq.reshape(rows, -1)), (ko, wk.reshape(rows, -1)), (vo, src[:, (H + G) * d :].double())):
            assert mc.err(got[:6], want[:6]) < tol and mc.err(got, want) < far, (eps, sizes)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_of_a_result_in_pieces_added_to_the_stream_with_the_next_norm(kn, dtype):
    for rows, width in ((9, 200), (1, 50), (70, 256), (3, 4100), (8, 4096), (2, 8200)):
        x = rnd(rows, width, seed=1, std=3.0)
        w, nw = rnd(width, seed=2) + 1, rnd(width, seed=3) + 1
        extra = rnd(rows, width, seed=4)
        for n, scales in ((1, (1.0,)), (2, (0.8, 0.9)), (2, (0.0, 1.5)), (3, (1.0, -0.5, 2.0)), (4, (0.25, 1.0, 1.0, 3.0))):
            y = rnd(n, rows, width, seed=5 + n, std=0.02)  # small: eps matters
            total = sum(sc * y[i].double() for i, sc in enumerate(scales))
            want = x.double() + pm.rms_norm(total, 1e-5, w.double())
            xd = dev(x)
            kn.postnorm_residual(xd, dev(y if n > 1 else y[0]), scales, dev(w), 1e-5)
            assert mc.err(xd, want) < 1e-6, (rows, width, n)
            xd = dev(x)
            h = torch.zeros((rows, width), dtype=dtype, device=DEV)
            kn.postnorm_residual(xd, dev(y), scales, dev(w), 1e-5, extra=dev(extra), next_weight=dev(nw), next_eps=1e-3, h=h)
            want = want + extra.double()
            assert mc.err(xd, want) < 1e-6
            assert mc.err(h, pm.rms_norm(want, 1e-3, nw.double())) < (1e-6 if dtype == torch.float32 else 5e-3)


def test_norm_a_head_with_a_sigmoid_gate_biases_of_a_gated_unit_and_scaling(kn):
    rows = 9
    y, z = rnd(rows, 120, seed=7, std=0.01), rnd(rows, 120, seed=8, std=2.0)
    for group, wlen in ((40, 40), (24, 24), (120, 120), (8, 8)):
        wt = rnd(wlen, seed=9)
        out = torch.zeros((rows, 120), device=DEV)
        kn.gated_rmsnorm(dev(y), dev(z), dev(wt), 1e-5, group, out, gate_first=False, gate="sigmoid")
        v = pm.rms_norm(y.double().view(rows, 120 // group, group), 1e-5).reshape(rows, 120)
        want = v * wt.double().repeat(120 // wlen) * torch.sigmoid(z.double())
        assert mc.err(out, want) < 1e-6, group
    # gated unit: biases on gate and up; the tail columns carry a one for the next product's bias
    gu, b = rnd(rows, 2 * 70, seed=6, std=2.0), rnd(2 * 70, seed=5)
    want = pm.silu(gu[:, :70].double() + b[:70].double()) * (gu[:, 70:].double() + b[70:].double())
    out = torch.zeros((rows, 70), device=DEV)
    kn.glu(dev(gu), out, "silu", bias=dev(b))
    assert mc.err(out, want) < 1e-6
    out = torch.full((rows, 78), 7.0, device=DEV)
    kn.glu(dev(gu), out, "silu", bias=dev(b), tail=8)
    assert mc.err(out[:, :70], want) < 1e-6 and bool((out[:, 70] == 1).all()) and bool((out[:, 71:] == 0).all())
    x = rnd(5, 333, seed=2)
    xd = dev(x)
    kn.scale(xd, 0.37)
    assert mc.err(xd, x.double() * 0.37) < 1e-7


def test_router_with_a_correction_within_the_best_groups(kn):
    """Against the plain router, row by row: choice by score plus correction (corrections large enough to turn the
    order over, and negative enough that a choice score below zero is common), weights without it; the groups'
    marks are the sums of their two best choice scores, and an expert outside the kept groups is never chosen
    however large its score."""
    rows = 200
    for E, top, groups, keep in ((16, 5, 4, 3), (6, 2, 3, 2), (12, 3, 4, 2), (8, 8, 2, 2), (4, 2, 4, 2), (9, 3, 3, 1),
                                 (7, 3, 0, 0), (64, 6, 8, 3)):
        z = rnd(rows, E, seed=E + top, std=2.0)
        corr = rnd(E, seed=E, std=0.6) - 0.7
        if groups:
            z[5, :] = -3.0
            z[5, 0] = 9.0  # one large score alone in its group: the group's mark has a poor second
        route = torch.zeros(rows, E, device=DEV)
        kn.moe_route(dev(z), route, top, False, correction=dev(corr), groups=groups, keep=keep)
        r = {"experts": E, "top": top}
        if groups:
            r["groups"] = {"count": groups, "keep": keep}
        s, chosen = pm.route(z.double(), r, {"m.router": torch.eye(E, dtype=F), "m.correction": corr.double()}, "m")
        got = route.cpu()
        close = 0
        for t in range(rows):
            mine = [e for e in range(E) if got[t, e] >= 0]
            if mine != sorted(chosen[t]):
                # only a call closer than 32-bit rounding may fall the other way
                c = (s[t] + corr.double()).tolist()
                diff = set(mine) ^ set(chosen[t])
                assert len(mine) == top and max(c[e] for e in diff) - min(c[e] for e in diff) < 1e-6, (E, t)
                close += 1
                continue
            for e in mine:
                assert float(got[t, e]) == pytest.approx(float(s[t, e]), rel=2e-6, abs=1e-9)
        assert close <= 1
        assert bool(((got >= 0).sum(-1) == top).all())
    # experts: silu(gate) up, the weight on the result
    E, ff = 6, 12
    z = rnd(rows, E, seed=3)
    route = torch.zeros(rows, E, device=DEV)
    kn.moe_route(dev(z), route, 2, False, correction=dev(rnd(E, seed=1)), groups=3, keep=2)
    gu = rnd(rows, E * 2 * ff, seed=2, std=2.0)
    out = torch.zeros(rows, E * ff, device=DEV)
    kn.moe_glu(dev(gu), route, out, E, ff, 0.0, False, activation="silu")
    v = gu.double().reshape(rows, E, 2, ff)
    wt = route.cpu().double()[:, :, None]
    want = torch.where(wt >= 0, pm.silu(v[:, :, 0]) * v[:, :, 1] * wt, torch.zeros_like(v[:, :, 0])).reshape(rows, E * ff)
    assert mc.err(out, want) < 1e-6


# ---- the engine ------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, dtype="float32", **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in made:
            made[key] = mc.Case(tmp_path_factory.mktemp("mifidra"), name, load, dtype=dtype,
                                rounding=dtype == "bfloat16", **kw)
        return made[key]

    return get


@pytest.mark.parametrize("name", ["attention", "delta", "dense", "moe", "loop"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    mc.whole_and_token_by_token(case, TOL_F32, lengths=(1, 2, 9, 70))
    mc.portions(case, TOL_F32, n=140)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_under_every_cutting_and_batching(cases, name):
    """(In "b" the two mixers' outputs nearly cancel at a few rows ahead of the norm of their sum, which multiplies
    32-bit rounding about ten-fold there, in the torch stand-in on the CPU just as here: rows around 1e-6, those
    rows 1e-5 to 3e-5.  A fault of the cache or the batch is orders of magnitude above either.)"""
    case = cases(name)
    tol = 6e-5 if name == "b" else TOL_F32
    mc.whole_and_token_by_token(case, tol)
    mc.portions(case, tol)
    mc.unequal_batches(case, tol)
    mc.slots_and_blocks_used_again(case, tol)


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("c", "float32"), ("c", "bfloat16")])
def test_prompt_rows_sorted_by_expert(cases, name, dtype, monkeypatch):
    """The same logits whether a prompt's rows run through all experts' columns or are sorted by expert."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    case = cases(name, dtype)
    t = mc.tokens(300, case.vocab, 12)
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 10 ** 9)
    every = case.run_cut(t, [300])
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    by_expert = case.run_cut(t, [200, 3, 90])
    if dtype == "float32":
        assert mc.err(by_expert, case.want(t)) < TOL_F32 and mc.err(by_expert, every) < TOL_F32
    else:
        mc.assert_close_bf16(by_expert, case.want(t), case.noise(t))


@pytest.mark.parametrize("seed", range(1, 13))
def test_configurations_drawn_from_a_seed(cases, seed):
    """Other sizes, head counts, ranks, taps, layer orders, loops, experts, groups and constants, in both dtypes."""
    case = cases(seed)
    t, u = mc.tokens(200, case.vocab, seed), mc.tokens(9, case.vocab, seed + 50)
    assert mc.err(case.run_cut(t, [150, 2, 1, 20]), case.want(t)) < TOL_F32
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:130], range(130))])
    assert mc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:130]])) < TOL_F32
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[130:131], [0])])
    assert mc.err(out, torch.stack([case.want(u)[8], case.want(t)[130]])) < TOL_F32
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()
    case16 = cases(seed, "bfloat16")
    mc.assert_close_bf16(case16.run_cut(t, [150, 2]), case16.want(t), case16.noise(t))


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(mc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 8
    for i, (g, w) in enumerate(zip(got, want)):
        assert mc.err(g, w) < TOL_F32, f"after layer run {i}"


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_bfloat16_whole_in_portions_and_in_batches(cases, name):
    case = cases(name, "bfloat16")
    t = mc.tokens(150, case.vocab, 3)
    want, noise = case.want(t), case.noise(t)
    mc.assert_close_bf16(case.run_cut(t, [150]), want, noise)
    mc.assert_close_bf16(case.run_cut(t, [64, 1, 63, 2, 3]), want, noise)
    u = mc.tokens(70, case.vocab, 4)
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, t[:100], range(100)), StepEntry(sb, u[:3], range(3))])
    mc.assert_close_bf16(out, torch.cat([want[:100], case.want(u)[:3]]), noise)
    got = []
    for i in range(20):
        got.append(eng.step([StepEntry(sb, [u[3 + i]], [0]), StepEntry(sa, [t[100 + i]], [0])]).clone())
    got = torch.cat(got)
    mc.assert_close_bf16(torch.cat([got[0::2], got[1::2]]), torch.cat([case.want(u)[3:23], want[100:120]]), noise)
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_bfloat16_decoding_over_long_contexts(cases):
    """Single tokens over several hundred cached rows against the same rows as parts of a prompt and against the
    plain implementation."""
    case = cases("c", "bfloat16")
    t, u = mc.tokens(640, case.vocab, 61), mc.tokens(330, case.vocab, 62)
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
    mc.assert_close_bf16(got, want, noise)
    mc.assert_close_bf16(got, whole.double(), noise)


def test_bfloat16_probabilities_on_the_causal_matrix_core_kernel(tmp_path_factory, monkeypatch):
    """The design keeps the softmax's weights 32-bit, so its attention runs on the general kernel.  A design that
    lets them be rounded to bfloat16 for their product with the values (the attention part's `probabilities`) runs
    heads whose keys and values are of one size, in bfloat16, through the causal kernel that the Llama shape uses:
    the same up to that rounding, in prompts, portions and single tokens over several hundred cached rows."""
    from longbow_quarrel_amd.parts.sink_attention import SinkWindowAttention
    case = mc.Case(tmp_path_factory.mktemp("mifidra_d"), "d", load, dtype="bfloat16", rounding=True)
    calls = []
    real = case.eng.kernels.attention
    monkeypatch.setattr(case.eng.kernels, "attention", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    t = mc.tokens(400, case.vocab, 71)
    want, noise = case.want(t), case.noise(t)
    general = case.run_cut(t, [300, 2, 64])
    assert not calls
    mc.assert_close_bf16(general, want, noise)
    parts = [s for m in case.eng.model._mixers() for s in m.sides if isinstance(s, SinkWindowAttention)]
    assert len(parts) == 3 and all(p.probabilities == "float32" for p in parts)
    for p in parts:
        p.probabilities = "bfloat16"
    fast = case.run_cut(t, [300, 2, 64])
    assert len(calls) == 5 * 37  # five layer runs, a prompt, two portions and 34 single tokens
    mc.assert_close_bf16(fast, want, noise)
    mc.assert_close_bf16(fast, general.double(), noise)
    reqs = [mc.tokens(n, case.vocab, 40 + n) for n in (3, 70, 9)]
    a = lq.generate(case.eng, reqs, max_new_tokens=20, stop_ids=[], use_graphs=False)
    b = lq.generate(case.eng, reqs, max_new_tokens=20, stop_ids=[], use_graphs=True)
    assert a.tokens == b.tokens
    # a float32 run takes the general kernel whatever the part allows
    case = mc.Case(tmp_path_factory.mktemp("mifidra_d32"), "d", load)
    for m in case.eng.model._mixers():
        m.sides[0].probabilities = "bfloat16"
    calls.clear()
    monkeypatch.setattr(case.eng.kernels, "attention", lambda *a, **k: calls.append(1))
    assert mc.err(case.run_cut(t[:200], [150, 2]), case.want(t[:200])) < TOL_F32 and not calls


def test_a_far_key_carries_the_result(cases):
    case = cases("attention", sharp=5.0)
    t = mc.tokens(330, case.vocab, 21)
    want = case.want(t)
    assert far_attention_rows(case, t)
    assert mc.err(case.run_cut(t, [330]), want) < TOL_F32
    assert mc.err(case.run_cut(t, [127, 1, 64, 2, 100]), want) < TOL_F32
    case = cases("c", sharp=4.0)
    t = mc.tokens(300, case.vocab, 22)
    assert mc.err(case.run_cut(t, [250]), case.want(t)) < 1e-4


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    case = cases("delta", memory=7.0)
    t = mc.tokens(260, case.vocab, 31)
    want = case.want(t)
    assert mc.err(case.run_cut(t, [260]), want) < TOL_F32
    assert mc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL_F32
    t = mc.tokens(640, case.vocab, 32)
    want = case.want(t)
    assert mc.err(case.run_cut(t, [600]), want) < TOL_F32
    assert mc.err(case.run_cut(t, [20, 580, 2]), want) < TOL_F32


def test_the_first_tokens_see_zeros_ahead_of_the_sequence(cases):
    case = cases("delta")
    eng = case.eng
    a, b = mc.tokens(30, case.vocab, 1), mc.tokens(6, case.vocab, 2)
    sa = eng.new_sequence()
    eng.step([StepEntry(sa, a, [])])
    eng.release(sa)
    for first in (1, 2, 3, 6):
        s = eng.new_sequence()
        assert s == sa
        out = eng.step([StepEntry(s, b[:first], range(first))])
        assert mc.err(out, case.want(b)[:first]) < TOL_F32
        if first < 6:
            out = eng.step([StepEntry(s, b[first:], range(6 - first))])
            assert mc.err(out, case.want(b)[first:]) < TOL_F32
        eng.release(s)
    case.assert_idle()


@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(cases, name):
    mc.long_decoding(cases(name), TOL_F32)


def test_float32_logits_do_not_depend_on_the_cutting_or_the_batch_by_more_than_rounding(cases):
    case = cases("a")
    t, u = mc.tokens(140, case.vocab, 7), mc.tokens(30, case.vocab, 8)
    whole = case.run_cut(t, [140]).double()
    assert mc.err(case.run_cut(t, [64, 1, 2, 70]), whole) < 2e-6 and mc.err(case.run_cut(t, [100]), whole) < 2e-6
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sb, u, []), StepEntry(sa, t[:90], range(90))])
    assert mc.err(out, whole[:90]) < 2e-6
    out = eng.step([StepEntry(sa, [t[90]], [0]), StepEntry(sb, [5], [])])
    assert mc.err(out[0], whole[90]) < 2e-6
    eng.release(sa)
    eng.release(sb)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(cases, graphs):
    case = cases("a")
    reqs, wants = mc.greedy(case, n_new=12, prompts=5)
    res = lq.generate(case.eng, reqs, max_new_tokens=12, max_batch=3, stop_ids=[], use_graphs=graphs)
    assert res.tokens == wants
    case.assert_idle()


def test_generation_in_bfloat16_captured_and_direct_steps_agree_and_stop_ids_end_requests(cases):
    case = cases("c", "bfloat16")
    assert case.eng.graph_safe
    reqs = [mc.tokens(n, case.vocab, 40 + n) for n in (3, 70, 9, 1, 130, 20)]
    direct = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[], use_graphs=False)
    stop = direct.tokens[1][7]
    a = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=False)
    b = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=True)
    assert a.tokens == b.tokens and a.finish == b.finish and "stop" in a.finish
    case.assert_idle()


def test_command_line_and_trace_replay(cases, tmp_path):
    case = cases("b")
    reqs, wants = mc.greedy(case, n_new=5, prompts=1)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quarrel"), "-model", case.folder, "-dtype", "float32",
                          "-prompt", " ".join(map(str, reqs[0])), "-n", "5", "-temp", "0", "-penalty", "1"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Architecture: Mifidra" in out.stdout
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in wants[0]]
    a, b = mc.tokens(70, case.vocab, 1), mc.tokens(9, case.vocab, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}, {"id": "b", "tokens": b[:7], "want": [6]}],
              "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [a[66]], "want": [0]}, {"id": "b", "tokens": [b[7]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [a[67]], "want": []}, {"id": "b", "tokens": [b[8]], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:], "want": [1]}], "end": ["a"]}]
    for dtype, check in (("float32", lambda g, w: mc.err(g, w) < TOL_F32), ("bfloat16", lambda g, w: mc.err(g, w) < 0.1)):
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
