"""The Mifidra design through the engine's own code (registry, loader, cache groups, step function, generation
loop) on the CPU, over the torch stand-in for the kernels, against the plain implementation.  The GPU tests
repeat every scenario with the HIP kernels; these catch faults of the parts, the cache and the batching."""
import copy
import math

import pytest
import torch

import longbow_quarrel_amd as lq
import mifidra_cases as mc
import plain_mifidra as pm
from cpu_kernels import CpuKernels
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.parts.base import KVNeed, StateNeed

TOL = 2e-5
F = torch.float64


def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=CpuKernels(),
                          max_slots=8, max_sequence_tokens=max_tokens)


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, **kw):
        key = (name, tuple(sorted(kw.items())))
        if key not in made:
            made[key] = mc.Case(tmp_path_factory.mktemp("mifidra"), name, load, **kw)
        return made[key]

    return get


# ---- configuration, registry, tensors, cache needs ----------------------------------------------------------------
def test_configuration_reads_every_size_and_writes_the_same_keys_back():
    for cfg in mc.CONFIGS.values():
        assert lq.MifidraConfig.from_dict(cfg).to_dict() == cfg
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import config_from_dict, spec_from_config

    config = config_from_dict(mc.CFG_A)
    assert isinstance(config, lq.MifidraConfig)
    model = DecoderModel(spec_from_config(config))
    # layers 1 and 2 run three times in a row; every pass after the first takes the embedding's output in again
    assert [(r.layer, r.add_input) for r in model.spec.schedule] == [
        (0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    names = {s.name for s in model.tensor_specs()}
    assert {"embed", "l0.norm1b", "l0.norm2b", "l0.mix.left.q", "l0.mix.right.q.conv", "l0.mix.right.A_log",
            "l0.mix.right.dt_bias", "l0.mix.right.a2", "l0.mix.right.g1", "l0.mix.right.norm", "l0.mlp.gate.b",
            "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e5.down", "l1.mlp.shared.up", "l3.mlp.e3.gate",
            "final.norm"} <= names
    assert not any(n.startswith("l2.mlp") for n in names) and "l3.mlp.shared.up" not in names
    assert [s.optional for s in model.tensor_specs() if s.name == "l2.norm2b"] == [True]
    assert "head" not in names  # the head is the embedding
    shapes = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert shapes["l0.mix.left.q"] == (6 * 24, 80) and shapes["l0.mix.left.k"] == (2 * 24, 80)
    assert shapes["l0.mix.left.v"] == (2 * 16, 80) and shapes["l0.mix.left.o"] == (80, 6 * 16)
    assert shapes["l0.mix.right.q"] == (2 * 12, 80) and shapes["l0.mix.right.v"] == (4 * 20, 80)
    assert shapes["l0.mix.right.v.conv"] == (80, 4) and shapes["l0.mix.right.b"] == (4, 80)
    assert shapes["l0.mix.right.A_log"] == (4,) and shapes["l0.mix.right.dt_bias"] == (4 * 12,)
    assert shapes["l0.mix.right.a1"] == (6, 80) and shapes["l0.mix.right.a2"] == (48, 6)
    assert shapes["l0.mix.right.g1"] == (10, 80) and shapes["l0.mix.right.g2"] == (80, 10)
    assert shapes["l0.mix.right.norm"] == (20,) and shapes["l1.mlp.correction"] == (6,)
    # every run of a layer has a cache of its own: keys and values of the attention, and the delta rule's state with
    # the convolutions' last inputs
    needs = model.cache_needs()
    assert len(needs) == 8
    from longbow_quarrel_amd.parts.base import MultiNeed
    assert needs[0] == MultiNeed((KVNeed(2, 24, 0, 16), MultiNeed((StateNeed((4, 20, 12), torch.float32),
                                                                    StateNeed((3, 2 * 2 * 12 + 4 * 20), torch.float32)))))
    assert needs[1] == needs[3] == needs[5] and needs[2] == needs[4] == needs[6]
    assert needs[2].needs[0] == KVNeed(1, 32, 0, 32) and needs[7].needs[0] == KVNeed(3, 8, 0, 24)


@pytest.mark.parametrize("key,value,text", [
    (("layers", 0, "type"), "attention", "layers[0].type"),
    (("layers", 0, "mixer", "left", "kv_heads"), 4, "kv_heads"),
    (("layers", 0, "mixer", "left", "scale"), None, "left.scale"),
    (("layers", 0, "mixer", "left", "rot", "dims"), 7, "rot.dims"),
    (("layers", 0, "mixer", "left", "rot", "dims"), 26, "rot.dims"),
    (("layers", 0, "mixer", "left", "rot", "scaling", "factor"), None, "rot.scaling.factor"),
    (("layers", 0, "mixer", "right", "conv"), 0, "right.conv"),
    (("layers", 0, "mixer", "right", "kv_heads"), 3, "kv_heads"),
    (("layers", 0, "mixer", "right_scale"), None, "right_scale"),
    (("layers", 0, "mlp", "kind"), "glu", "mlp.kind"),
    (("layers", 1, "mlp", "router", "top"), 7, "router.top"),
    (("layers", 1, "mlp", "router", "groups", "count"), 4, "groups"),
    (("layers", 1, "mlp", "router", "groups", "keep"), 4, "groups"),
    (("layers", 1, "mlp", "expert", "ff"), None, "expert.ff"),
    (("loop", "stop"), 5, "loop"),
    (("loop", "times"), 0, "loop.times"),
    (("norm", "eps"), "tiny", "norm.eps"),
    (("width",), None, "width"),
])
def test_configuration_errors_name_their_key(key, value, text):
    cfg = copy.deepcopy(mc.CFG_A)
    d = cfg
    for k in key[:-1]:
        d = d[k]
    d[key[-1]] = value
    with pytest.raises(lq.ConfigError) as e:
        lq.MifidraConfig.from_dict(cfg)
    assert text in str(e.value)


def test_groups_too_small_for_the_experts_asked_of_them_are_refused():
    cfg = copy.deepcopy(mc.CFG_MOE)  # 12 experts in 4 groups, 2 kept: at most 6 can be chosen
    cfg["layers"][0]["mlp"]["router"]["top"] = 7
    with pytest.raises(lq.ConfigError) as e:
        lq.MifidraConfig.from_dict(cfg)
    assert "groups" in str(e.value)


def test_keys_that_a_configuration_leaves_out():
    cfg = copy.deepcopy(mc.CFG_DELTA)
    left, right = cfg["layers"][0]["mixer"]["left"], cfg["layers"][0]["mixer"]["right"]
    del left["kv_heads"], left["vdim"], right["kv_heads"], right["vdim"], cfg["logit_scale"]
    got = lq.MifidraConfig.from_dict(cfg)
    assert got.layers[0].left.kv_heads == 1 and got.layers[0].left.vdim == 8 and got.layers[0].left.rot is None
    assert got.layers[0].right.kv_heads == 4 and got.layers[0].right.vdim == 12
    assert got.logit_scale == 1.0 and got.loop is None and got.run_order() == [(0, False)]


def test_sizes_that_no_key_gives_come_from_the_file(tmp_path):
    """The ranks of the decay's and the gate's bottlenecks are the shapes of their first matrices, layer by layer;
    without a file they must be stated."""
    cfg = copy.deepcopy(mc.CFG_A)
    weights = mc.make_weights(cfg, 5)
    for layer in cfg["layers"]:
        del layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"]
    folder = mc.write_folder(tmp_path, cfg, weights, "norank")
    eng = load(folder, "float32", 256)
    assert [(x.right.decay_rank, x.right.gate_rank) for x in eng.config.layers] == [(6, 10), (3, 5), (8, 8), (4, 2)]
    t = mc.tokens(20, cfg["vocab"], 1)
    got = eng.step([StepEntry(eng.new_sequence(), t, range(20))])
    assert mc.err(got, pm.forward(cfg, weights, t)) < TOL
    with pytest.raises(lq.ConfigError) as e:
        lq.random_engine(lq.MifidraConfig.from_dict(cfg), 1, device="cpu", kernels=CpuKernels())
    assert "rank" in str(e.value)


def test_the_norms_of_an_absent_feed_forward_may_be_in_the_file(tmp_path):
    cfg = copy.deepcopy(mc.CFG_DELTA)
    weights = mc.make_weights(cfg, 5)
    weights.pop("l0.norm2", None)
    weights.pop("l0.norm2b", None)
    t = mc.tokens(12, cfg["vocab"], 1)
    got = []
    extra = {"l0.norm2": torch.full((cfg["width"],), 3.0), "l0.norm2b": torch.full((cfg["width"],), -2.0)}
    for name, more in (("without", {}), ("with", extra)):
        eng = load(mc.write_folder(tmp_path, cfg, {**weights, **more}, name), "float32", 256)
        got.append(eng.step([StepEntry(eng.new_sequence(), t, range(12))]))
    assert torch.equal(got[0], got[1]) and mc.err(got[0], pm.forward(cfg, weights, t)) < TOL


def test_missing_and_unexpected_tensors_are_named(tmp_path):
    cfg = copy.deepcopy(mc.CFG_MOE)
    weights = mc.make_weights(cfg, 5)
    weights["l0.mlp.e12.up"] = weights["l0.mlp.e0.up"].clone()
    del weights["l0.mlp.correction"], weights["l0.mix.right.k.conv"]
    folder = mc.write_folder(tmp_path, cfg, weights, "bad")
    with pytest.raises(lq.WeightError) as e:
        load(folder, "float32", 256)
    assert e.value.missing == ["l0.mix.right.k.conv", "l0.mlp.correction"] and e.value.unexpected == ["l0.mlp.e12.up"]


# ---- the plain implementation's own mechanisms against hand-made cases ---------------------------------------------
def test_plain_rotation_pairs_neighbours_and_passes_the_rest():
    rot = {"base": 100.0, "dims": 4}
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]] * 4, dtype=F)
    y = pm.rotate(x, rot)
    f = [1.0, 100.0 ** -0.5]
    c0, s0, c1, s1 = math.cos(3 * f[0]), math.sin(3 * f[0]), math.cos(3 * f[1]), math.sin(3 * f[1])
    assert torch.equal(y[0], x[0])  # position 0
    assert torch.allclose(y[3, 0], torch.tensor([1 * c0 - 2 * s0, 2 * c0 + 1 * s0, 3 * c1 - 4 * s1, 4 * c1 + 3 * s1,
                                                 5.0, 6.0], dtype=F))


def test_plain_yarn_frequencies_and_the_librarys():
    """Pairs that turn often within the original length keep their frequency, slow ones are divided by the factor,
    those between are blended along a ramp over the pair's index; cos and sin grow by 0.1 ln(factor) + 1."""
    from longbow_quarrel_amd.parts.rope import rotary_frequencies, rotary_magnitude

    for dims, base, sc in ((32, 10000.0, {"factor": 4.0, "original": 2000, "fast": 32.0, "slow": 1.0}),
                           (16, 3000.0, {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 1.5}),
                           (8, 100.0, {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
                           (64, 500000.0, {"factor": 16.0, "original": 4096, "fast": 64.0, "slow": 2.0}),
                           (12, 50.0, {"factor": 3.0, "original": 7, "fast": 1.0, "slow": 1.0})):  # (an empty ramp)
        f, mag = pm.rotary_table({"base": base, "dims": dims, "scaling": sc})
        plain = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
        assert mag == 0.1 * math.log(sc["factor"]) + 1
        assert bool(((f <= plain * (1 + 1e-12)) & (f >= plain / sc["factor"] * (1 - 1e-12))).all())
        lib = rotary_frequencies(dims, base, {"rope_type": "yarn", **sc})
        assert torch.allclose(torch.tensor(lib, dtype=F), f, rtol=1e-12, atol=0)
        assert rotary_magnitude({"rope_type": "yarn", **sc}) == mag
    f, _ = pm.rotary_table({"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 2000, "fast": 32.0,
                                                                      "slow": 1.0}})
    assert float(f[0]) == 1.0 and float(f[15]) == pytest.approx(10000.0 ** (-30 / 32) / 4, rel=1e-12)
    # lo = floor(32 ln(2000 / (64 pi)) / (2 ln 10000)) = 3, hi = ceil(32 ln(2000 / (2 pi)) / (2 ln 10000)) = 11
    assert float(f[3]) == 10000.0 ** (-6 / 32) and float(f[11]) == pytest.approx(10000.0 ** (-22 / 32) / 4, rel=1e-12)
    assert float(f[7]) == pytest.approx(10000.0 ** (-14 / 32) * (0.5 / 4 + 0.5), rel=1e-12)


def test_plain_short_convolution_ends_on_the_current_token():
    x = torch.tensor([[1.0], [2.0], [4.0], [8.0]], dtype=F)
    y = pm.short_conv(x, torch.tensor([[100.0, 10.0, 1.0]], dtype=F))
    z = torch.tensor([1.0, 12.0, 124.0, 248.0], dtype=F)
    assert torch.allclose(y[:, 0], z / (1 + torch.exp(-z)))


def _delta_weights(width, m, **given):
    """Weights of one delta-rule mixer that does nothing until `given` says otherwise: convolutions that pass the
    current token, zero projections."""
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    w = {"q": torch.zeros(G * d, width), "k": torch.zeros(G * d, width), "v": torch.zeros(H * vd, width),
         "b": torch.zeros(H, width), "A_log": torch.zeros(H), "a1": torch.zeros(1, width), "a2": torch.zeros(H * d, 1),
         "dt_bias": torch.zeros(H * d), "g1": torch.zeros(1, width), "g2": torch.zeros(H * vd, 1),
         "norm": torch.ones(vd), "o": torch.eye(H * vd)}
    for n, c in (("q", G * d), ("k", G * d), ("v", H * vd)):
        w[n + ".conv"] = torch.zeros(c, m["conv"])
        w[n + ".conv"][:, -1] = 1.0
    w.update({k: torch.tensor(v) for k, v in given.items()})
    return {"x." + k: v.to(F) for k, v in w.items()}


def test_plain_delta_rule_forgets_each_key_channel_at_its_own_rate():
    """Two key channels and two value channels.  The first token writes value channel 0 under the key along
    channel 0, the second writes value channel 1 under the key along channel 1 (the keys are orthogonal, so neither
    write corrects the other), later tokens have no key and write nothing.  The query reads both channels alike, so
    the two outputs at token t are in the ratio g_0^t / g_1^(t - 1), which the norm over the value channels keeps."""
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "conv": 1}
    big = 40.0  # silu(big) = big, silu(0) = 0; beta = sigmoid(big) = 1
    # the input's columns: key channel 0, key channel 1, value channel 0, value channel 1, one
    w = _delta_weights(5, m, q=[[0, 0, 0, 0, big], [0, 0, 0, 0, big]], k=[[big, 0, 0, 0, 0], [0, big, 0, 0, 0]],
                       v=[[0, 0, big, 0, 0], [0, 0, 0, big, 0]], b=[[0, 0, 0, 0, big]], dt_bias=[0.3, -1.2],
                       A_log=[0.4])
    h = torch.tensor([[1.0, 0, 1, 0, 1], [0, 1.0, 0, 1, 1]] + [[0, 0, 0, 0, 1.0]] * 4, dtype=F)
    y = pm.delta_rule(h, m, w, "x", 0.0, False)
    g = [math.exp(-math.exp(0.4) * math.log1p(math.exp(b))) for b in (0.3, -1.2)]
    assert 0.2 < g[0] < 0.3 and 0.6 < g[1] < 0.8
    for t in range(1, 6):
        assert float(y[t, 0] / y[t, 1]) == pytest.approx(g[0] ** t / g[1] ** (t - 1), rel=1e-6)
    # the gate's bottleneck is zero, so the gate is one half, and the norm makes the mean square one
    assert float((y[3] * y[3]).mean()) == pytest.approx(0.25, rel=1e-9)


def test_plain_delta_rule_overwrites_what_a_key_held():
    """A key written twice with step size one holds the second value only; with step size 1/2 (a zero logit), the
    mean of both: the rule corrects what the state gives for the key towards the new value."""
    m = {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 2, "conv": 1}
    big = 40.0
    for logit, mix in ((big, 1.0), (0.0, 0.5)):
        w = _delta_weights(3, m, q=[[big, 0, 0]], k=[[big, 0, 0]], v=[[0, big, 0], [0, 0, big]],
                           b=[[logit, 0, 0]], dt_bias=[-60.0])  # (a decay of one)
        h = torch.tensor([[1.0, 1.0, 0.25], [1.0, 0.25, 1.0]], dtype=F)
        y = pm.delta_rule(h, m, w, "x", 0.0, False)
        v0, v1 = (torch.tensor(x, dtype=F) * big / (1 + torch.exp(torch.tensor(x, dtype=F) * -big))
                  for x in ([1.0, 0.25], [0.25, 1.0]))
        s1 = mix * v0
        s2 = s1 + mix * (v1 - s1)
        assert float(y[1, 0] / y[1, 1]) == pytest.approx(float(s2[0] / s2[1]), rel=1e-5)


def test_plain_router_keeps_the_best_groups_and_weights_without_the_correction():
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}
    z = [2.0, -3.0, 0.5, 0.4, -1.0, 1.5]  # groups (0, 1), (2, 3), (4, 5)
    w = {"m.router": torch.tensor([[v] for v in z], dtype=F),
         "m.correction": torch.tensor([-2.0, 0.0, 0.0, 0.0, 0.1, -0.3], dtype=F)}
    s, chosen = pm.route(torch.ones(1, 1, dtype=F), r, w, "m")
    sig = [1 / (1 + math.exp(-v)) for v in z]
    assert torch.allclose(s[0], torch.tensor(sig, dtype=F))
    # choice scores: -1.12, 0.05, 0.62, 0.60, 0.37, 0.52; groups' marks -1.07, 1.22, 0.89: groups 1 and 2 stay, and
    # expert 0, whose plain score is the largest of all, cannot be chosen
    assert chosen == [[2, 3]]
    r["groups"]["keep"] = 3
    assert pm.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[2, 3]]
    w["m.correction"] = torch.tensor([-2.0, 0.0, 0.0, -0.5, 0.1, -0.3], dtype=F)
    assert pm.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[2, 5]]
    # all corrections negative and large: the best of the kept groups are still chosen, not the masked ones
    w["m.correction"] = torch.tensor([-9.0, -9.5, -7.0, -7.5, -8.0, -8.5], dtype=F)
    r["groups"]["keep"] = 1
    assert pm.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[2, 3]]
    mlp = {"router": r, "expert": {"ff": 1}}
    for e in range(6):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"] = torch.tensor([[1.0]], dtype=F), torch.tensor([[1.0]], dtype=F)
        w[f"m.e{e}.down"] = torch.tensor([[10.0 ** e]], dtype=F)
    a = 1 / (1 + math.exp(-1.0))
    assert float(pm.experts(torch.ones(1, 1, dtype=F), mlp, w, "m", False)) == pytest.approx(
        a * (sig[2] * 100 + sig[3] * 1000))


# ---- every mechanism alone, and all of them, through the engine ------------------------------------------------------
@pytest.mark.parametrize("name", ["attention", "delta", "dense", "moe", "loop"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    mc.whole_and_token_by_token(case, TOL, lengths=(1, 2, 9, 70))
    mc.portions(case, TOL, n=140)


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_against_token_by_token_decoding(cases, name):
    mc.whole_and_token_by_token(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_portions_of_several_sizes_down_to_two_tokens(cases, name):
    mc.portions(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_batches_of_unequal_requests_against_each_alone(cases, name):
    mc.unequal_batches(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "loop"])
def test_slots_and_blocks_are_freed_and_used_again(cases, name):
    mc.slots_and_blocks_used_again(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "moe"])
def test_prompt_rows_sorted_by_expert(cases, name, monkeypatch):
    """A prompt step of many rows sorts them by expert and runs every expert over its own rows: the same logits."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    case = cases(name)
    t = mc.tokens(90, case.vocab, 12)
    assert mc.err(case.run_cut(t, [50, 3, 30]), case.want(t)) < TOL


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_configurations_drawn_from_a_seed(cases, seed):
    case = cases(seed)
    assert lq.MifidraConfig.from_dict(case.cfg).to_dict() == case.cfg
    t, u = mc.tokens(70, case.vocab, seed), mc.tokens(9, case.vocab, seed + 50)
    assert mc.err(case.run_cut(t, [40, 2, 1, 20]), case.want(t)) < TOL
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:66], range(66))])
    assert mc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:66]])) < TOL
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[66:67], [0])])
    assert mc.err(out, torch.stack([case.want(u)[8], case.want(t)[66]])) < TOL
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(mc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 8
    for i, (g, w) in enumerate(zip(got, want)):
        assert mc.err(g, w) < TOL, f"after layer run {i}"


def test_every_pass_of_a_loop_has_a_cache_of_its_own(cases):
    """Were two passes to share keys or a state, the second pass would read what the first wrote for the same
    positions; and the input fed in again shows when left out: both against the plain implementation, in decoding
    after a prompt, and the plain implementation without the loop differs by much."""
    case = cases("loop")
    t = mc.tokens(50, case.vocab, 4)
    assert mc.err(case.run_cut(t, [30, 5]), case.want(t)) < TOL
    once = copy.deepcopy(case.cfg)
    once["loop"]["times"] = 1
    assert mc.err(pm.forward(once, case.weights, t), case.want(t)) > 1e-2


def far_attention_rows(case, t, back=100):
    """Whether, in the attention of the case's first layer, some late row puts most of its weight on one key at
    least `back` positions before it."""
    w = {k: v.double() for k, v in case.weights.items()}
    m = case.cfg["layers"][0]["mixer"]["left"]
    eps = case.cfg["norm"]["eps"]
    n = len(t)
    h = pm.rms_norm(w["embed"][torch.tensor(t)], eps, w["l0.norm1"])
    q = pm.rms_norm(pm.rotate((h @ w["l0.mix.left.q"].T).view(n, m["heads"], m["dim"]), m.get("rot")), eps)
    k = pm.rms_norm(pm.rotate((h @ w["l0.mix.left.k"].T).view(n, m["kv_heads"], m["dim"]), m.get("rot")), eps)
    k = k.repeat_interleave(m["heads"] // m["kv_heads"], 1)
    s = torch.einsum("thd,uhd->htu", q, k) * m["scale"]
    p = torch.softmax(s.masked_fill(~torch.ones(n, n, dtype=torch.bool).tril(), float("-inf")), -1)
    best, where = p[:, 2 * back:].max(-1)
    return bool(((torch.arange(2 * back, n)[None] - where >= back) & (best > 0.5)).any())


def test_a_far_key_carries_the_result(cases):
    """Peaked attention: rows whose weight sits on one key hundreds of positions back, across cache blocks, in a
    prompt and in decoding; a key that is one place off, or a block's edge that is handled wrongly, shows."""
    case = cases("attention", sharp=5.0)
    t = mc.tokens(330, case.vocab, 21)
    want = case.want(t)
    assert mc.err(case.run_cut(t, [330]), want) < TOL
    assert mc.err(case.run_cut(t, [127, 1, 64, 2, 100]), want) < TOL
    assert far_attention_rows(case, t)


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    """Decays close to one: the first tokens still weigh in the state after hundreds of steps, so a state that is
    lost, reset or carried to the wrong slot shows far from where it happened."""
    case = cases("delta", memory=7.0)
    t = mc.tokens(260, case.vocab, 31)
    want = case.want(t)
    other = case.want([(t[0] + 1) % case.vocab] + t[1:])
    assert mc.err(other[-1], want[-1]) > 1e-3  # the first token still matters at the end
    assert mc.err(case.run_cut(t, [260]), want) < TOL
    assert mc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL


def test_the_first_tokens_see_zeros_ahead_of_the_sequence(cases):
    """The short convolutions read zeros before the first token, also in a slot that another sequence has left, and
    whether the first step brings one token or several."""
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
        assert mc.err(out, case.want(b)[:first]) < TOL
        if first < 6:
            out = eng.step([StepEntry(s, b[first:], range(6 - first))])
            assert mc.err(out, case.want(b)[first:]) < TOL
        eng.release(s)
    case.assert_idle()


def test_long_decoding(cases):
    mc.long_decoding(cases("a"), TOL)


def test_greedy_generation_through_the_generation_loop(cases):
    case = cases("a")
    reqs, wants = mc.greedy(case)
    result = lq.generate(case.eng, reqs, max_new_tokens=10)
    assert result.tokens == wants
    case.assert_idle()


def test_bfloat16_run_rounds_where_the_plain_implementation_does(tmp_path_factory):
    case = mc.Case(tmp_path_factory.mktemp("mifidra16"), "a", load, dtype="bfloat16", rounding=True)
    t = mc.tokens(80, case.vocab, 3)
    mc.assert_close_bf16(case.run_cut(t, [50, 2]), case.want(t), case.noise(t))
