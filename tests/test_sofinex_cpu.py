"""The Sofinex design through the engine's own code (registry, loader, cache groups, step function, generation
loop) on the CPU, over the torch stand-in for the kernels, against the plain implementation.  The GPU tests
repeat every scenario with the HIP kernels; these catch faults of the parts, the cache and the batching."""
import copy
import math

import pytest
import torch

import longbow_quarrel_amd as lq
import plain_sofinex as ps
import sofinex_cases as sc
from cpu_kernels import CpuKernels
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.parts.base import KVNeed, MultiNeed, StateNeed

TOL = 2e-5
F = torch.float64


def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=CpuKernels(),
                          max_slots=8, max_sequence_tokens=max_tokens)


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, **kw):
        key = (name, tuple(sorted((k, str(v)) for k, v in kw.items())))
        if key not in made:
            made[key] = sc.Case(tmp_path_factory.mktemp("sofinex"), name, load, **kw)
        return made[key]

    return get


# ---- configuration, registry, tensors, cache needs ----------------------------------------------------------------
def test_configuration_reads_every_size_and_writes_the_same_keys_back():
    for cfg in sc.CONFIGS.values():
        assert lq.SofinexConfig.from_dict(cfg).to_dict() == cfg
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import config_from_dict, spec_from_config

    config = config_from_dict(sc.CFG_A)
    assert isinstance(config, lq.SofinexConfig)
    model = DecoderModel(spec_from_config(config))
    # layers 1 and 2 run three times in a row, nothing else happens between the passes
    assert [(r.layer, r.add_input) for r in model.spec.schedule] == [
        (0, False), (1, False), (2, False), (1, False), (2, False), (1, False), (2, False), (3, False), (4, False)]
    specs = {s.name: s for s in model.tensor_specs()}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm2", "l0.mix.left.sink", "l0.mix.left.out",
            "l0.mix.right.out", "l0.mix.right.q.conv", "l0.mix.right.a2", "l0.mlp.up", "l1.mix.lq1", "l1.mix.lk2",
            "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e3.down", "l1.mlp.shared.sg", "l4.mlp.shared.up"} <= set(specs)
    assert "l0.mlp.gate" not in specs and "l1.mlp.e4.up" not in specs  # no gate in a dense layer; identity experts have no tensors
    assert not any(n.startswith("l2.mlp") for n in specs) and "l3.mlp.shared.up" not in specs
    assert specs["l2.norm2"].optional and not specs["l1.norm2"].optional
    shapes = {n: tuple(s.shape) for n, s in specs.items()}
    assert shapes["l1.mix.q"] == (2 * 2 * 16, 80) and shapes["l1.mix.k"] == (2 * 2 * 16, 80)
    assert shapes["l1.mix.v"] == (2 * 40, 80) and shapes["l1.mix.o"] == (80, 2 * 40) and shapes["l1.mix.lq2"] == (16,)
    assert shapes["l3.mix.q"] == (3 * 2 * 8, 80) and shapes["l3.mix.k"] == (1 * 2 * 8, 80) and shapes["l3.mix.v"] == (24, 80)
    assert shapes["l0.mix.left.q"] == (6 * 24, 80) and shapes["l0.mix.left.sink"] == (6,)
    assert shapes["l1.mlp.router"] == (6, 80) and shapes["l1.mlp.correction"] == (6,)  # four experts and two identity ones
    assert shapes["l1.mlp.shared.sg"] == (1, 80) and shapes["l0.mlp.up"] == (56, 80)
    # every run of a layer has a cache of its own.  Differential attention keeps both maps' keys in one row a kv head
    needs = model.cache_needs()
    assert len(needs) == 9
    assert needs[1] == KVNeed(2, 2 * 16, 70, 40) and needs[1] == needs[3] == needs[5]
    assert needs[7] == KVNeed(1, 2 * 8, 1000, 24) and needs[8] == KVNeed(2, 2 * 12, 0, 12)
    assert needs[0] == MultiNeed((KVNeed(2, 24, 20, 16), MultiNeed((StateNeed((4, 20, 12), torch.float32),
                                                                     StateNeed((3, 2 * 2 * 12 + 4 * 20), torch.float32)))))
    assert needs[2].needs[0] == KVNeed(1, 32, 130, 32) and needs[2] == needs[4] == needs[6]


@pytest.mark.parametrize("key,value,text", [
    (("layers", 0, "type"), "delta", "layers[0].type"),
    (("layers", 0, "mixer", "left", "kv_heads"), 4, "kv_heads"),
    (("layers", 0, "mixer", "left", "scale"), None, "left.scale"),
    (("layers", 0, "mixer", "left", "mask", "size"), 0, "mask.size"),
    (("layers", 0, "mixer", "left", "rot", "dims"), 7, "rot.dims"),
    (("layers", 0, "mixer", "left", "rot", "dims"), 26, "rot.dims"),
    (("layers", 0, "mixer", "left", "rot", "scaling", "factor"), None, "rot.scaling.factor"),
    (("layers", 0, "mixer", "right", "conv"), 0, "right.conv"),
    (("layers", 1, "mixer", "diff"), None, "mixer.diff"),
    (("layers", 1, "mixer", "rot", "scaling", "high"), None, "rot.scaling.high"),
    (("layers", 1, "mixer", "rot", "scaling", "high"), 1.0, "rot.scaling"),
    (("layers", 0, "mlp", "kind"), "glu", "mlp.kind"),
    (("layers", 1, "mlp", "router", "top"), 7, "router.top"),
    (("layers", 1, "mlp", "router", "top"), 3, "groups"),
    (("layers", 1, "mlp", "router", "identity"), 1, "groups"),
    (("layers", 1, "mlp", "router", "groups", "keep"), 4, "groups"),
    (("layers", 1, "mlp", "expert", "ff"), None, "expert.ff"),
    (("loop", "stop"), 6, "loop"),
    (("loop", "times"), 0, "loop.times"),
    (("norm", "eps"), "tiny", "norm.eps"),
    (("embedding", "scale"), "big", "embedding.scale"),
    (("width",), None, "width"),
])
def test_configuration_errors_name_their_key(key, value, text):
    cfg = copy.deepcopy(sc.CFG_A)
    d = cfg
    for k in key[:-1]:
        d = d[k]
    d[key[-1]] = value
    with pytest.raises(lq.ConfigError) as e:
        lq.SofinexConfig.from_dict(cfg)
    assert text in str(e.value)


def test_keys_that_a_configuration_leaves_out():
    cfg = copy.deepcopy(sc.CFG_DIFF)
    m = cfg["layers"][0]["mixer"]
    del m["kv_heads"], m["vdim"], m["mask"], m["rot"], cfg["embedding"]
    got = lq.SofinexConfig.from_dict(cfg)
    a = got.layers[0].attention
    assert (a.kv_heads, a.vdim, a.window, a.rot) == (4, 16, 0, None)
    assert got.embedding_scale == 1.0 and got.loop is None and got.run_order() == [0]
    cfg = copy.deepcopy(sc.CFG_MOE)
    router = cfg["layers"][0]["mlp"]["router"]
    del router["identity"], router["groups"]
    mlp = lq.SofinexConfig.from_dict(cfg).layers[0].mlp
    assert (mlp.identity, mlp.groups, mlp.keep) == (0, 0, 0)


def test_sizes_that_no_key_gives_come_from_the_file(tmp_path):
    cfg = copy.deepcopy(sc.CFG_A)
    weights = sc.make_weights(cfg, 5)
    for layer in cfg["layers"]:
        if layer["type"] == "parallel":
            del layer["mixer"]["right"]["decay_rank"], layer["mixer"]["right"]["gate_rank"]
    eng = load(sc.write_folder(tmp_path, cfg, weights, "norank"), "float32", 256)
    assert [(x.right.decay_rank, x.right.gate_rank) for x in eng.config.layers if x.right] == [(6, 10), (8, 8)]
    t = sc.tokens(20, cfg["vocab"], 1)
    got = eng.step([StepEntry(eng.new_sequence(), t, range(20))])
    assert sc.err(got, ps.forward(cfg, weights, t)) < TOL
    with pytest.raises(lq.ConfigError) as e:
        lq.random_engine(lq.SofinexConfig.from_dict(cfg), 1, device="cpu", kernels=CpuKernels())
    assert "rank" in str(e.value)


def test_the_norm_of_an_absent_feed_forward_may_be_in_the_file(tmp_path):
    cfg = copy.deepcopy(sc.CFG_DIFF)
    weights = sc.make_weights(cfg, 5)
    weights.pop("l0.norm2", None)
    t = sc.tokens(12, cfg["vocab"], 1)
    got = []
    for name, more in (("without", {}), ("with", {"l0.norm2": torch.full((cfg["width"],), 3.0)})):
        eng = load(sc.write_folder(tmp_path, cfg, {**weights, **more}, name), "float32", 256)
        got.append(eng.step([StepEntry(eng.new_sequence(), t, range(12))]))
    assert torch.equal(got[0], got[1]) and sc.err(got[0], ps.forward(cfg, weights, t)) < TOL


def test_missing_and_unexpected_tensors_are_named(tmp_path):
    cfg = copy.deepcopy(sc.CFG_MOE)  # nine experts and three identity ones
    weights = sc.make_weights(cfg, 5)
    weights["l0.mlp.e9.up"] = weights["l0.mlp.e0.up"].clone()  # an identity expert has no tensors
    del weights["l0.mlp.shared.sg"], weights["l0.mix.lk1"]
    with pytest.raises(lq.WeightError) as e:
        load(sc.write_folder(tmp_path, cfg, weights, "bad"), "float32", 256)
    assert e.value.missing == ["l0.mix.lk1", "l0.mlp.shared.sg"] and e.value.unexpected == ["l0.mlp.e9.up"]


# ---- the plain implementation's own mechanisms against hand-made cases ---------------------------------------------
def test_plain_rotation_pairs_an_entry_with_the_one_half_the_rotated_part_on():
    rot = {"base": 100.0, "dims": 4}
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]] * 4, dtype=F)
    y = ps.rotate_half(x, rot)
    f = [1.0, 100.0 ** -0.5]
    c0, s0, c1, s1 = math.cos(3 * f[0]), math.sin(3 * f[0]), math.cos(3 * f[1]), math.sin(3 * f[1])
    assert torch.equal(y[0], x[0])  # position 0
    # pairs (0, 2) and (1, 3); entries 4 and 5 pass
    assert torch.allclose(y[3, 0], torch.tensor([1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1,
                                                 5.0, 6.0], dtype=F))


def test_plain_frequency_blend_by_wavelength_and_the_librarys():
    """Short waves keep their frequency, long ones are divided by the factor, those between are blended by where
    their wavelength lies between original / high and original / low; cos and sin are not stretched."""
    from longbow_quarrel_amd.config.sofinex import RotaryTurn
    from longbow_quarrel_amd.parts.rope import rotary_frequencies, rotary_magnitude

    for dims, base, s in ((32, 10000.0, {"factor": 4.0, "original": 2000, "low": 1.0, "high": 4.0}),
                          (16, 3000.0, {"factor": 6.0, "original": 48, "low": 2.0, "high": 3.0}),
                          (8, 100.0, {"factor": 2.0, "original": 16, "low": 0.5, "high": 8.0}),
                          (12, 50.0, {"factor": 3.0, "original": 7, "low": 1.0, "high": 1.5})):
        f, mag = ps.frequencies({"base": base, "dims": dims, "scaling": s})
        plain = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
        assert mag == 1.0
        assert bool(((f <= plain * (1 + 1e-12)) & (f >= plain / s["factor"] * (1 - 1e-12))).all())
        params = RotaryTurn.from_dict({"base": base, "dims": dims, "scaling": s}, "rot", dims).as_parameters()
        assert params["pairing"] == "half"
        lib = rotary_frequencies(dims, base, params["scaling"])
        assert torch.allclose(torch.tensor(lib, dtype=F), f, rtol=1e-12, atol=0)
        assert rotary_magnitude(params["scaling"]) == 1.0
    # base 10000 over 32 entries, 2000 positions: wavelengths 2 pi 10000^(i / 16).  Pair 0 (6.3) and pair 7 (354) are
    # shorter than 2000 / 4; pair 11 (3 533) and the last are longer than 2000 / 1; pair 9 (1 117) lies between:
    # s = (2000 / 1117.3 - 1) / 3
    f, _ = ps.frequencies({"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 2000, "low": 1.0,
                                                                    "high": 4.0}})
    assert float(f[0]) == 1.0 and float(f[7]) == 10000.0 ** (-14 / 32)
    assert float(f[11]) == pytest.approx(10000.0 ** (-22 / 32) / 4, rel=1e-12)
    wave = 2 * math.pi * 10000.0 ** (18 / 32)
    s = (2000 / wave - 1.0) / 3.0
    assert 0.2 < s < 0.3
    assert float(f[9]) == pytest.approx(10000.0 ** (-18 / 32) * ((1 - s) / 4 + s), rel=1e-12)
    # a scaling with `fast` and `slow` is the other kind: a ramp over the pairs, and cos and sin stretched
    params = RotaryTurn.from_dict({"base": 3000.0, "dims": 16, "scaling": sc.YARN}, "rot", 16).as_parameters()
    f, mag = ps.frequencies({"base": 3000.0, "dims": 16, "scaling": sc.YARN})
    assert mag == 0.1 * math.log(6.0) + 1 == rotary_magnitude(params["scaling"])
    assert torch.allclose(torch.tensor(rotary_frequencies(16, 3000.0, params["scaling"]), dtype=F), f, rtol=1e-12, atol=0)


def test_plain_window_sees_itself_and_the_tokens_before_it():
    seen = ps.window_mask(6, 3)
    assert seen.tolist() == [[j <= i and i - j < 3 for j in range(6)] for i in range(6)]
    assert seen[5].tolist() == [False, False, False, True, True, True]
    assert ps.window_mask(4, 1).tolist() == torch.eye(4, dtype=torch.bool).tolist()


def test_plain_softmax_with_a_sink():
    """The sink adds exp(b) to the denominator and nothing else: with scores 0 and ln 3 and b = ln 4 the weights
    are 1/8 and 3/8, and a hidden column takes no part."""
    score = torch.tensor([[0.0, math.log(3.0), 50.0]], dtype=F)
    seen = torch.tensor([[True, True, False]])
    p = ps.softmax_rows(score, seen, math.log(4.0))
    assert torch.allclose(p, torch.tensor([[1 / 8, 3 / 8, 0.0]], dtype=F))
    assert torch.allclose(ps.softmax_rows(score, seen), torch.tensor([[1 / 4, 3 / 4, 0.0]], dtype=F))
    # a sink far above the scores takes nearly all the weight; one far below none
    assert float(ps.softmax_rows(score, seen, 40.0).sum()) < 1e-15
    assert float(ps.softmax_rows(score, seen, -40.0).sum()) == pytest.approx(1.0)


def _diff_weights(width, m, **given):
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    w = {"q": torch.zeros(H * 2 * d, width), "k": torch.zeros(G * 2 * d, width), "v": torch.zeros(G * vd, width),
         "lq1": torch.zeros(d), "lk1": torch.zeros(d), "lq2": torch.zeros(d), "lk2": torch.zeros(d),
         "o": torch.eye(H * vd)}
    w.update({k: torch.tensor(v) for k, v in given.items()})
    return {"x." + k: v.to(F) for k, v in w.items()}


def test_plain_differential_attention_takes_the_second_map_off_the_first():
    """One head, maps of one entry, two value channels.  Token 0 has value (1, 0), token 1 value (0, 1).  At token 1
    map 1 scores the keys 0 and ln 3 (weights 1/4, 3/4) and map 2 scores both 0 (weights 1/2, 1/2).  With
    lambda = exp(0.5 * 2) - exp(0) + 0.25 the result is a1 - lambda a2, then the norm over the two channels and the
    factor 1 - 0.25."""
    m = {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 2, "scale": 1.0, "diff": 0.25, "mask": {"size": 8}}
    ln3 = math.log(3.0)
    # the input's columns: the key of map 1, value channel 0, value channel 1, one
    w = _diff_weights(4, m, q=[[0, 0, 0, 1.0], [0, 0, 0, 1.0]], k=[[1.0, 0, 0, 0], [0, 0, 0, 0]],
                      v=[[0, 1.0, 0, 0], [0, 0, 1.0, 0]], lq1=[0.5], lk1=[2.0])
    h = torch.tensor([[0.0, 1, 0, 1], [ln3, 0, 1, 1]], dtype=F)
    lam = math.e - 1 + 0.25
    assert ps.differential_lambda(w, "x", 0.25) == pytest.approx(lam)
    y = ps.differential_attention(h, m, w, "x", 0.0, False)
    o = torch.tensor([1 / 4 - lam / 2, 3 / 4 - lam / 2], dtype=F)
    assert torch.allclose(y[1], o / torch.sqrt((o * o).mean()) * 0.75)
    # the first token sees itself alone in both maps: (1 - lambda) (1, 0), normed
    assert torch.allclose(y[0], torch.tensor([-math.sqrt(2.0) * 0.75, 0.0], dtype=F))


def test_plain_differential_maps_lie_head_by_head_and_share_the_kv_heads_values():
    """Two query heads on one key/value head: rows of q are (head 0 map 1, head 0 map 2, head 1 map 1, head 1 map 2).
    Swapping the two maps' rows of a head is another model; with lambda = 1 it flips that head's sign."""
    m = {"heads": 2, "kv_heads": 1, "dim": 2, "vdim": 3, "scale": 0.7, "diff": 0.0, "mask": {"size": 4}}
    g = torch.Generator().manual_seed(1)
    w = {"x." + k: torch.randn(s, generator=g, dtype=F) for k, s in
         (("q", (8, 5)), ("k", (4, 5)), ("v", (3, 5)), ("o", (6, 6)))}
    w.update({"x." + k: torch.zeros(2, dtype=F) for k in ("lq1", "lk1", "lq2", "lk2")})  # lambda = 1 - 1 + 0
    w["x.lq1"] = torch.tensor([math.log(2.0), 0.0], dtype=F)
    w["x.lk1"] = torch.tensor([1.0, 5.0], dtype=F)  # lambda = 2 - 1 + 0 = 1
    w["x.o"] = torch.eye(6, dtype=F)
    h = torch.randn(5, 5, generator=g, dtype=F)
    y = ps.differential_attention(h, m, w, "x", 0.0, False)
    swapped = dict(w)
    swapped["x.q"] = w["x.q"][[2, 3, 0, 1, 4, 5, 6, 7]]
    swapped["x.k"] = w["x.k"][[2, 3, 0, 1]]
    z = ps.differential_attention(h, m, swapped, "x", 0.0, False)
    # both heads read the swapped keys; head 0 also swapped its queries, so its maps trade places: a2 - a1
    assert torch.allclose(z[1:, :3], -y[1:, :3]) and not torch.allclose(z[1:, 3:], y[1:, 3:])


def test_plain_router_scores_by_softmax_and_marks_a_group_by_its_best():
    r = {"experts": 4, "identity": 2, "top": 2, "groups": {"count": 3, "keep": 2}}
    z = [2.0, -3.0, 0.5, 0.4, -1.0, 1.5]  # groups (0, 1), (2, 3), (4, 5); outputs 4 and 5 are identity experts
    w = {"m.router": torch.tensor([[v] for v in z], dtype=F),
         "m.correction": torch.tensor([-0.5, 0.3, 0.0, 0.0, 0.05, -0.2], dtype=F)}
    s, chosen = ps.route(torch.ones(1, 1, dtype=F), r, w, "m")
    e = [math.exp(v) for v in z]
    soft = [v / sum(e) for v in e]
    assert torch.allclose(s[0], torch.tensor(soft, dtype=F))
    # scores .460 .003 .103 .093 .023 .279; choice scores -.040 .303 .103 .093 .073 .079; the groups' best: .303
    # .103 .079: groups 0 and 1 stay, the choice is outputs 1 and 2, and output 0, whose score is the largest, is not
    # chosen.  With the sum of a group's two best as its mark group 0 would still be kept; with keep = 1 only group 0
    assert chosen == [[1, 2]]
    r["groups"]["keep"] = 1
    assert ps.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[1, 0]]
    # the best groups by their largest score, not by the sum of their two largest: group 2 (0.02, 0.55) beats
    # group 1 (0.3, 0.3)
    w["m.correction"] = torch.tensor([-9.0, -9.0, 0.3 - soft[2], 0.3 - soft[3], 0.02 - soft[4], 0.55 - soft[5]], dtype=F)
    assert ps.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[5, 4]]
    # choice scores may all be negative: an expert outside the kept groups still cannot be chosen
    w["m.correction"] = torch.tensor([-7.0, -7.5, -9.0, -9.5, -8.0, -8.5], dtype=F)
    assert ps.route(torch.ones(1, 1, dtype=F), r, w, "m")[1] == [[0, 1]]


def test_plain_experts_renormalise_and_identity_experts_hand_their_input_on():
    r = {"experts": 2, "identity": 1, "top": 2}
    z = [0.0, math.log(2.0), math.log(5.0)]  # scores 1/8, 2/8, 5/8
    w = {"m.router": torch.tensor([[v, 0.0] for v in z], dtype=F), "m.correction": torch.zeros(3, dtype=F)}
    for e in range(2):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"] = torch.tensor([[1.0, 0.0]], dtype=F), torch.tensor([[1.0, 0.0]], dtype=F)
        w[f"m.e{e}.down"] = torch.tensor([[10.0 ** (e + 1)], [0.0]], dtype=F)
    h = torch.tensor([[1.0, 3.0]], dtype=F)
    mlp = {"router": r, "expert": {"ff": 1}}
    act = 1 / (1 + math.exp(-1.0))
    # chosen: output 2 (identity, 5/8) and expert 1 (2/8); weights 5/7 and 2/7
    assert torch.allclose(ps.experts(h, mlp, w, "m", False),
                          torch.tensor([[5 / 7 * 1.0 + 2 / 7 * act * 100, 5 / 7 * 3.0]], dtype=F))
    # the correction moves the choice and not the weights: expert 0 in the identity expert's place, weights 1/3, 2/3
    w["m.correction"] = torch.tensor([0.0, 0.0, -1.0], dtype=F)
    assert torch.allclose(ps.experts(h, mlp, w, "m", False),
                          torch.tensor([[1 / 3 * act * 10 + 2 / 3 * act * 100, 0.0]], dtype=F))
    # a shared expert behind a gate of one number a token: sigmoid(ln 3) = 3/4
    mlp["shared"] = {"ff": 1}
    w["m.shared.gate"], w["m.shared.up"] = torch.tensor([[1.0, 0.0]], dtype=F), torch.tensor([[2.0, 0.0]], dtype=F)
    w["m.shared.down"] = torch.tensor([[0.0], [1000.0]], dtype=F)
    w["m.shared.sg"] = torch.tensor([[math.log(3.0), 0.0]], dtype=F)
    assert torch.allclose(ps.experts(h, mlp, w, "m", False),
                          torch.tensor([[1 / 3 * act * 10 + 2 / 3 * act * 100, 0.75 * act * 2 * 1000]], dtype=F))


def test_plain_dense_layer_uses_the_exact_gelu():
    w = {"m.up": torch.tensor([[1.0]], dtype=F), "m.down": torch.tensor([[1.0]], dtype=F)}
    y = ps.dense(torch.tensor([[1.0], [-2.0]], dtype=F), w, "m", False)
    assert float(y[0]) == pytest.approx(0.5 * (1 + math.erf(1 / math.sqrt(2))), rel=1e-12)
    assert float(y[1]) == pytest.approx(-2.0 * 0.5 * (1 + math.erf(-2 / math.sqrt(2))), rel=1e-12)
    assert abs(float(y[1]) - (-2.0 * 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * (-2 - 0.044715 * 8))))) > 5e-5


def test_plain_norm_stores_its_gain_around_zero():
    x = torch.tensor([[3.0, 4.0]], dtype=F)
    y = ps.one_plus_norm(x, 0.0, torch.tensor([0.0, -0.5], dtype=F))
    assert torch.allclose(y, torch.tensor([[3 / math.sqrt(12.5), 0.5 * 4 / math.sqrt(12.5)]], dtype=F))


# ---- every mechanism alone, and all of them, through the engine ------------------------------------------------------
@pytest.mark.parametrize("name", ["diff", "sink", "delta", "dense", "moe", "loop"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    sc.whole_and_token_by_token(case, TOL, lengths=(1, 2, 9, 70))
    sc.portions(case, TOL, n=140)


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_against_token_by_token_decoding(cases, name):
    sc.whole_and_token_by_token(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_portions_of_several_sizes_down_to_two_tokens(cases, name):
    sc.portions(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_batches_of_unequal_requests_against_each_alone(cases, name):
    sc.unequal_batches(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "loop"])
def test_slots_and_blocks_are_freed_and_used_again(cases, name):
    sc.slots_and_blocks_used_again(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "moe"])
def test_prompt_rows_sorted_by_expert(cases, name, monkeypatch):
    """A prompt step of many rows sorts them by expert and runs every expert over its own rows; the identity
    experts' share and the gated shared expert are added beside: the same logits."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    case = cases(name)
    t = sc.tokens(90, case.vocab, 12)
    assert sc.err(case.run_cut(t, [50, 3, 30]), case.want(t)) < TOL


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_configurations_drawn_from_a_seed(cases, seed):
    case = cases(seed)
    assert lq.SofinexConfig.from_dict(case.cfg).to_dict() == case.cfg
    t, u = sc.tokens(70, case.vocab, seed), sc.tokens(9, case.vocab, seed + 50)
    assert sc.err(case.run_cut(t, [40, 2, 1, 20]), case.want(t)) < TOL
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:66], range(66))])
    assert sc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:66]])) < TOL
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[66:67], [0])])
    assert sc.err(out, torch.stack([case.want(u)[8], case.want(t)[66]])) < TOL
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(sc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 9
    for i, (g, w) in enumerate(zip(got, want)):
        assert sc.err(g, w) < TOL, f"after layer run {i}"


def test_every_pass_of_a_loop_has_a_cache_of_its_own(cases):
    """Were two passes to share keys or a state, the second pass would read what the first wrote for the same
    positions: against the plain implementation, in decoding after a prompt; and the plain implementation without
    the loop differs by much."""
    case = cases("loop")
    t = sc.tokens(50, case.vocab, 4)
    assert sc.err(case.run_cut(t, [30, 5]), case.want(t)) < TOL
    once = copy.deepcopy(case.cfg)
    once["loop"]["times"] = 1
    assert sc.err(ps.forward(once, case.weights, t), case.want(t)) > 1e-2


@pytest.mark.parametrize("kind", ["diff", "sink"])
@pytest.mark.parametrize("window", [1, 2, 63, 64, 65, 130])
def test_keys_just_inside_and_just_outside_the_window(cases, kind, window):
    """Peaked attention under windows of one token, of a cache block less one, a block, a block and one, and two
    blocks and two: the last key a row sees and the first it does not, in a prompt, across portions and in
    decoding.  The plain implementation with a window one token off differs by much at these rows."""
    case = cases(f"{kind}-window-{window}", cfg=sc.windowed(kind, window), sharp=6.0)
    n = max(2 * window + 10, 80)
    t = sc.tokens(n, case.vocab, 40 + window)
    rows = list(range(window, n))
    sc.a_window_off_by_one_would_show(case, t, kind, rows)
    want = case.want(t)
    assert sc.err(case.run_cut(t, [n]), want) < TOL
    assert sc.err(case.run_cut(t, [window, 1, 1, 2, window - 1 or 1, 3]), want) < TOL
    assert sc.err(case.run_cut(t, [max(1, window - 1)]), want) < TOL  # decoding across the window's edge
    case.assert_idle()


def test_the_sink_takes_weight_from_every_row(cases):
    """Without the sink's term the result differs by much; and a sink score is per query head, not scaled."""
    case = cases("sink")
    t = sc.tokens(30, case.vocab, 9)
    for change in (lambda s: s - 30.0, lambda s: s.flip(0), lambda s: s * case.cfg["layers"][0]["mixer"]["left"]["scale"]):
        other = dict(case.weights)
        other["l0.mix.left.sink"] = change(case.weights["l0.mix.left.sink"])
        assert sc.err(ps.forward(case.cfg, other, t), case.want(t)) > 1e-3
    assert sc.err(case.run_cut(t, [20, 2]), case.want(t)) < TOL


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    """Decays close to one: the first tokens still weigh in the state after hundreds of steps, far beyond every
    window, so a state that is lost, reset or carried to the wrong slot shows far from where it happened."""
    case = cases("delta", memory=7.0)
    t = sc.tokens(260, case.vocab, 31)
    want = case.want(t)
    other = case.want([(t[0] + 1) % case.vocab] + t[1:])
    assert sc.err(other[-1], want[-1]) > 1e-3  # the first token still matters at the end
    assert sc.err(case.run_cut(t, [260]), want) < TOL
    assert sc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL


def test_the_first_tokens_see_zeros_ahead_of_the_sequence(cases):
    """The short convolutions read zeros before the first token and the windows are not yet full, also in a slot that
    another sequence has left, and whether the first step brings one token or several."""
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
        assert sc.err(out, case.want(b)[:first]) < TOL
        if first < 6:
            out = eng.step([StepEntry(s, b[first:], range(6 - first))])
            assert sc.err(out, case.want(b)[first:]) < TOL
        eng.release(s)
    case.assert_idle()


def test_windowed_groups_give_their_blocks_back(cases):
    """A window of 20 tokens never needs more than two blocks a sequence however long it grows, and every run of a
    layer holds blocks of its own."""
    case = cases("sink")  # one layer, a window of 40
    eng = case.eng
    s = eng.new_sequence()
    t = sc.tokens(400, case.vocab, 3)
    eng.step([StepEntry(s, t[:300], [])])
    for i in range(300, 400):
        eng.step([StepEntry(s, t[i : i + 1], [])])
    assert all(g.blocks.taken_count <= 2 for g in eng.cache.kv_groups)
    out = eng.step([StepEntry(s, [5], [0])])
    assert sc.err(out[0], case.want(t + [5])[-1]) < TOL
    eng.release(s)
    case.assert_idle()


def test_long_decoding(cases):
    sc.long_decoding(cases("a"), TOL)


def test_greedy_generation_through_the_generation_loop(cases):
    case = cases("a")
    reqs, wants = sc.greedy(case)
    result = lq.generate(case.eng, reqs, max_new_tokens=10)
    assert result.tokens == wants
    case.assert_idle()


def test_bfloat16_run_rounds_where_the_plain_implementation_does(tmp_path_factory):
    case = sc.Case(tmp_path_factory.mktemp("sofinex16"), "a", load, dtype="bfloat16", rounding=True)
    t = sc.tokens(80, case.vocab, 3)
    sc.assert_close_bf16(case.run_cut(t, [50, 2]), case.want(t), case.noise(t))
