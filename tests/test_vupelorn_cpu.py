"""The Vupelorn design through the engine's own code (registry, loader, cache groups, step function, generation
loop) on the CPU, over the torch stand-in for the kernels, against the plain implementation.  The GPU tests
repeat every scenario with the HIP kernels; these catch faults of the parts, the cache and the batching."""
import copy
import math

import pytest
import torch

import longbow_quarrel_amd as lq
import plain_vupelorn as pv
import vupelorn_cases as uc
from cpu_kernels import CpuKernels
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.model import EMBEDDING_RUN
from longbow_quarrel_amd.parts.base import KVNeed, StateNeed

TOL = 2e-5


def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=CpuKernels(),
                          max_slots=8, max_sequence_tokens=max_tokens)


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, **kw):
        key = (name, tuple(sorted(kw.items())))
        if key not in made:
            made[key] = uc.Case(tmp_path_factory.mktemp("vupelorn"), name, load, **kw)
        return made[key]

    return get


# ---- configuration, registry, tensors, cache needs ----------------------------------------------------------------
def test_configuration_reads_every_size_and_writes_the_same_keys_back():
    for cfg in uc.CONFIGS.values():
        assert lq.VupelornConfig.from_dict(cfg).to_dict() == cfg
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import config_from_dict, spec_from_config

    model = DecoderModel(spec_from_config(config_from_dict(uc.CFG_A)))
    assert [(r.layer, r.cache_of) for r in model.spec.schedule] == [(0, None), (1, None), (2, None), (3, 2), (4, None)]
    names = {s.name for s in model.tensor_specs()}
    assert {"bigram", "l0.mix.dkv.norm", "l1.mix.a2.b", "l2.mix.dkv", "l3.mix.uk", "l0.mlp.e4.down", "l0.mlp.router",
            "l4.norm2", "final.norm"} <= names
    assert "l3.mix.dkv" not in names and "l3.mix.dkv.norm" not in names  # the layer reads another's latent
    assert not any(n.startswith("l1.mlp") for n in names)  # no feed-forward
    # the norm of a feed-forward that is not there may be in a file or not
    assert [s.optional for s in model.tensor_specs() if s.name == "l1.norm2"] == [True]
    assert "head" not in names  # the head is the embedding
    needs = model.cache_needs()
    assert set(needs) == {EMBEDDING_RUN, 0, 1, 2, 4}
    assert needs[0] == KVNeed(1, 48 + 16, 0, 48) and needs[2] == KVNeed(1, 32 + 8, 0, 32)
    assert needs[1] == StateNeed((2, 24, 40), torch.float32) and needs[EMBEDDING_RUN] == StateNeed((1,), torch.int32)


@pytest.mark.parametrize("key,value,text", [
    (("layers", 0, "type"), "attention", "layers[0].type"),
    (("layers", 0, "mixer", "kv_rank"), None, "layers[0].mixer.kv_rank"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"),
    (("layers", 0, "mixer", "rot", "dims"), 32, "rot.dims"),
    (("layers", 0, "mixer", "rot", "scaling", "factor"), None, "rot.scaling.factor"),
    (("layers", 0, "mlp", "router", "top"), 6, "router.top"),
    (("layers", 0, "mlp", "kind"), "dense", "mlp.kind"),
    (("layers", 1, "mixer", "tau"), 0.0, "tau"),
    (("layers", 3, "mixer", "kv_from"), 3, "kv_from"),
    (("layers", 3, "mixer", "kv_from"), 1, "kv_from"),
    (("layers", 3, "mixer", "kv_rank"), 16, "differ"),
    (("embedding", "bigram", "buckets"), 0, "embedding.bigram.buckets"),
    (("norm", "eps"), "tiny", "norm.eps"),
    (("width",), None, "width"),
])
def test_configuration_errors_name_their_key(key, value, text):
    cfg = copy.deepcopy(uc.CFG_A)
    d = cfg
    for k in key[:-1]:
        d = d[k]
    d[key[-1]] = value
    with pytest.raises(lq.ConfigError) as e:
        lq.VupelornConfig.from_dict(cfg)
    assert text in str(e.value)


def test_keys_that_a_configuration_leaves_out_take_the_sizes_they_follow():
    cfg = copy.deepcopy(uc.CFG_LATENT2)
    m = cfg["layers"][0]["mixer"]
    del m["rot"]["dims"], m["vdim"]
    got = lq.VupelornConfig.from_dict(cfg).layers[0].latent
    assert got.rot.dims == m["rot_dim"] and got.vdim == m["dim"]


def test_a_size_that_no_key_gives_comes_from_the_file(tmp_path):
    """The rank of the decay's bottleneck is the shape of its first matrix; without a file it must be stated."""
    cfg = copy.deepcopy(uc.CFG_GLA)
    weights = uc.make_weights(cfg, 5)
    del cfg["layers"][0]["mixer"]["decay_rank"]
    folder = uc.write_folder(tmp_path, cfg, weights, "norank")
    eng = load(folder, "float32", 256)
    assert eng.config.layers[0].gla.decay_rank == 4
    t = uc.tokens(20, cfg["vocab"], 1)
    s = eng.new_sequence()
    got = eng.step([StepEntry(s, t, range(20))])
    assert uc.err(got, pv.forward(cfg, weights, t)) < TOL
    with pytest.raises(lq.ConfigError) as e:
        lq.random_engine(lq.VupelornConfig.from_dict(cfg), 1, device="cpu", kernels=CpuKernels())
    assert "decay" in str(e.value)


def test_the_norm_of_an_absent_feed_forward_may_be_in_the_file(tmp_path):
    cfg = copy.deepcopy(uc.CFG_GLA)
    weights = uc.make_weights(cfg, 5)
    assert "l0.norm2" not in weights
    t = uc.tokens(12, cfg["vocab"], 1)
    got = []
    for name, extra in (("without", {}), ("with", {"l0.norm2": torch.full((cfg["width"],), 3.0)})):
        eng = load(uc.write_folder(tmp_path, cfg, {**weights, **extra}, name), "float32", 256)
        got.append(eng.step([StepEntry(eng.new_sequence(), t, range(12))]))
    assert torch.equal(got[0], got[1]) and uc.err(got[0], pv.forward(cfg, weights, t)) < TOL


def test_missing_and_unexpected_tensors_are_named(tmp_path):
    cfg = copy.deepcopy(uc.CFG_LATENT2)
    weights = uc.make_weights(cfg, 5)
    weights["l1.mix.dkv"] = weights["l0.mix.dkv"].clone()  # a layer that reads another's latent has none
    del weights["l0.mix.dq.norm"]
    folder = uc.write_folder(tmp_path, cfg, weights, "bad")
    with pytest.raises(lq.WeightError) as e:
        load(folder, "float32", 256)
    assert e.value.missing == ["l0.mix.dq.norm"] and e.value.unexpected == ["l1.mix.dkv"]


# ---- the plain implementation's own mechanisms against hand-made cases ---------------------------------------------
def test_plain_bigram_rows():
    assert pv.bigram_rows([4, 9, 9, 0], 7, 3, 5) == [7, (4 * 3 + 9 * 5) % 7, (9 * 3 + 9 * 5) % 7, (9 * 3) % 7]


def test_plain_rotation_pairings_and_yarn():
    rot = {"base": 100.0, "dims": 4}
    cos, sin = pv.rotary_table(rot, torch.tensor([0, 3]))
    f = [1.0, 100.0 ** -0.5]
    assert torch.allclose(cos[1], torch.tensor([math.cos(3 * f[0]), math.cos(3 * f[1])], dtype=torch.float64))
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0, 5.0], [1.0, 2.0, 3.0, 4.0, 5.0]], dtype=torch.float64)
    half = pv.rotate(x, cos, sin, 4, interleaved=False)
    inter = pv.rotate(x, cos, sin, 4, interleaved=True)
    assert torch.equal(half[0], x[0]) and torch.equal(inter[0], x[0]) and half[1, 4] == 5 and inter[1, 4] == 5
    c0, s0, c1, s1 = math.cos(3 * f[0]), math.sin(3 * f[0]), math.cos(3 * f[1]), math.sin(3 * f[1])
    assert torch.allclose(half[1, :4], torch.tensor([1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1],
                                                     dtype=torch.float64))
    assert torch.allclose(inter[1, :4], torch.tensor([1 * c0 - 2 * s0, 2 * c0 + 1 * s0, 3 * c1 - 4 * s1, 4 * c1 + 3 * s1],
                                                      dtype=torch.float64))
    # YaRN: pairs that turn often within the original length keep their frequency, slow ones are divided by the
    # factor, and both tables grow by 0.1 ln(factor) + 1
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 2000, "fast": 32.0, "slow": 1.0}}
    cos, sin = pv.rotary_table(rot, torch.tensor([1]))
    mag = 0.1 * math.log(4.0) + 1
    ang = torch.atan2(sin[0], cos[0])
    plain = torch.tensor([10000.0 ** (-2.0 * i / 32) for i in range(16)], dtype=torch.float64)
    assert torch.allclose(cos[0] ** 2 + sin[0] ** 2, torch.full((16,), mag * mag, dtype=torch.float64))
    assert abs(float(ang[0]) - 1.0) < 1e-12 and abs(float(ang[15]) - float(plain[15]) / 4) < 1e-12
    from longbow_quarrel_amd.parts.rope import rotary_frequencies, rotary_magnitude
    sc = {"rope_type": "yarn", **rot["scaling"]}
    assert torch.allclose(torch.tensor(rotary_frequencies(32, 10000.0, sc), dtype=torch.float64), ang, atol=1e-12)
    assert rotary_magnitude(sc) == mag and rotary_magnitude(None) == 1.0


def test_plain_gla_forgets_at_the_rate_of_its_decay():
    """One key channel, two value channels: the first is fed a one at every token, the second at the first token
    only.  The state's two entries are then a geometric sum and a pure power of the decay a = sigmoid(b)^(1 / tau),
    and the norm over the value channels keeps their ratio: a^t (1 - a) / (1 - a^(t + 1))."""
    m = {"heads": 1, "dim": 1, "vdim": 2, "tau": 2.0}
    w = {"q": [[1.0, 0.0]], "k": [[1.0, 0.0]], "v": [[1.0, 0.0], [0.0, 1.0]], "a1": [[0.0, 0.0]], "a2": [[0.0]],
         "a2.b": [0.7], "norm": [1.0, 1.0], "g": [[1.0, 0.0], [1.0, 0.0]], "o": [[1.0, 0.0], [0.0, 1.0]]}
    w = {"x." + k: torch.tensor(v) for k, v in w.items()}
    h = torch.tensor([[1.0, 1.0]] + [[1.0, 0.0]] * 5, dtype=torch.float64)
    y = pv.gla(m, "x.", w, h, 0.0, False)
    a = (1 / (1 + math.exp(-0.7))) ** 0.5
    for t in range(6):
        assert float(y[t, 1] / y[t, 0]) == pytest.approx(a ** t * (1 - a) / (1 - a ** (t + 1)), rel=1e-6)  # (the bias is a 32-bit 0.7)


def test_plain_moe_weights_the_input_of_the_chosen_experts():
    mlp = {"expert": {"ff": 1, "limit": 1.5}, "router": {"experts": 3, "top": 2}}
    w = {"m.router": torch.tensor([[1.0], [3.0], [2.0]])}
    for e, (g, u, d) in enumerate(((1.0, 1.0, 1.0), (2.0, -4.0, 1.0), (0.5, 1.0, 10.0))):
        w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"] = (torch.tensor([[v]]) for v in (g, u, d))
    h = torch.ones(1, 1, dtype=torch.float64)
    s = [1 / (1 + math.exp(-z)) for z in (1.0, 3.0, 2.0)]

    def one(g, u, d, wt):
        g, u = min(g * wt, 1.5), max(-1.5, min(1.5, u * wt))
        return d * g / (1 + math.exp(-1.702 * g)) * (u + 1)

    want = one(2.0, -4.0, 1.0, s[1]) + one(0.5, 1.0, 10.0, s[2])  # experts 1 and 2, each reading s_e h
    assert float(pv.moe(mlp, "m.", w, h, False)) == pytest.approx(want)


# ---- every mechanism alone, and all of them, through the engine ------------------------------------------------------
@pytest.mark.parametrize("name", ["gla", "latent", "latent2", "moe", "bigram"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    uc.whole_and_token_by_token(case, TOL, lengths=(1, 2, 9, 70))
    uc.portions(case, TOL, n=140)


@pytest.mark.parametrize("name", ["a", "b"])
def test_whole_prompts_against_token_by_token_decoding(cases, name):
    uc.whole_and_token_by_token(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_portions_of_several_sizes_down_to_two_tokens(cases, name):
    uc.portions(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_batches_of_unequal_requests_against_each_alone(cases, name):
    uc.unequal_batches(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "b"])
def test_slots_and_blocks_are_freed_and_used_again(cases, name):
    uc.slots_and_blocks_used_again(cases(name), TOL)


@pytest.mark.parametrize("name", ["a", "moe"])
def test_prompt_rows_sorted_by_expert(cases, name, monkeypatch):
    """A prompt step of many rows sorts them by expert and runs every expert over its own rows: the same logits."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    case = cases(name)
    t = uc.tokens(90, case.vocab, 12)
    assert uc.err(case.run_cut(t, [50, 3, 30]), case.want(t)) < TOL


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_configurations_drawn_from_a_seed(cases, seed):
    case = cases(seed)
    assert lq.VupelornConfig.from_dict(case.cfg).to_dict() == case.cfg
    t, u = uc.tokens(70, case.vocab, seed), uc.tokens(9, case.vocab, seed + 50)
    assert uc.err(case.run_cut(t, [40, 2, 1, 20]), case.want(t)) < TOL
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:66], range(66))])
    assert uc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:66]])) < TOL
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[66:67], [0])])
    assert uc.err(out, torch.stack([case.want(u)[8], case.want(t)[66]])) < TOL
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(uc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 5
    for i, (g, w) in enumerate(zip(got, want)):
        assert uc.err(g, w) < TOL, f"after layer {i}"


def test_a_far_key_carries_the_result(cases):
    """Peaked attention: rows whose weight sits on one key hundreds of positions back, across cache blocks, in a
    prompt and in decoding; a key that is one place off, or a block's edge that is handled wrongly, shows."""
    case = cases("latent2", sharp=6.0)
    t = uc.tokens(330, case.vocab, 21)
    want = case.want(t)
    assert uc.err(case.run_cut(t, [330]), want) < TOL
    assert uc.err(case.run_cut(t, [127, 1, 64, 2, 100]), want) < TOL
    # the attention is indeed peaked and far: some late row puts most of its weight on one key at least 100 back
    m = case.cfg["layers"][0]["mixer"]
    h = pv.embedding(case.cfg, case.weights, t)
    c, kr = pv.latent_kv(m, "l0.mix.", case.weights, h, 1e-6, True, False)
    cq = pv.rms(pv.lin(case.weights["l0.mix.dq"], h), 1e-6) * case.weights["l0.mix.dq.norm"].double()
    q = pv.lin(case.weights["l0.mix.uq"], cq).reshape(330, 2, 24)
    cos, sin = pv.rotary_table(m["rot"], torch.arange(330))
    s = (torch.einsum("thd,uhd->htu", q[..., :16], pv.lin(case.weights["l0.mix.uk"], c).reshape(330, 2, 16))
         + torch.einsum("thd,ud->htu", pv.rotate(q[..., 16:], cos, sin, 8, True), kr)) * m["scale"]
    p = torch.softmax(s.masked_fill(~torch.ones(330, 330, dtype=torch.bool).tril(), float("-inf")), -1)
    best, where = p[:, 200:].max(-1)
    far = (torch.arange(200, 330)[None] - where >= 100) & (best > 0.5)
    assert bool(far.any())


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    """Decays close to one: the first tokens still weigh in the state after hundreds of steps, so a state that is
    lost, reset or carried to the wrong slot shows far from where it happened."""
    case = cases("gla", memory=6.0)
    t = uc.tokens(260, case.vocab, 31)
    want = case.want(t)
    other = case.want([(t[0] + 1) % case.vocab] + t[1:])
    assert uc.err(other[-1], want[-1]) > 1e-3  # the first token still matters at the end
    assert uc.err(case.run_cut(t, [260]), want) < TOL
    assert uc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL


def test_long_decoding(cases):
    uc.long_decoding(cases("a"), TOL)


def test_the_token_before_a_step_is_the_sequences_own(cases):
    """The bigram row of a step's first token hashes the token that ended the sequence's step before, whatever
    other sequences ran in between and whichever slot they took."""
    case = cases("bigram")
    eng = case.eng
    a, b = uc.tokens(12, case.vocab, 1), uc.tokens(9, case.vocab, 2)
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, a[:5], [4]), StepEntry(sb, b[:1], [0])])
    assert uc.err(out[0], case.want(a)[4]) < TOL and uc.err(out[1], case.want(b)[0]) < TOL
    out = eng.step([StepEntry(sb, b[1:7], range(6))])
    assert uc.err(out, case.want(b)[1:7]) < TOL
    out = eng.step([StepEntry(sb, b[7:8], [0]), StepEntry(sa, a[5:6], [0])])  # the other order in the batch
    assert uc.err(out[0], case.want(b)[7]) < TOL and uc.err(out[1], case.want(a)[5]) < TOL
    eng.release(sa)
    sc = eng.new_sequence()  # takes the slot that a left: its first token must not see a's last
    out = eng.step([StepEntry(sc, a[:3], range(3))])
    assert sc == sa and uc.err(out, case.want(a)[:3]) < TOL
    eng.release(sb)
    eng.release(sc)
    case.assert_idle()


def test_greedy_generation_through_the_generation_loop(cases):
    case = cases("a")
    reqs, wants = uc.greedy(case)
    result = lq.generate(case.eng, reqs, max_new_tokens=10)
    assert result.tokens == wants
    case.assert_idle()


def test_bfloat16_run_rounds_where_the_plain_implementation_does(tmp_path_factory):
    case = uc.Case(tmp_path_factory.mktemp("vupelorn16"), "a", load, dtype="bfloat16", rounding=True)
    t = uc.tokens(80, case.vocab, 3)
    uc.assert_close_bf16(case.run_cut(t, [50, 2]), case.want(t), case.noise(t))
