"""The Vafodra design through the engine's own code (registry, loader, cache groups, step function, generation
loop) on the CPU, over the torch stand-in for the kernels, against the plain implementation.  The GPU tests
repeat every scenario with the HIP kernels; these catch faults of the parts, the cache and the batching."""
import copy

import pytest
import torch

import longbow_quarrel_amd as lq
import vafodra_cases as vc
from cpu_kernels import CpuKernels
from longbow_quarrel_amd.cache import BLOCK_SIZE, CacheManager
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.parts.base import KVNeed, MultiNeed, StateNeed

TOL = 2e-5


def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=CpuKernels(),
                          max_slots=8, max_sequence_tokens=max_tokens)


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, sharp=1.0):
        if (name, sharp) not in made:
            made[(name, sharp)] = vc.Case(tmp_path_factory.mktemp("vafodra"), name, load, sharp=sharp)
        return made[(name, sharp)]

    return get


def test_configuration_reads_every_size_and_writes_the_same_keys_back():
    for cfg in vc.CONFIGS.values():
        assert lq.VafodraConfig.from_dict(cfg).to_dict() == cfg
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import config_from_dict, spec_from_config

    model = DecoderModel(spec_from_config(config_from_dict(vc.CFG_A)))
    # four layers, three with tensors of their own: the third runs layer 0's block again with its own cache
    assert [r.layer for r in model.spec.schedule] == [0, 1, 0, 2] and len(model.blocks) == 3
    names = {s.name for s in model.tensor_specs()}
    assert "l0.mix.left.g" in names and "l1.mix.q.conv" in names and "l3.mix.dt_bias" in names
    assert not any(n.startswith("l2.") for n in names) and "l1.mlp.gate" not in names
    needs = model.cache_needs()
    assert len(needs) == 4 and needs[0] == needs[2] and needs[1] != needs[3]
    assert needs[0].needs[0] == KVNeed(2, 32, 7, 16, 2)


@pytest.mark.parametrize("key,value,text", [
    (("layers", 0, "type"), "other", "layers[0].type"),
    (("layers", 0, "mixer", "left", "mask", "size"), None, "layers[0].mixer.left.mask.size"),
    (("layers", 0, "mixer", "right", "norm_groups"), 5, "norm_groups"),
    (("layers", 1, "mixer", "kv_heads"), 3, "layers[1].mixer.heads"),
    (("layers", 2, "weights_of"), 2, "weights_of"),
    (("layers", 2, "weights_of"), 1, "differs"),
    (("layers", 3, "mlp", "kind"), "routed", "mlp.kind"),
    (("norm", "eps"), "tiny", "norm.eps"),
    (("vocab",), None, "vocab"),
])
def test_configuration_errors_name_their_key(key, value, text):
    cfg = copy.deepcopy(vc.CFG_A)
    d = cfg
    for k in key[:-1]:
        d = d[k]
    d[key[-1]] = value
    with pytest.raises(lq.ConfigError) as e:
        lq.VafodraConfig.from_dict(cfg)
    assert text in str(e.value)


def test_keys_that_a_configuration_leaves_out_mean_that_the_model_has_no_such_thing():
    cfg = copy.deepcopy(vc.CFG_A)
    left, right = cfg["layers"][0]["mixer"]["left"], cfg["layers"][0]["mixer"]["right"]
    del left["mask"]["keep_first"], left["kv_heads"], right["groups"], right["norm_groups"], cfg["layers"][1]["mlp"]
    cfg["layers"][2] = copy.deepcopy(cfg["layers"][0])
    cfg["layers"][2]["weights_of"] = 0
    c = lq.VafodraConfig.from_dict(cfg)
    assert c.layers[0].left.keep_first == 0 and c.layers[0].left.kv_heads == 4
    assert c.layers[0].right.groups == 1 and c.layers[0].right.norm_groups == 1 and c.layers[1].ff is None


def test_generation_with_delta_layers_alone(cases):
    case = cases("f")
    reqs, wants = vc.greedy(case, n_new=5, prompts=2)
    res = lq.generate(case.eng, reqs, max_new_tokens=5, max_batch=2, stop_ids=[], use_graphs=False)
    assert res.tokens == wants


def test_weight_errors_list_missing_and_wrongly_shaped_tensors(tmp_path):
    w = vc.make_weights(vc.CFG_B, 1)
    del w["l1.mix.left.out"]
    w["l0.mix.A_log"] = torch.zeros(5)
    w["l2.norm1"] = torch.zeros(72)  # layer 2 runs with layer 0's tensors and has none
    folder = vc.write_folder(tmp_path, vc.CFG_B, w, "broken")
    with pytest.raises(lq.WeightError) as e:
        load(folder, "float32", 256)
    assert e.value.missing == ["l1.mix.left.out"] and e.value.unexpected == ["l2.norm1"]
    assert len(e.value.wrong_shape) == 1 and "l0.mix.A_log" in e.value.wrong_shape[0]


def test_a_window_that_keeps_first_tokens_gives_the_blocks_between_back():
    need = MultiNeed((KVNeed(1, 8, window=10, value_dim=4, keep_first=3), StateNeed((2, 3))))
    cm = CacheManager({0: need, 1: need, 2: KVNeed(1, 8, window=10)}, max_tokens=64 * 6, max_slots=2,
                      dtype=torch.float32, device=torch.device("cpu"))
    kept, plain_window = cm.kv_groups
    assert tuple(kept.v.shape[1:]) == (6, 1, 4, BLOCK_SIZE) and tuple(kept.k.shape[1:]) == (6, 1, BLOCK_SIZE, 8)
    s = cm.acquire()
    cm.reserve({s: 300})
    cm.advance({s: 300})
    assert [b is not None for b in kept.owned[s]] == [True, False, False, False, True]
    assert [b is not None for b in plain_window.owned[s]] == [False, False, False, False, True]
    view = cm.layer_views()[1]
    assert view.parts[0].k.shape[0] == 6 and tuple(view.parts[1].state.shape) == (2, 2, 3)
    view.parts[1].state[s] += 1.0
    cm.release(s)
    assert cm.acquire() == s and float(cm.layer_views()[1].parts[1].state[s].abs().sum()) == 0.0
    assert kept.blocks.taken_count == 0 and cm.free_blocks() == 6


@pytest.mark.parametrize("name", ["a", "b", "c", "d", "f"])
def test_whole_prompts_and_token_by_token(cases, name):
    vc.whole_and_token_by_token(cases(name), TOL, lengths=(1, 2, 3, 70))


@pytest.mark.parametrize("name", ["a", "c"])
def test_portions_down_to_two_tokens(cases, name):
    vc.portions(cases(name), TOL, n=140)


@pytest.mark.parametrize("name", ["a", "b"])
def test_unequal_batches_against_each_request_alone(cases, name):
    vc.unequal_batches(cases(name), TOL)


def test_slots_and_blocks_that_are_used_again(cases):
    vc.slots_and_blocks_used_again(cases("a"), TOL)
    vc.slots_and_blocks_used_again(cases("c"), TOL)


def test_peaked_attention_shows_every_edge_of_window_and_kept_tokens(cases):
    """q and k scaled up: one key carries most of a row's weight, so a key read one place off, a kept token
    dropped or a sink left out moves the logits by far more than the tolerance."""
    case = cases("a", sharp=8.0)
    t = vc.tokens(90, case.vocab, 4)
    base = case.want(t)
    assert vc.err(case.run_cut(t, [60]), base) < TOL
    import plain_vafodra as pv
    for change in ({"size": 6}, {"size": 8}, {"keep_first": 1}, {"keep_first": 3}):
        other = copy.deepcopy(case.cfg)
        other["layers"][0]["mixer"]["left"]["mask"].update(change)
        assert vc.err(pv.forward(other, case.weights, t), base) > 100 * TOL, change


def test_long_decoding(cases):
    vc.long_decoding(cases("b"), TOL, steps=150)


def test_greedy_generation_through_the_entry_point_and_the_generation_loop(cases):
    case = cases("a")
    reqs, wants = vc.greedy(case, n_new=6, prompts=3)
    res = lq.generate(case.eng, reqs, max_new_tokens=6, max_batch=2, stop_ids=[], use_graphs=False)
    assert res.tokens == wants
    case.assert_idle()
