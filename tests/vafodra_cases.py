"""Configurations, weights and scenarios for the Vafodra tests, shared by the CPU tests (the engine's own code
over the torch stand-in for the kernels) and the GPU tests (the same over the HIP kernels).  Every comparison
is against `plain_vafodra`, run over whole sequences in float64."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import torch

import longbow_quarrel_amd as lq
import plain_vafodra as pv
from longbow_quarrel_amd.engine import StepEntry


def _parallel(left, right, ff, weights_of=None):
    d = {"type": "parallel", "mixer": {"left": left, "right": right},
         "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def _delta(mixer, ff, weights_of=None):
    d = {"type": "delta", "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def _config(vocab, width, scale, eps, mult, layers):
    return {"architecture": "Vafodra", "embedding": {"scale": scale}, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "vocab": vocab, "width": width}


# A: a short window that keeps two tokens, keys wider than values, a layer run twice, a layer without feed-forward
_A_LEFT = {"dim": 32, "vdim": 16, "heads": 4, "kv_heads": 2, "mask": {"size": 7, "keep_first": 2}, "scale": 0.2}
_A_RIGHT = {"conv": 3, "groups": 1, "heads": 4, "norm_groups": 4, "state": 24, "vdim": 16}
CFG_A = _config(200, 96, 2.0, 1e-6, 0.5, [
    _parallel(_A_LEFT, _A_RIGHT, 160),
    _delta({"conv": 2, "dim": 16, "heads": 4, "kv_heads": 2, "vdim": 32}, None),
    _parallel(_A_LEFT, _A_RIGHT, 160, weights_of=0),
    _delta({"conv": 4, "dim": 48, "heads": 2, "kv_heads": 2, "vdim": 16}, 64),
])
# B: sizes that are multiples of nothing much (the kernels' size-agnostic ways), no kept tokens, a window longer
# than a cache block, every head its own key/value head and group, one norm group, a delta layer first
_B_DELTA = {"conv": 3, "dim": 24, "heads": 2, "kv_heads": 1, "vdim": 40}
CFG_B = _config(131, 72, 0.7, 1e-5, 1.0, [
    _delta(_B_DELTA, 100),
    _parallel({"dim": 24, "vdim": 40, "heads": 3, "kv_heads": 3, "mask": {"size": 70, "keep_first": 0}, "scale": 0.3},
              {"conv": 2, "groups": 3, "heads": 3, "norm_groups": 1, "state": 20, "vdim": 24}, None),
    _delta(_B_DELTA, 100, weights_of=0),
])
# C: window and kept tokens that both pass a block's edge, a large state, values wider than keys
CFG_C = _config(97, 64, 1.5, 1e-5, 0.25, [
    _parallel({"dim": 16, "vdim": 32, "heads": 2, "kv_heads": 1, "mask": {"size": 66, "keep_first": 65}, "scale": 0.25},
              {"conv": 4, "groups": 2, "heads": 2, "norm_groups": 2, "state": 130, "vdim": 64}, 96),
    _parallel({"dim": 48, "vdim": 48, "heads": 1, "kv_heads": 1, "mask": {"size": 1, "keep_first": 1}, "scale": 1.0},
              {"conv": 1, "groups": 1, "heads": 1, "norm_groups": 8, "state": 16, "vdim": 64}, 32),
])
# D: nothing is a multiple of 8 (every product and every kernel takes its size-agnostic way), five taps, three
# norm groups of 20, a state of 9
CFG_D = _config(77, 100, 1.0, 1e-4, 0.8, [
    _parallel({"dim": 20, "vdim": 12, "heads": 5, "kv_heads": 5, "mask": {"size": 3, "keep_first": 5}, "scale": 0.4},
              {"conv": 5, "groups": 5, "heads": 5, "norm_groups": 3, "state": 9, "vdim": 12}, 50),
    _delta({"conv": 2, "dim": 12, "heads": 3, "kv_heads": 3, "vdim": 20}, 52),
])
# E: head sizes, state and width of the kind that the fast kernels are made for
CFG_E = _config(1000, 512, 1.0, 1e-5, 0.5, [
    _parallel({"dim": 128, "vdim": 128, "heads": 4, "kv_heads": 1, "mask": {"size": 100, "keep_first": 3}, "scale": 0.09},
              {"conv": 4, "groups": 2, "heads": 8, "norm_groups": 2, "state": 128, "vdim": 64}, 1792),
    _delta({"conv": 4, "dim": 128, "heads": 4, "kv_heads": 2, "vdim": 128}, 1792),
    _parallel({"dim": 64, "vdim": 256, "heads": 2, "kv_heads": 2, "mask": {"size": 200, "keep_first": 0}, "scale": 0.125},
              {"conv": 4, "groups": 1, "heads": 16, "norm_groups": 1, "state": 64, "vdim": 32}, None),
])
# F: delta layers alone (no keys and values anywhere in the cache), the later layer lending its tensors to the earlier
CFG_F = _config(50, 48, 1.2, 1e-5, 0.6, [
    _delta({"conv": 3, "dim": 8, "heads": 6, "kv_heads": 2, "vdim": 8}, 24, weights_of=1),
    _delta({"conv": 3, "dim": 8, "heads": 6, "kv_heads": 2, "vdim": 8}, 24),
])
CONFIGS = {"a": CFG_A, "b": CFG_B, "c": CFG_C, "d": CFG_D, "e": CFG_E, "f": CFG_F}


def make_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, torch.Tensor]:
    """Random weights whose values bfloat16 holds exactly (both run dtypes then see the same model), with
    spreads that make every constant matter; `sharp` scales the attention's q and k so that it is peaked."""
    config = lq.VafodraConfig.from_dict(cfg)
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import spec_from_config

    g = torch.Generator().manual_seed(seed)
    out = {}
    for s in DecoderModel(spec_from_config(config)).tensor_specs():
        n, shape = s.name, tuple(s.shape)
        leaf = n.split(".")[-1]
        normal = lambda std, mean=0.0: torch.empty(shape).normal_(mean, std, generator=g)
        uniform = lambda lo, hi: torch.empty(shape).uniform_(lo, hi, generator=g)
        if n == "embed":
            t = normal(0.5)
        elif leaf == "alpha":
            t = normal(0.15, 0.7)
        elif n.endswith("norm1") or n.endswith("final.norm") or leaf in ("norm", "out", "D"):
            t = normal(0.3, 1.0)
        elif n.endswith("conv.b") or (leaf == "b" and len(shape) == 1):
            t = normal(0.2)
        elif leaf == "conv":
            t = normal(0.4)
        elif leaf == "dt_bias":
            t = uniform(-2.0, 0.5)
        elif leaf == "A_log":
            t = uniform(-1.5, 0.5)
        else:
            t = normal(1.0 / (shape[-1] ** 0.5))
            if ".left." in n and leaf in ("q", "k"):
                t = t * sharp
        out[n] = t.to(torch.bfloat16).float()
    return out


def write_folder(tmp_path, cfg: dict, weights: Dict[str, torch.Tensor], name: str) -> str:
    from safetensors.torch import save_file

    folder = os.path.join(str(tmp_path), name)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({n: t.to(torch.bfloat16).contiguous() for n, t in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def tokens(n: int, vocab: int, seed: int) -> List[int]:
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, (got.shape, want.shape)
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


class Case:
    """An engine (made by `load`, which the CPU and the GPU tests bring) beside the plain implementation."""

    def __init__(self, tmp_path, name: str, load, dtype: str = "float32", seed: int = 3, sharp: float = 1.0,
                 max_tokens: int = 2048) -> None:
        self.cfg = copy.deepcopy(CONFIGS[name])
        self.weights = make_weights(self.cfg, seed, sharp)
        self.folder = write_folder(tmp_path, self.cfg, self.weights, f"{name}_{seed}_{sharp}")
        self.eng = load(self.folder, dtype, max_tokens)
        self.vocab = self.cfg["vocab"]
        self._want = {}

    def want(self, toks: List[int]) -> torch.Tensor:
        key = tuple(toks)
        if key not in self._want:
            self._want[key] = pv.forward(self.cfg, self.weights, toks)
        return self._want[key]

    def run_cut(self, toks: List[int], cuts: List[int]) -> torch.Tensor:
        """The sequence in portions of the sizes `cuts` (the rest token by token), all logits."""
        eng = self.eng
        s = eng.new_sequence()
        got, at = [], 0
        sizes = list(cuts)
        while at < len(toks):
            n = min(sizes.pop(0) if sizes else 1, len(toks) - at)
            got.append(eng.step([StepEntry(s, toks[at : at + n], range(n))]).clone())
            at += n
        eng.release(s)
        return torch.cat(got)

    def assert_idle(self) -> None:
        c = self.eng.cache
        assert c.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in c.kv_groups)


def whole_and_token_by_token(case: Case, tol: float, lengths=(1, 2, 3, 9, 70, 131)) -> None:
    for i, n in enumerate(lengths):
        t = tokens(n, case.vocab, 10 + i)
        assert err(case.run_cut(t, [n]), case.want(t)) < tol, f"whole, {n} tokens"
    t = tokens(75, case.vocab, 99)
    assert err(case.run_cut(t, []), case.want(t)) < tol, "token by token from the first"
    case.assert_idle()


def portions(case: Case, tol: float, n: int = 150) -> None:
    t = tokens(n, case.vocab, 5)
    for cuts in ([2] * 40, [64, 1, 63, 2, 3], [63, 2, 64], [5, 17, 1, 1, 40], [1, 128], [3, 61, 66]):
        assert err(case.run_cut(t, cuts), case.want(t)) < tol, f"portions {cuts[:6]}"
    case.assert_idle()


def unequal_batches(case: Case, tol: float) -> None:
    """Requests of unequal lengths start together, decode together, the shorter end earlier; then another
    batch takes over their slots and blocks."""
    eng = case.eng
    for round_, lengths in enumerate(((90, 3, 140, 1, 66), (5, 129, 64), (70, 2))):
        reqs = [tokens(n, case.vocab, 1000 * round_ + n) for n in lengths]
        split = [max(1, n - 4 - 2 * i) for i, n in enumerate(lengths)]
        slots = [eng.new_sequence() for _ in reqs]
        out = eng.step([StepEntry(s, r[:k], range(k)) for s, r, k in zip(slots, reqs, split)])
        at = 0
        for r, k in zip(reqs, split):
            assert err(out[at : at + k], case.want(r)[:k]) < tol
            at += k
        pos = list(split)
        for i, r in enumerate(reqs):
            if pos[i] == len(r):
                eng.release(slots[i])
        while any(pos[i] < len(r) for i, r in enumerate(reqs)):
            live = [i for i, r in enumerate(reqs) if pos[i] < len(r)]
            out = eng.step([StepEntry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                assert err(out[j], case.want(reqs[i])[pos[i]]) < tol, f"batch {lengths}, request {i}, position {pos[i]}"
                pos[i] += 1
                if pos[i] == len(reqs[i]):
                    eng.release(slots[i])
    case.assert_idle()


def slots_and_blocks_used_again(case: Case, tol: float) -> None:
    """A slot whose sequence ended holds that sequence's state and blocks until the next one takes them: the
    next one must start from zero and must not see the old keys."""
    eng = case.eng
    a, b, c = tokens(140, case.vocab, 1), tokens(9, case.vocab, 2), tokens(100, case.vocab, 3)
    sa = eng.new_sequence()
    eng.step([StepEntry(sa, a, [])])
    sb = eng.new_sequence()
    eng.step([StepEntry(sb, b, [])])
    eng.release(sa)
    sc = eng.new_sequence()
    assert sc == sa  # the lowest free slot comes first
    out = eng.step([StepEntry(sc, c[:70], range(70)), StepEntry(sb, [b[0]], [])])
    assert err(out, case.want(c)[:70]) < tol
    out = eng.step([StepEntry(sc, c[70:], range(30))])
    assert err(out, case.want(c)[70:]) < tol
    eng.release(sb)
    eng.release(sc)
    case.assert_idle()


def long_decoding(case: Case, tol: float, prompt: int = 6, steps: int = 200) -> None:
    t = tokens(prompt + steps, case.vocab, 77)
    assert err(case.run_cut(t, [prompt]), case.want(t)) < tol
    case.assert_idle()


def greedy(case: Case, n_prompt: int = 6, n_new: int = 10, prompts: int = 3):
    """Greedy tokens of the plain implementation for a few prompts (a margin between the best two logits is
    asserted, so that rounding cannot change the choice)."""
    reqs, wants = [], []
    for i in range(prompts):
        t = tokens(n_prompt + 3 * i, case.vocab, 500 + i)
        new = []
        for _ in range(n_new):
            top = torch.topk(case.want(t + new)[-1], 2).values
            assert float(top[0] - top[1]) > 1e-4 * float(top[0].abs())
            new.append(int(case.want(t + new)[-1].argmax()))
        reqs.append(t)
        wants.append(new)
    return reqs, wants
