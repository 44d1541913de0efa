"""Configurations, weights and the engine-beside-plain case for the Vupelorn tests, shared by the CPU tests (the
engine's own code over the torch stand-in for the kernels) and the GPU tests (the same over the HIP kernels).
Every comparison is against `plain_vupelorn`, run over whole sequences in float64.  The scenarios (cuttings,
batches, reuse of slots, long decoding, greedy tokens) are those of `vafodra_cases`, which ask nothing of a case
but its engine, its vocabulary and the plain logits."""
from __future__ import annotations

import copy
from typing import Dict, List

import torch

import longbow_quarrel_amd as lq
import plain_vupelorn as pv
from vafodra_cases import (err, greedy, long_decoding, portions, slots_and_blocks_used_again, tokens,  # noqa: F401
                           unequal_batches, whole_and_token_by_token, write_folder)
from longbow_quarrel_amd.engine import StepEntry


def _moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def _gla(heads, dim, vdim, tau, rank, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": rank}, "mlp": mlp}


def _latent(kind, heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, mlp=None, rot_dims=None, scaling=None,
            kv_from=None):
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling is not None:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "scale": scale, "rot": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": kind, "mixer": m, "mlp": mlp}


def _config(vocab, width, eps, layers, bigram=None):
    d = {"architecture": "Vupelorn", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if bigram is not None:
        d["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))}
    return d


_YARN = {"factor": 8.0, "original": 40, "fast": 16.0, "slow": 2.0}
# A: every kind of layer; YaRN whose blend lies inside the pairs; a layer without feed-forward; a layer that reads
# another's latent with other head counts and sizes of its own; all experts chosen in one layer, one in another;
# tau 1; a bigram table
CFG_A = _config(211, 96, 1e-6, [
    _latent("latent_attention", 3, 16, 16, 32, 48, 40, 0.2, 5000.0, _moe(5, 2, 24, 1.5), scaling=_YARN),
    _gla(2, 40, 24, 8.0, 6),
    _latent("latent_attention_2", 4, 32, 8, 16, 32, 24, 0.15, 10000.0, _moe(3, 1, 40, 3.0)),
    _latent("latent_attention_2", 2, 16, 8, 48, 32, 56, 0.3, 10000.0, _moe(4, 4, 16, 0.5), kv_from=2),
    _gla(3, 8, 8, 1.0, 2, _moe(2, 1, 32, 2.0)),
], bigram=(97, 13, 5))
# B: sizes that are multiples of nothing (the kernels' size-agnostic ways), no bigram table, a rotation of fewer
# entries than the rotated part holds, one head, a gated-linear-attention layer first and a shared latent two
# layers back
CFG_B = _config(131, 50, 1e-5, [
    _gla(1, 17, 9, 3.5, 3, _moe(2, 1, 9, 1.0)),
    _latent("latent_attention_2", 5, 10, 6, 7, 13, 11, 0.25, 300.0, None, rot_dims=4),
    _latent("latent_attention", 1, 24, 10, 12, 20, 18, 0.2, 1000.0, _moe(3, 2, 10, 2.5),
            scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
    _latent("latent_attention_2", 2, 6, 6, 10, 13, 9, 0.4, 300.0, None, rot_dims=4, kv_from=1),
], bigram=None)
# C: head sizes, ranks and widths of the kind that the fast kernels are made for
CFG_C = _config(1000, 256, 1e-5, [
    _latent("latent_attention", 4, 64, 32, 64, 96, 128, 0.1, 10000.0, _moe(4, 2, 128, 7.0),
            scaling={"factor": 4.0, "original": 128, "fast": 32.0, "slow": 1.0}),
    _gla(4, 64, 64, 16.0, 16, _moe(8, 2, 64, 7.0)),
    _latent("latent_attention_2", 8, 32, 16, 32, 48, 64, 0.14, 10000.0, _moe(4, 1, 128, 7.0)),
    _latent("latent_attention_2", 16, 16, 16, 16, 48, 64, 0.2, 10000.0, None, kv_from=2),
], bigram=(509, 3, 11))
# one mechanism a model: what fails here names its mechanism
CFG_GLA = _config(60, 48, 1e-6, [_gla(3, 16, 8, 4.0, 4)], bigram=None)
CFG_LATENT = _config(60, 48, 1e-6, [
    _latent("latent_attention", 2, 16, 8, 24, 16, 12, 0.25, 100.0, scaling={"factor": 3.0, "original": 20, "fast": 8.0, "slow": 1.0})])
CFG_LATENT2 = _config(60, 48, 1e-6, [
    _latent("latent_attention_2", 2, 16, 8, 24, 16, 12, 0.25, 100.0),
    _latent("latent_attention_2", 3, 8, 8, 16, 16, 20, 0.3, 100.0, kv_from=0)])
CFG_MOE = _config(60, 48, 1e-6, [_gla(1, 8, 8, 2.0, 2, _moe(6, 3, 20, 1.0))], bigram=None)
CFG_BIGRAM = _config(60, 48, 1e-6, [_gla(1, 8, 8, 2.0, 2)], bigram=(7, 1000003, 999983))
CONFIGS = {"a": CFG_A, "b": CFG_B, "c": CFG_C, "gla": CFG_GLA, "latent": CFG_LATENT, "latent2": CFG_LATENT2,
           "moe": CFG_MOE, "bigram": CFG_BIGRAM}


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: sizes, head counts, ranks, the order of the layers, which layers lend
    their latent, experts and constants all vary; some sizes are multiples of 16, some of nothing."""
    import random

    rng = random.Random(seed)
    even = lambda lo, hi: 2 * rng.randint(lo // 2, hi // 2)
    width = rng.choice([40, 56, 64, 72, 100, 128, 136])
    layers, latents = [], {}  # latents: layer index -> (kind, kv_rank, rot_dim, rot)
    for i in range(rng.randint(2, 6)):
        mlp = None if rng.random() < 0.2 else _moe(rng.randint(2, 6), 1, rng.choice([8, 12, 20, 32]), rng.choice([0.5, 2.0, 7.0]))
        if mlp is not None:
            mlp["router"]["top"] = rng.randint(1, mlp["router"]["experts"])
        kind = rng.choice(["gla", "latent_attention", "latent_attention_2", "latent_attention_2"])
        if kind == "gla":
            layers.append(_gla(rng.randint(1, 4), rng.choice([8, 12, 16, 24, 40]), rng.choice([8, 12, 16, 36]),
                               rng.choice([1.0, 4.0, 16.0]), rng.randint(1, 8), mlp))
            continue
        lend = [j for j, v in latents.items() if v[0] == kind]
        if kind == "latent_attention_2" and lend and rng.random() < 0.5:
            j = rng.choice(lend)
            _, kv_rank, rot_dim, rot = latents[j]
            layer = _latent(kind, rng.randint(1, 5), rng.choice([8, 16, 20]), rot_dim, rng.choice([8, 16, 28]), kv_rank,
                            rng.choice([12, 16, 40]), rng.choice([0.1, 0.25]), rot["base"], mlp, kv_from=j)
        else:
            rot_dim = even(2, 24) if rng.random() < 0.5 else rng.choice([8, 16, 32])
            scaling = None
            if kind == "latent_attention":
                scaling = {"factor": rng.choice([2.0, 4.0, 8.0]), "original": rng.choice([16, 64, 2048]),
                           "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
            layer = _latent(kind, rng.randint(1, 5), rng.choice([8, 16, 20, 32]), rot_dim, rng.choice([8, 16, 28]),
                            rng.choice([8, 16, 24, 40, 48]), rng.choice([12, 16, 40]), rng.choice([0.1, 0.25]),
                            rng.choice([100.0, 10000.0, 250000.0]), mlp, scaling=scaling)
            latents[i] = (kind, layer["mixer"]["kv_rank"], rot_dim, layer["mixer"]["rot"])
        layers.append(layer)
    bigram = None if rng.random() < 0.3 else (rng.randint(3, 300), rng.randint(1, 99), rng.randint(1, 99))
    return _config(rng.randint(30, 300), width, rng.choice([1e-6, 1e-5]), layers, bigram)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0, memory: float = 0.0) -> Dict[str, torch.Tensor]:
    """Random weights whose values bfloat16 holds exactly (both run dtypes then see the same model), with spreads
    that make every constant matter.  `sharp` scales the queries' and the latents' projections so that attention
    is peaked (a far key can then carry a row's result); `memory` is added to the decays' biases, so that a gated
    linear attention state forgets slowly and old tokens stay in it."""
    config = lq.VupelornConfig.from_dict(cfg)
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import spec_from_config

    g = torch.Generator().manual_seed(seed)
    out = {}
    for s in DecoderModel(spec_from_config(config)).tensor_specs():
        if s.optional:  # (the norm of a feed-forward that is not there)
            continue
        n, shape = s.name, tuple(s.shape)
        leaf = n.split(".")[-1]
        normal = lambda std, mean=0.0: torch.empty(shape).normal_(mean, std, generator=g)
        if n in ("embed", "bigram"):
            t = normal(0.5)
        elif leaf in ("norm", "norm1", "norm2") or n == "final.norm":
            t = normal(0.3, 1.0)
        elif n.endswith("a2.b"):
            t = normal(1.0, 1.0 + memory)
        elif leaf == "router":  # (scores well inside (0, 1): two that both round to 1 in 32-bit would be a tie there)
            t = normal(0.5 / (shape[-1] ** 0.5))
        else:
            t = normal(1.0 / (shape[-1] ** 0.5))
            if leaf in ("uq", "dkv"):
                t = t * sharp
        out[n] = t.to(torch.bfloat16).float()
    return out


def assert_close_bf16(got: torch.Tensor, want: torch.Tensor, noise: float, most: float = 0.25) -> None:
    """A bfloat16 run against the plain implementation that rounds where such a run does.  Rounding moves a
    router's score by a few thousandths, so now and then a token's close call between two experts falls the other
    way; that row then differs by much more than rounding, and so, less, do the rows after it, which read it
    through the recurrent states and the cached latents.  (Measured on these configurations over 150 tokens: the
    plain implementation with against without rounding has a median row error of 0.003 to 0.022 and single rows up
    to 0.42; the engine over the torch stand-in and over the HIP kernels differ from it alike, median 0.018, single
    rows up to 0.75.)  So the rows' typical error is held against three times what rounding alone does to the
    plain implementation on the same tokens (`noise`, from `Case.noise`), and the share of rows beyond a larger
    limit is bounded, not the worst row; the sharp comparisons are the float32 ones, through the same kernels'
    32-bit forms."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape
    rows = (got - want).abs().max(-1).values / want.abs().max()
    assert float(rows.median()) < 3 * noise, (float(rows.median()), noise)
    assert float((rows > most).double().mean()) <= 0.1, sorted(rows.tolist())[-8:]


class Case:
    """An engine (made by `load`, which the CPU and the GPU tests bring) beside the plain implementation."""

    def __init__(self, tmp_path, name: str, load, dtype: str = "float32", seed: int = 3, sharp: float = 1.0,
                 memory: float = 0.0, max_tokens: int = 2048, rounding: bool = False) -> None:
        self.cfg = copy.deepcopy(CONFIGS[name] if isinstance(name, str) else random_config(name))
        self.weights = make_weights(self.cfg, seed, sharp, memory)
        self.folder = write_folder(tmp_path, self.cfg, self.weights, f"{name}_{seed}_{sharp}_{memory}")
        self.eng = load(self.folder, dtype, max_tokens)
        self.vocab = self.cfg["vocab"]
        self.rounding = rounding
        self._want = {}

    def want(self, toks: List[int]) -> torch.Tensor:
        key = tuple(toks)
        if key not in self._want:
            self._want[key] = pv.forward(self.cfg, self.weights, toks, rounding=self.rounding)
        return self._want[key]

    def noise(self, toks: List[int]) -> float:
        """What rounding alone does on these tokens: the median over the rows of the largest difference (over the
        largest logit) between the plain implementation with and without rounding."""
        a = pv.forward(self.cfg, self.weights, toks, rounding=True)
        b = pv.forward(self.cfg, self.weights, toks, rounding=False)
        return float(((a - b).abs().max(-1).values / b.abs().max()).median())

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

    def layers(self, toks: List[int]):
        """The residual stream after every layer, from the engine's observer and from the plain implementation."""
        got = []
        s = self.eng.new_sequence()
        self.eng.step([StepEntry(s, toks, [])],
                      observe=lambda name, x, pending: got.append(x.float().cpu().clone()) if name != "embed" else None)
        self.eng.release(s)
        want = []
        pv.forward(self.cfg, self.weights, toks, rounding=self.rounding, layers_out=want)
        return got, want

    def assert_idle(self) -> None:
        c = self.eng.cache
        assert c.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in c.kv_groups)
