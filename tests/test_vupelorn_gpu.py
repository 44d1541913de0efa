"""The Vupelorn design on the GPU.  First every new kernel alone against the plain implementation's function of
the same mechanism (float64), with inputs made so that a fault shows; then the engine in float32 and in bfloat16
under every cutting and batching; then generation through the entry point, with captured steps and direct ones,
the command line and the trace replay."""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import longbow_quarrel_amd as lq
import plain_vupelorn as pv
import vupelorn_cases as uc
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


# ---- kernels alone -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("sizes", [(2, 16, 8, 4.0), (3, 40, 24, 16.0), (1, 17, 9, 1.0), (2, 64, 64, 8.0), (1, 130, 70, 2.0),
                                   (4, 128, 128, 16.0), (1, 600, 16, 3.0)])
def test_gated_linear_attention_scan_in_portions(kn, sizes):
    """Two sequences in unequal portions, states in slots that are not in order; the decays near one in some
    channels and near zero in others, so that both a lost state and a wrong channel show."""
    H, dk, dv, tau = sizes
    lengths, slots = (45, 19), (3, 1)
    g = torch.Generator().manual_seed(dk)
    seqs = []
    for n in lengths:
        q, k, v = (torch.empty(n, H * d).normal_(0, 1, generator=g) for d in (dk, dk, dv))
        z = torch.empty(n, H * dk).normal_(0, 3, generator=g)
        seqs.append((q, k, v, z))
    bias = torch.empty(H * dk).normal_(2, 3, generator=g)

    def plain(q, k, v, z):
        n = q.shape[0]
        a = torch.sigmoid(z.double() + bias.double()).pow(1 / tau).reshape(n, H, dk)
        S, out = torch.zeros(H, dk, dv, dtype=F), torch.zeros(n, H, dv, dtype=F)
        for t in range(n):
            S = a[t][:, :, None] * S + k[t].double().reshape(H, dk)[:, :, None] * v[t].double().reshape(H, dv)[:, None, :]
            out[t] = torch.einsum("hkv,hk->hv", S, q[t].double().reshape(H, dk) * dk ** -0.5)
        return out.reshape(n, H * dv), S

    state = torch.full((5, H, dv, dk), 7.0, device=DEV)
    state[list(slots)] = 0
    got = [[], []]
    at = [0, 0]
    for portion in ((17, 1), (1, 1), (20, 16), (7, 1)):
        rows = [seqs[b][0][at[b] : at[b] + n].shape[0] for b, n in enumerate(portion)]
        cat = [dev(torch.cat([seqs[b][j][at[b] : at[b] + portion[b]] for b in range(2)])) for j in range(4)]
        out = torch.zeros(sum(rows), H * dv, device=DEV)
        kn.gla_scan(*cat, dev(bias), state, out, H, dk, dv, dk ** -0.5, 1 / tau, i32(slots), i32([0, rows[0], sum(rows)]), 2)
        got[0].append(out[: rows[0]].cpu())
        got[1].append(out[rows[0] :].cpu())
        at = [a + n for a, n in zip(at, portion)]
    for b in range(2):
        want, S = plain(*seqs[b])
        assert uc.err(torch.cat(got[b]), want) < TOL_F32, f"sequence {b}"
        assert uc.err(state[slots[b]].cpu(), S.transpose(1, 2)) < TOL_F32  # held [head, value, key]
    assert bool((state[[0, 2, 4]] == 7.0).all())  # nobody else's state was touched


@pytest.mark.parametrize("sizes", [(2, 32, 24, 4.0), (1, 128, 256, 16.0), (3, 17, 9, 2.0)])
def test_gated_linear_attention_scan_of_a_long_prompt_in_segments(kn, sizes):
    """A long prompt beside a short one: the launch cuts the long one into segments that run side by side (from zero,
    end states chained with the products of the decays, again from the true starts); the state it leaves is the
    one that a token-by-token walk leaves, and a single token goes on from it."""
    H, dk, dv, tau = sizes
    n_long, n_short = 701, 30
    g = torch.Generator().manual_seed(dk)
    q, k, v = (torch.empty(n_long + n_short + 2, H * d).normal_(0, 1, generator=g) for d in (dk, dk, dv))
    z = torch.empty(n_long + n_short + 2, H * dk).normal_(1, 2, generator=g)
    bias = torch.empty(H * dk).normal_(2, 2, generator=g)
    start = torch.empty(4, H, dv, dk).normal_(0, 1, generator=g)  # the sequences do not start from nothing

    def plain(rows, S):
        S = S.double().transpose(1, 2).clone()  # [head, key, value]
        outs = []
        for r in rows:
            a = torch.sigmoid(z[r].double() + bias.double()).pow(1 / tau).reshape(H, dk)
            S = a[:, :, None] * S + k[r].double().reshape(H, dk)[:, :, None] * v[r].double().reshape(H, dv)[:, None, :]
            outs.append(torch.einsum("hkv,hk->hv", S, q[r].double().reshape(H, dk) * dk ** -0.5).reshape(-1))
        return torch.stack(outs), S.transpose(1, 2)

    need = kn.gla_scan_workspace(2, H, dk, dv, n_long)
    assert need > 0
    state = start.clone().to(DEV)
    rows = n_long + n_short
    out = torch.zeros(rows, H * dv, device=DEV)
    kn.gla_scan(dev(q[:rows]), dev(k[:rows]), dev(v[:rows]), dev(z[:rows]), dev(bias), state, out, H, dk, dv, dk ** -0.5,
                1 / tau, i32([2, 0]), i32([0, n_long, rows]), 2, max_rows=n_long,
                workspace=torch.zeros(need, device=DEV))
    want_long, s_long = plain(range(n_long), start[2])
    want_short, s_short = plain(range(n_long, rows), start[0])
    assert uc.err(out[:n_long].cpu(), want_long) < TOL_F32 and uc.err(out[n_long:].cpu(), want_short) < TOL_F32
    assert uc.err(state[2].cpu(), s_long) < TOL_F32 and uc.err(state[0].cpu(), s_short) < TOL_F32
    assert torch.equal(state[[1, 3]].cpu(), start[[1, 3]])
    one = torch.zeros(2, H * dv, device=DEV)
    kn.gla_scan(dev(q[rows:]), dev(k[rows:]), dev(v[rows:]), dev(z[rows:]), dev(bias), state, one, H, dk, dv, dk ** -0.5,
                1 / tau, i32([2, 0]), i32([0, 1, 2]), 2)
    assert uc.err(one[0].cpu(), plain([rows], s_long)[0][0]) < TOL_F32
    assert uc.err(one[1].cpu(), plain([rows + 1], s_short)[0][0]) < TOL_F32


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_over_columns_rotation_and_the_norm_of_a_result(kn, dtype):
    rows, n = 9, 52
    wide = rnd(rows, 80, seed=1)
    w = rnd(n, seed=2) + 1
    out = torch.zeros(rows, 64, dtype=dtype, device=DEV)
    kn.rmsnorm_cols(dev(wide)[:, 12 : 12 + n], dev(w), 1e-5, out[:, 4 : 4 + n])
    want = pv.rms(wide[:, 12 : 12 + n].double(), 1e-5) * w.double()
    tol = TOL_F32 if dtype == torch.float32 else 5e-3
    assert uc.err(out[:, 4 : 4 + n].float().cpu(), want) < tol and bool((out[:, :4] == 0).all()) and bool((out[:, 56:] == 0).all())
    # rotation: both pairings, fewer rotated entries than the vector holds, positions far out, a magnitude, and
    # every head's vector landing in a run of columns of a wider row
    heads, size, dims, stride = 3, 10, 6, 17
    src = rnd(rows, heads * size, seed=3)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 1000, 70000, 5])
    rot = {"base": 50.0, "dims": dims, "scaling": {"factor": 4.0, "original": 30, "fast": 4.0, "slow": 1.0}}
    cos, sin = pv.rotary_table(rot, pos)
    from longbow_quarrel_amd.parts.rope import rotary_frequencies, rotary_magnitude
    sc = {"rope_type": "yarn", **rot["scaling"]}
    freqs = torch.tensor(rotary_frequencies(dims, 50.0, sc), dtype=torch.float64, device=DEV)
    for inter in (False, True):
        out = torch.zeros(rows, 60, dtype=dtype, device=DEV)
        kn.rotary(dev(src), out[:, 5:], heads, size, stride, dims, inter, freqs, rotary_magnitude(sc), i32(pos.tolist()))
        want = pv.rotate(src.double().reshape(rows, heads, size), cos, sin, dims, inter)
        for h in range(heads):
            assert uc.err(out[:, 5 + h * stride : 5 + h * stride + size].float().cpu(), want[:, h]) < (2e-5 if dtype == torch.float32 else 5e-3)
        assert bool((out[:, :5] == 0).all()) and bool((out[:, 5 + size : 5 + stride] == 0).all())
    # x += norm(y) w, and x in the run's dtype beside it
    x, y, g = rnd(rows, 100, seed=4), rnd(rows, 100, seed=5, std=30.0), rnd(100, seed=6) + 1
    xd, rounded = dev(x), torch.zeros(rows, 100, dtype=dtype, device=DEV)
    kn.rmsnorm_residual(xd, dev(y), dev(g), 1e-6, rounded)
    want = x.double() + pv.rms(y.double(), 1e-6) * g.double()
    assert uc.err(xd.cpu(), want) < TOL_F32 and uc.err(rounded.float().cpu(), want) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(21, 5, 24, 13, 19), (21, 5, 32, 13, 19), (150, 3, 128, 192, 256), (1, 2, 16, 70, 70)])
def test_products_a_head(kn, dtype, sizes):
    rows, heads, k, n, stride = sizes
    x, w = rnd(rows, heads * k, seed=1).to(dtype), rnd(heads, n, k, seed=2).to(dtype)
    out = torch.zeros(rows, heads * stride + 3, dtype=dtype, device=DEV)
    kn.linear_heads(dev(x, dtype), dev(w, dtype), out[:, 3:], heads, stride)
    for h in range(heads):
        want = x[:, h * k : (h + 1) * k].double() @ w[h].double().t()
        assert uc.err(out[:, 3 + h * stride : 3 + h * stride + n].float().cpu(), want) < (TOL_F32 if dtype == torch.float32 else 8e-3)
    assert bool((out[:, :3] == 0).all())


def test_router_and_experts_activation(kn):
    rows, E, ff, top, limit = 37, 7, 12, 3, 1.25
    z = rnd(rows, E, seed=1, std=2.0)
    z[3, 2] = z[3, 5] = z[3].max() + 1  # a tie: the lower index wins
    route = torch.zeros(rows, E, device=DEV)
    kn.moe_route(dev(z), route, top)
    s = torch.sigmoid(z)
    for r in range(rows):
        chosen = sorted(range(E), key=lambda e: (-float(s[r, e]), e))[:top]
        for e in range(E):
            assert float(route[r, e]) == (pytest.approx(float(s[r, e]), rel=1e-6) if e in chosen else -1.0)
    assert float(route[3, 2]) > 0 and float(route[3, 5]) > 0
    kn.moe_route(dev(z), route, top, True)
    assert torch.allclose(route.clamp(min=0).sum(-1).cpu(), torch.ones(rows), atol=1e-6)
    kn.moe_route(dev(z), route, top)
    gu = rnd(rows, E * 2 * ff, seed=2, std=2.0)
    for on_input in (True, False):
        out = torch.zeros(rows, E * ff, device=DEV)
        kn.moe_glu(dev(gu), route, out, E, ff, limit, on_input)
        v = gu.double().reshape(rows, E, 2, ff)
        wt = route.cpu().double()[:, :, None]
        sc = wt if on_input else torch.ones_like(wt)
        g, u = torch.clamp(v[:, :, 0] * sc, max=limit), torch.clamp(v[:, :, 1] * sc, -limit, limit)
        y = g * torch.sigmoid(1.702 * g) * (u + 1) * (1 if on_input else wt)
        want = torch.where(wt >= 0, y, torch.zeros_like(y)).reshape(rows, E * ff)
        assert uc.err(out.cpu(), want) < TOL_F32


def test_rows_sorted_by_expert_and_back(kn):
    rows, E, width = 300, 5, 40
    route = torch.where(rnd(rows, E, seed=1) > 0.3, rnd(rows, E, seed=2).abs(), torch.full((rows, E), -1.0))
    route[7] = -1.0  # a row that chose nothing
    pairs = int((route >= 0).sum())
    counts, order = torch.zeros(E, dtype=torch.int32, device=DEV), torch.full((rows * E,), -7, dtype=torch.int32, device=DEV)
    weight, place_of = torch.zeros(rows * E, 1, device=DEV), torch.zeros(rows, E, dtype=torch.int32, device=DEV)
    kn.moe_sort(dev(route), counts, order, weight, place_of)
    assert counts.tolist() == (route >= 0).sum(0).tolist()
    want_order = [r for e in range(E) for r in range(rows) if route[r, e] >= 0]
    assert order[:pairs].tolist() == want_order and bool((order[pairs:] == -7).all())
    want_w = [float(route[r, e]) for e in range(E) for r in range(rows) if route[r, e] >= 0]
    assert weight[:pairs, 0].tolist() == want_w
    at = 0
    for e in range(E):
        for r in range(rows):
            if route[r, e] >= 0:
                assert int(place_of[r, e]) == at
                at += 1
            else:
                assert int(place_of[r, e]) == -1
    for dtype in (torch.float32, torch.bfloat16):
        src = rnd(rows, width + 8, seed=3).to(dtype)
        dst = torch.zeros(rows * E, width, dtype=dtype, device=DEV)
        kn.moe_gather(dev(src, dtype)[:, :width], order, dst, pairs)
        assert torch.equal(dst[:pairs].cpu(), src[want_order, :width]) and bool((dst[pairs:] == 0).all())
    ys = rnd(pairs, width, seed=4)
    out = torch.full((rows, width), 9.0, device=DEV)
    kn.moe_scatter(dev(ys), place_of, out)
    want = torch.zeros(rows, width, dtype=torch.float64)
    for i, r in enumerate(want_order):
        want[r] += ys[i].double()
    assert uc.err(out.cpu(), want) < 1e-6 and bool((out[7] == 0).all())


def test_bigram_rows_and_the_token_kept_between_steps(kn):
    width, buckets, vocab = 24, 11, 50
    table = rnd(buckets + 1, width, seed=1)
    last = torch.full((4, 1), 49, dtype=torch.int32, device=DEV)
    a, b = [5, 7, 7, 49, 0, 3], [9, 9, 1]
    # step 1: a's first four tokens and b's first; step 2: one more of each, in the other order
    x = torch.zeros(5, width, device=DEV)
    kn.bigram_add(x, dev(table), i32(a[:4] + b[:1]), last, buckets, 1000003, 17, vocab, i32([0, 1, 2, 3, 0]),
                  i32([0, 0, 0, 0, 1]), i32([2, 0]), i32([0, 4, 5]), 2)
    rows = pv.bigram_rows(a, buckets, 1000003, 17)
    assert uc.err(x[:4].cpu(), table[rows[:4]].double()) < 1e-7 and uc.err(x[4].cpu(), table[buckets].double()) < 1e-7
    assert last[:, 0].tolist() == [b[0], 49, a[3], 49]
    x = torch.ones(2, width, device=DEV)
    kn.bigram_add(x, dev(table), i32([b[1], a[4]]), last, buckets, 1000003, 17, vocab, i32([1, 4]), i32([0, 1]),
                  i32([0, 2]), i32([0, 1, 2]), 2)
    want = torch.stack([table[pv.bigram_rows(b, buckets, 1000003, 17)[1]], table[rows[4]]]).double() + 1
    assert uc.err(x.cpu(), want) < 1e-7 and last[:, 0].tolist() == [b[1], 49, a[4], 49]


# ---- the engine ------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, dtype="float32", **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in made:
            made[key] = uc.Case(tmp_path_factory.mktemp("vupelorn"), name, load, dtype=dtype,
                                rounding=dtype == "bfloat16", **kw)
        return made[key]

    return get


@pytest.mark.parametrize("name", ["gla", "latent", "latent2", "moe", "bigram"])
def test_a_mechanism_alone(cases, name):
    case = cases(name)
    uc.whole_and_token_by_token(case, TOL_F32, lengths=(1, 2, 9, 70))
    uc.portions(case, TOL_F32, n=140)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_under_every_cutting_and_batching(cases, name):
    case = cases(name)
    uc.whole_and_token_by_token(case, TOL_F32)
    uc.portions(case, TOL_F32)
    uc.unequal_batches(case, TOL_F32)
    uc.slots_and_blocks_used_again(case, TOL_F32)


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("c", "float32"), ("c", "bfloat16")])
def test_prompt_rows_sorted_by_expert(cases, name, dtype, monkeypatch):
    """The same logits whether a prompt's rows run through all experts' columns or are sorted by expert."""
    from longbow_quarrel_amd.parts.feedforward import MixtureOfExperts
    case = cases(name, dtype)
    t = uc.tokens(300, case.vocab, 12)
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 10 ** 9)
    every = case.run_cut(t, [300])
    monkeypatch.setattr(MixtureOfExperts, "sort_from_rows", 2)
    by_expert = case.run_cut(t, [200, 3, 90])
    if dtype == "float32":
        assert uc.err(by_expert, case.want(t)) < TOL_F32 and uc.err(by_expert, every) < TOL_F32
    else:
        uc.assert_close_bf16(by_expert, case.want(t), case.noise(t))


@pytest.mark.parametrize("seed", range(1, 13))
def test_configurations_drawn_from_a_seed(cases, seed):
    """Other sizes, head counts, ranks, layer orders, lenders of latents, experts and constants, in both dtypes."""
    case = cases(seed)
    t, u = uc.tokens(200, case.vocab, seed), uc.tokens(9, case.vocab, seed + 50)
    assert uc.err(case.run_cut(t, [150, 2, 1, 20]), case.want(t)) < TOL_F32
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, u[:8], range(8)), StepEntry(sb, t[:130], range(130))])
    assert uc.err(out, torch.cat([case.want(u)[:8], case.want(t)[:130]])) < TOL_F32
    out = eng.step([StepEntry(sa, u[8:], [0]), StepEntry(sb, t[130:131], [0])])
    assert uc.err(out, torch.stack([case.want(u)[8], case.want(t)[130]])) < TOL_F32
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()
    case16 = cases(seed, "bfloat16")
    uc.assert_close_bf16(case16.run_cut(t, [150, 2]), case16.want(t), case16.noise(t))


def test_the_residual_stream_after_every_layer(cases):
    case = cases("a")
    got, want = case.layers(uc.tokens(37, case.vocab, 8))
    assert len(got) == len(want) == 5
    for i, (g, w) in enumerate(zip(got, want)):
        assert uc.err(g, w) < TOL_F32, f"after layer {i}"


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_bfloat16_whole_in_portions_and_in_batches(cases, name):
    case = cases(name, "bfloat16")
    t = uc.tokens(150, case.vocab, 3)
    want, noise = case.want(t), case.noise(t)
    uc.assert_close_bf16(case.run_cut(t, [150]), want, noise)
    uc.assert_close_bf16(case.run_cut(t, [64, 1, 63, 2, 3]), want, noise)
    u = uc.tokens(70, case.vocab, 4)
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sa, t[:100], range(100)), StepEntry(sb, u[:3], range(3))])
    uc.assert_close_bf16(out, torch.cat([want[:100], case.want(u)[:3]]), noise)
    got = []
    for i in range(20):
        got.append(eng.step([StepEntry(sb, [u[3 + i]], [0]), StepEntry(sa, [t[100 + i]], [0])]).clone())
    got = torch.cat(got)
    uc.assert_close_bf16(torch.cat([got[0::2], got[1::2]]), torch.cat([case.want(u)[3:23], want[100:120]]), noise)
    eng.release(sa)
    eng.release(sb)
    case.assert_idle()


def test_bfloat16_decoding_over_contexts_whose_keys_are_shared_out(cases, kn):
    """Single tokens over several hundred cached rows: a tile's keys go to several workgroups and a second launch
    merges them; against the same rows as parts of a prompt (one workgroup a tile) and against the plain
    implementation."""
    case = cases("c", "bfloat16")
    m = case.cfg["layers"][0]["mixer"]
    assert kn.sink_attention_workspace(torch.bfloat16, 2, 2, m["heads"], 1, m["kv_rank"] + m["rot_dim"], m["kv_rank"], 64, 0, 0,
                                       700) > 0
    assert kn.sink_attention_workspace(torch.float32, 2, 2, m["heads"], 1, m["kv_rank"] + m["rot_dim"], m["kv_rank"], 64, 0, 0,
                                       700) == 0
    t, u = uc.tokens(640, case.vocab, 61), uc.tokens(330, case.vocab, 62)
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
    uc.assert_close_bf16(got, want, noise)
    uc.assert_close_bf16(got, whole.double(), noise)


def test_a_far_key_carries_the_result(cases):
    case = cases("latent2", sharp=6.0)
    t = uc.tokens(330, case.vocab, 21)
    want = case.want(t)
    assert uc.err(case.run_cut(t, [330]), want) < TOL_F32
    assert uc.err(case.run_cut(t, [127, 1, 64, 2, 100]), want) < TOL_F32
    case = cases("c", sharp=4.0)
    t = uc.tokens(300, case.vocab, 22)
    # (scores of a hundred and more: 32-bit rounding of a score is then a few 1e-5 of a probability)
    assert uc.err(case.run_cut(t, [250]), case.want(t)) < 1e-4


def test_a_slow_decay_keeps_old_tokens_in_the_state(cases):
    case = cases("gla", memory=6.0)
    t = uc.tokens(260, case.vocab, 31)
    want = case.want(t)
    assert uc.err(case.run_cut(t, [260]), want) < TOL_F32
    assert uc.err(case.run_cut(t, [3, 64, 1, 2, 130]), want) < TOL_F32
    # a prompt long enough for the scan in segments, then decoding from the state it left
    t = uc.tokens(640, case.vocab, 32)
    want = case.want(t)
    assert uc.err(case.run_cut(t, [600]), want) < TOL_F32
    assert uc.err(case.run_cut(t, [20, 580, 2]), want) < TOL_F32


@pytest.mark.parametrize("name", ["a", "c"])
def test_long_decoding(cases, name):
    uc.long_decoding(cases(name), TOL_F32)


def test_float32_logits_do_not_depend_on_the_cutting_or_the_batch_at_all(cases):
    case = cases("a")
    t, u = uc.tokens(140, case.vocab, 7), uc.tokens(30, case.vocab, 8)
    whole = case.run_cut(t, [140])
    assert torch.equal(case.run_cut(t, [64, 1, 2, 70]), whole) and torch.equal(case.run_cut(t, [100]), whole)
    eng = case.eng
    sa, sb = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(sb, u, []), StepEntry(sa, t[:90], range(90))])
    assert torch.equal(out, whole[:90])
    out = eng.step([StepEntry(sa, [t[90]], [0]), StepEntry(sb, [5], [])])
    assert torch.equal(out[0], whole[90])
    eng.release(sa)
    eng.release(sb)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(cases, graphs):
    case = cases("a")
    reqs, wants = uc.greedy(case, n_new=12, prompts=5)
    res = lq.generate(case.eng, reqs, max_new_tokens=12, max_batch=3, stop_ids=[], use_graphs=graphs)
    assert res.tokens == wants
    case.assert_idle()


def test_generation_in_bfloat16_captured_and_direct_steps_agree_and_stop_ids_end_requests(cases):
    case = cases("c", "bfloat16")
    assert case.eng.graph_safe
    reqs = [uc.tokens(n, case.vocab, 40 + n) for n in (3, 70, 9, 1, 130, 20)]
    direct = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[], use_graphs=False)
    stop = direct.tokens[1][7]
    a = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=False)
    b = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=True)
    assert a.tokens == b.tokens and a.finish == b.finish and "stop" in a.finish
    case.assert_idle()


def test_command_line_and_trace_replay(cases, tmp_path):
    case = cases("b")
    reqs, wants = uc.greedy(case, n_new=5, prompts=1)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quarrel"), "-model", case.folder, "-dtype", "float32",
                          "-prompt", " ".join(map(str, reqs[0])), "-n", "5", "-temp", "0", "-penalty", "1"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Architecture: Vupelorn" in out.stdout
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in wants[0]]
    a, b = uc.tokens(70, case.vocab, 1), uc.tokens(9, case.vocab, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}, {"id": "b", "tokens": b[:7], "want": [6]}],
              "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [a[66]], "want": [0]}, {"id": "b", "tokens": [b[7]], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": [a[67]], "want": []}, {"id": "b", "tokens": [b[8]], "want": [0]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[68:], "want": [1]}], "end": ["a"]}]
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", case.folder, "--dtype", "float32",
                             "--out", str(tmp_path), "--max-tokens", "79"], stdin=subprocess.PIPE, stdout=subprocess.PIPE,
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
    read = lambda n: torch.from_numpy(np.fromfile(os.path.join(str(tmp_path), f"{n}.f32"), dtype="<f4").reshape(-1, case.vocab).copy())
    wa, wb = case.want(a), case.want(b)
    assert uc.err(read(0), torch.stack([wa[0], wa[65], wb[6]])) < TOL_F32
    assert uc.err(read(1), wa[66:67]) < TOL_F32 and uc.err(read(2), wb[8:9]) < TOL_F32
    assert uc.err(read(3), wa[69:70]) < TOL_F32
