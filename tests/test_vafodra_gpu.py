"""The Vafodra design on the GPU.  First every mechanism alone, a kernel against the plain implementation's
function of the same name (float64), with inputs made so that a fault shows; then the engine in float32 and in
bfloat16 under every cutting and batching; then generation through the entry point, with captured steps and
direct ones, the command line and the trace replay."""
import copy
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import longbow_quarrel_amd as lq
import plain_vafodra as pv
import vafodra_cases as vc
from longbow_quarrel_amd.engine import StepEntry

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
TOL_F32 = 2e-5
# bfloat16 against the plain implementation that rounds nothing: measured 2.0e-3 to 3.7e-3 on these configurations
# (prompts of 3 to 330 tokens, whole and with the last 40 tokens one by one); fixed once at three times the largest
TOL_BF16 = 1.2e-2


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


class Paged:
    """One or several sequences' keys and values in a paged cache whose blocks lie in no particular order."""

    def __init__(self, lengths, kv_heads, key_dim, value_dim, dtype, bs=64, seed=0):
        per = [(n + bs - 1) // bs for n in lengths]
        order = torch.randperm(sum(per) + 3, generator=torch.Generator().manual_seed(seed)).tolist()
        self.table = torch.zeros((len(lengths), max(per)), dtype=torch.int32)
        for s, n in enumerate(per):
            self.table[s, :n] = torch.tensor([order.pop() for _ in range(n)])
        self.table = self.table.to(DEV)
        self.k = torch.zeros((sum(per) + 3, kv_heads, bs, key_dim), dtype=dtype, device=DEV)
        self.v = torch.zeros((sum(per) + 3, kv_heads, value_dim, bs), dtype=dtype, device=DEV)
        self.bs = bs


# ---------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [
    # heads, kv heads, key size, value size, window, kept, sink, generic kernel
    (4, 2, 32, 16, 7, 2, True, False), (2, 2, 48, 80, 70, 0, True, False), (3, 1, 16, 16, 64, 65, False, False),
    (2, 1, 24, 40, 9, 3, True, False), (4, 4, 64, 64, 0, 0, True, False), (4, 2, 32, 16, 7, 2, True, True),
    (1, 1, 160, 144, 1, 1, True, False),
])
def test_windowed_attention_with_sink_kept_tokens_and_gate(kn, sizes, dtype):
    """Rows of a prompt and the same rows as single tokens.  Every eighth row's query is aimed at one key (its
    score stands out): the key just inside the window, just outside it, the last kept token, the first one
    that is not kept, a key far back, in turn."""
    H, G, D, P, window, keep, sink, generic = sizes
    T = 200
    q, k, v = rnd(T, H, D, seed=1), rnd(T, G, D, seed=2), rnd(T, G, P, seed=3)
    gate = rnd(T, H, seed=4)
    w = window if window else T
    for n, i in enumerate(range(70, T, 8)):
        j = [i - w + 1, i - w, keep - 1, keep, i // 3][n % 5]
        if 0 <= j <= i:
            for h in range(H):
                q[i, h] = k[j, h // (H // G)] * 6.0 / k[j, h // (H // G)].norm()
    q, k, v, gate = (t.to(dtype).double() for t in (q, k, v, gate))  # what the kernel is given, exactly
    scale = 1.0 / math.sqrt(D)
    want = pv.sink_attention(q, k, v, scale, w, keep)
    if not sink:  # the plain function always has the sink: undo it (p_j (1 + sum) / sum)
        i_, j_ = torch.arange(T)[:, None], torch.arange(T)[None, :]
        mask = (j_ <= i_) & ((i_ - j_ < w) | (j_ < keep))
        for h in range(H):
            e = torch.where(mask, torch.exp((q[:, h] @ k[:, h // (H // G)].T) * scale), torch.zeros(T, T, dtype=q.dtype))
            want[:, h] = (e / e.sum(-1, keepdim=True)) @ v[:, h // (H // G)]
    want = (want * torch.sigmoid(gate)[:, :, None]).reshape(T, H * P)
    cache = Paged([T], G, D, P, dtype, seed=5)
    pos, seq, slot = i32(range(T)), i32([0] * T), i32([0])
    kn.force_generic = generic
    try:
        kn.kv_store(dev(k.reshape(T, -1), dtype), dev(v.reshape(T, -1), dtype), G, D, P, pos, seq, slot, cache.table,
                    cache.k, cache.v, 64)
        qd, gd = dev(q.reshape(T, -1), dtype), dev(gate, dtype)
        out = torch.zeros((T, H * P), dtype=dtype, device=DEV)
        kn.sink_attention(qd, out, H, G, D, P, pos, seq, slot, cache.table, cache.k, cache.v, 64, scale, window=window,
                          keep_first=keep, sink=sink, gate=gd)
        tol = 1e-5 if dtype == torch.float32 else 1e-2  # (bfloat16: the output's own rounding)
        assert vc.err(out, want) < tol
        for r in list(range(60, 76)) + [127, 128, 129, 191, 199]:  # single tokens, over block edges too
            one = torch.zeros((1, H * P), dtype=dtype, device=DEV)
            kn.sink_attention(qd[r : r + 1], one, H, G, D, P, i32([r]), i32([0]), slot, cache.table, cache.k, cache.v, 64,
                              scale, window=window, keep_first=keep, sink=sink, gate=gd[r : r + 1], decode=True)
            assert vc.err(one[0], want[r]) < tol, r
            if dtype == torch.float32 and not generic:
                assert torch.equal(one[0], out[r]), r  # the same sums in the same order
    finally:
        kn.force_generic = False


@pytest.mark.parametrize("taps,bias", [(4, True), (2, False), (3, True), (1, True)])
def test_short_convolution_carries_its_last_inputs(kn, taps, bias):
    C, slots = 70, 3
    lengths = [23, 1, 9]
    xs = [rnd(n, C, seed=10 + i) for i, n in enumerate(lengths)]
    w, b = rnd(C, taps, seed=20), rnd(C, seed=21) if bias else None
    want = [pv.silu(pv.causal_conv(x.double(), w.double(), None if b is None else b.double())) for x in xs]
    state = torch.full((slots, max(1, taps - 1), C), 7.0, device=DEV)  # what an earlier sequence left
    state[[2, 0, 1]] = 0.0  # ... and the zeros of a slot that was taken anew
    at = [0, 0, 0]
    for cut in ([5, 1, 2], [1, 0, 3], [2, 0, 1], [15, 0, 3]):  # rows of each sequence in this step
        live = [i for i, n in enumerate(cut) if n]
        x = torch.cat([xs[i][at[i] : at[i] + cut[i]] for i in live])
        rows = x.shape[0]
        cu = [0]
        for i in live:
            cu.append(cu[-1] + cut[i])
        out = torch.zeros((rows, C), device=DEV)
        kn.causal_conv(dev(x), dev(w), None if b is None else dev(b), state, out,
                       i32([at[i] + r for i in live for r in range(cut[i])]),
                       i32([n for n, i in enumerate(live) for _ in range(cut[i])]), i32([[2, 0, 1][i] for i in live]),
                       i32([at[i] for i in live]), i32([at[i] + cut[i] for i in live]), i32(cu), len(live))
        exp = torch.cat([want[i][at[i] : at[i] + cut[i]] for i in live])
        assert vc.err(out, exp) < 1e-6
        for i in live:
            at[i] += cut[i]
    assert at == lengths


@pytest.mark.parametrize("sizes", [(4, 16, 24, 1), (3, 24, 20, 3), (2, 64, 130, 2), (6, 40, 64, 2), (1, 8, 300, 1), (2, 12, 9, 2),
                                   (1, 4, 600, 1), (8, 64, 128, 2)])
def test_state_space_scan_in_portions(kn, sizes):
    H, P, N, G = sizes
    T = 45
    x, B, C, dt = rnd(T, H, P, seed=1), rnd(T, G, N, seed=2, std=0.5), rnd(T, G, N, seed=3, std=0.5), rnd(T, H, seed=4)
    dt_bias, a_log, d_skip = rnd(H, seed=5), rnd(H, seed=6, std=0.7), rnd(H, seed=7)
    want = pv.ssd_scan(x.double(), B.double(), C.double(), pv.softplus(dt.double() + dt_bias.double()),
                       a_log.double(), d_skip.double()).reshape(T, H * P)
    state = torch.zeros((2, H, P, N), device=DEV)
    state[0] = 3.0  # another sequence's
    got, at = [], 0
    for n in (1, 1, 7, 2, 30, 4):
        y = torch.zeros((n, H * P), device=DEV)
        sl = slice(at, at + n)
        kn.ssd_scan(dev(x[sl].reshape(n, -1)), dev(B[sl].reshape(n, -1)), dev(C[sl].reshape(n, -1)), dev(dt[sl]),
                    dev(dt_bias), dev(a_log), dev(d_skip), state, y, H, P, N, G, i32([1]), i32([0, n]), 1)
        got.append(y)
        at += n
    assert vc.err(torch.cat(got), want) < 2e-6
    assert float((state[0] - 3.0).abs().max()) == 0.0
    # two sequences in one step equal each alone
    both = torch.zeros((2, H, P, N), device=DEV)
    y2 = torch.zeros((T + 10, H * P), device=DEV)
    cat = lambda t: dev(torch.cat([t[:10], t]).reshape(T + 10, -1))
    kn.ssd_scan(cat(x), cat(B), cat(C), cat(dt), dev(dt_bias), dev(a_log), dev(d_skip), both, y2, H, P, N, G,
                i32([1, 0]), i32([0, 10, T + 10]), 2)
    assert vc.err(y2[10:], want) < 2e-6 and vc.err(y2[:10], want[:10]) < 2e-6
    assert torch.equal(y2[10:], torch.cat(got))


def test_state_space_scan_of_a_long_prompt_in_segments(kn):
    """A long sequence beside a short one: the long one is cut into segments that run side by side (given scratch);
    results and the state left behind equal the plain recurrence, and the same launch without scratch."""
    H, P, N, G = 3, 24, 40, 1
    T, T2 = 1100, 37
    x, B, C, dt = rnd(T, H, P, seed=1), rnd(T, G, N, seed=2, std=0.5), rnd(T, G, N, seed=3, std=0.5), rnd(T, H, seed=4)
    dt_bias, a_log, d_skip = rnd(H, seed=5), rnd(H, seed=6, std=0.7) - 1.0, rnd(H, seed=7)
    want = pv.ssd_scan(x.double(), B.double(), C.double(), pv.softplus(dt.double() + dt_bias.double()),
                       a_log.double(), d_skip.double()).reshape(T, H * P)
    cat = lambda t: dev(torch.cat([t[:T2], t]).reshape(T + T2, -1))
    need = kn.ssd_scan_workspace(2, H, P, N, T)
    assert need > 0 and kn.ssd_scan_workspace(2, H, P, N, 511) == 0
    outs, states = [], []
    for scratch in (torch.zeros(need, device=DEV), None):
        state = torch.zeros((3, H, P, N), device=DEV)
        y = torch.zeros((T + T2, H * P), device=DEV)
        kn.ssd_scan(cat(x), cat(B), cat(C), cat(dt), dev(dt_bias), dev(a_log), dev(d_skip), state, y, H, P, N, G,
                    i32([2, 0]), i32([0, T2, T + T2]), 2, max_rows=T, workspace=scratch)
        assert vc.err(y[T2:], want) < 5e-6 and vc.err(y[:T2], want[:T2]) < 5e-6
        outs.append(y)
        states.append(state)
    assert vc.err(states[0], states[1]) < 5e-6 and float(states[0][1].abs().max()) == 0.0
    assert torch.equal(outs[0][:T2], outs[1][:T2])  # the short sequence runs whole either way
    # ... and goes on from the state that the segments left
    y = torch.zeros((1, H * P), device=DEV)
    more = [rnd(1, H, P, seed=11), rnd(1, G, N, seed=12), rnd(1, G, N, seed=13), rnd(1, H, seed=14)]
    for st in states:
        kn.ssd_scan(*[dev(t.reshape(1, -1)) for t in more], dev(dt_bias), dev(a_log), dev(d_skip), st, y, H, P, N, G,
                    i32([0]), i32([0, 1]), 1)
    assert vc.err(states[0][0], states[1][0]) < 5e-6


@pytest.mark.parametrize("sizes", [(4, 2, 16, 32), (2, 2, 48, 16), (2, 1, 24, 40), (3, 3, 128, 64), (1, 1, 272, 8), (3, 3, 12, 20),
                                   (1, 1, 520, 4)])
def test_gated_delta_rule_scan_in_portions(kn, sizes):
    H, G, D, P = sizes
    T = 40
    q, k, v = rnd(T, G, D, seed=1), rnd(T, G, D, seed=2), rnd(T, H, P, seed=3)
    beta, a = rnd(T, H, seed=4), rnd(T, H, seed=5)
    dt_bias, a_log = rnd(H, seed=6), rnd(H, seed=7, std=0.7)
    qd, kd = q.double(), k.double()
    qn = qd / torch.sqrt((qd * qd).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    kn_ = kd / torch.sqrt((kd * kd).sum(-1, keepdim=True) + 1e-6)
    g = torch.exp(-torch.exp(a_log.double()) * pv.softplus(a.double() + dt_bias.double()))
    want = pv.delta_scan(qn, kn_, v.double(), torch.sigmoid(beta.double()), g).reshape(T, H * P)
    state = torch.zeros((1, H, P, D), device=DEV)
    got, at = [], 0
    for n in (1, 2, 1, 20, 16):
        o = torch.zeros((n, H * P), device=DEV)
        sl = slice(at, at + n)
        kn.delta_scan(dev(q[sl].reshape(n, -1)), dev(k[sl].reshape(n, -1)), dev(v[sl].reshape(n, -1)), dev(beta[sl]),
                      dev(a[sl]), dev(dt_bias), dev(a_log), state, o, H, G, D, P, D ** -0.5, 1e-6, i32([0]), i32([0, n]), 1)
        got.append(o)
        at += n
    assert vc.err(torch.cat(got), want) < 5e-6


def test_norms_gates_and_element_wise_steps(kn):
    rows, width = 9, 200
    x, d1, d2 = rnd(rows, width, seed=1), rnd(rows, width, seed=2), rnd(rows, width, seed=3)
    w, b, alpha = rnd(width, seed=4), rnd(width, seed=5), torch.tensor([0.6])
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 5e-3)):
        xd = dev(x)
        out = torch.zeros((rows, width), dtype=dtype, device=DEV)
        kn.dynamic_tanh(xd, dev(w), dev(b), dev(alpha), out, delta=dev(torch.stack([d1, d2])), delta_scale=0.3)
        stream = x.double() + 0.3 * (d1.double() + d2.double())
        assert vc.err(xd, stream) < 1e-6  # the stream is brought up to date
        assert vc.err(out, pv.dynamic_tanh(stream, w.double(), b.double(), alpha.double())) < tol
        kn.dynamic_tanh(xd, dev(w), dev(b), dev(alpha), out)
        assert vc.err(xd, stream) < 1e-6
    xd = dev(x)
    kn.add_scaled(xd, dev(torch.stack([d1, d2])), -1.5)
    assert vc.err(xd, x.double() - 1.5 * (d1.double() + d2.double())) < 1e-6
    # gated linear unit
    gu = rnd(rows, 2 * 70, seed=6, std=2.0)
    for act, fn in (("relu", torch.relu), ("silu", pv.silu), ("gelu_tanh", pv.gelu_tanh)):
        out = torch.zeros((rows, 70), device=DEV)
        kn.glu(dev(gu), out, act)
        assert vc.err(out, fn(gu[:, :70].double()) * gu[:, 70:].double()) < 1e-6, act
    # RMS norm in groups with a gate, both orders; a weight per column and one that the groups share
    y, z = rnd(rows, 120, seed=7), rnd(rows, 120, seed=8)
    for group, wlen, first in ((40, 120, True), (120, 120, True), (24, 24, False), (8, 120, False)):
        wt = rnd(wlen, seed=9)
        out = torch.zeros((rows, 120), device=DEV)
        kn.gated_rmsnorm(dev(y), dev(z), dev(wt), 1e-3, group, out, gate_first=first)
        yd, gate = y.double(), pv.silu(z.double())
        v = (yd * gate if first else yd).view(rows, 120 // group, group)
        v = pv.rms_divide(v, 1e-3).reshape(rows, 120) * wt.double().repeat(120 // wlen)
        assert vc.err(out, v if first else v * gate) < 1e-6, (group, wlen, first)
    # mean of branches, each RMS-normed with its own weight
    for n in (1, 2, 3):
        stack, ws = rnd(n, rows, width, seed=10), [rnd(width, seed=11 + i) for i in range(n)]
        out = torch.zeros((rows, width), device=DEV)
        kn.rmsnorm_mean(dev(stack), [dev(t) for t in ws], 1e-4, out)
        want = sum(pv.rms_divide(stack[i].double(), 1e-4) * ws[i].double() for i in range(n)) / n
        assert vc.err(out, want) < 1e-6
    # the embedding's scale
    table = rnd(50, 64, seed=12).to(torch.bfloat16)
    out = torch.zeros((4, 64), device=DEV)
    kn.embed(table.to(DEV), i32([3, 49, 0, 3]), out, scale=2.5)
    assert vc.err(out, table.double()[[3, 49, 0, 3]] * 2.5) < 1e-7


# ---------------------------------------------------------------------------------------- the engine
def load(folder, dtype, max_tokens):
    return lq.load_engine(folder, dtype=dtype, max_tokens=max_tokens, max_slots=8, max_sequence_tokens=max_tokens)


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    made = {}

    def get(name, dtype="float32", sharp=1.0):
        if (name, dtype, sharp) not in made:
            made[(name, dtype, sharp)] = vc.Case(tmp_path_factory.mktemp("vafodra"), name, load, dtype=dtype, sharp=sharp)
        return made[(name, dtype, sharp)]

    return get


def tol(dtype):
    return TOL_F32 if dtype == "float32" else TOL_BF16


PARAMS = [(n, d) for n in ("a", "b", "c", "d", "f") for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_whole_prompts_and_token_by_token(cases, name, dtype):
    vc.whole_and_token_by_token(cases(name, dtype), tol(dtype))


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_portions_down_to_two_tokens(cases, name, dtype):
    vc.portions(cases(name, dtype), tol(dtype))


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_unequal_batches_against_each_request_alone(cases, name, dtype):
    vc.unequal_batches(cases(name, dtype), tol(dtype))


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_slots_and_blocks_that_are_used_again(cases, name, dtype):
    vc.slots_and_blocks_used_again(cases(name, dtype), tol(dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_of_a_small_real_model(cases, dtype):
    case = cases("e", dtype)
    t = vc.tokens(330, case.vocab, 6)
    for cuts in ([330], [290], [130, 70, 100]):
        assert vc.err(case.run_cut(t, cuts), case.want(t)) < tol(dtype), cuts
    case.assert_idle()


def test_a_prompt_long_enough_for_the_scan_in_segments_then_decoding(cases):
    case = cases("a", "float32")
    t = vc.tokens(700, case.vocab, 12)
    assert vc.err(case.run_cut(t, [690]), case.want(t)) < TOL_F32
    u = vc.tokens(40, case.vocab, 13)  # a long and a short request in one step
    eng = case.eng
    s1, s2 = eng.new_sequence(), eng.new_sequence()
    out = eng.step([StepEntry(s1, u, range(40)), StepEntry(s2, t[:600], range(600))])
    assert vc.err(out[:40], case.want(u)) < TOL_F32 and vc.err(out[40:], case.want(t)[:600]) < TOL_F32
    out = eng.step([StepEntry(s2, t[600:], range(100))])
    assert vc.err(out, case.want(t)[600:]) < TOL_F32
    eng.release(s1)
    eng.release(s2)
    case.assert_idle()


@pytest.mark.parametrize("name", ["a", "c"])
def test_peaked_attention_in_prompts_and_in_decoding(cases, name):
    case = cases(name, "float32", sharp=8.0)
    t = vc.tokens(150, case.vocab, 4)
    for cuts in ([150], [60], [3, 64, 64]):
        assert vc.err(case.run_cut(t, cuts), case.want(t)) < TOL_F32, cuts


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("b", "bfloat16"), ("c", "float32")])
def test_long_decoding(cases, name, dtype):
    vc.long_decoding(cases(name, dtype), tol(dtype), steps=300)


def test_float32_logits_do_not_depend_on_the_cutting_or_the_batch_at_all(cases):
    case = cases("a", "float32")
    t, u = vc.tokens(140, case.vocab, 8), vc.tokens(31, case.vocab, 9)
    whole = case.run_cut(t, [140])
    eng = case.eng
    s1, s2 = eng.new_sequence(), eng.new_sequence()
    first = eng.step([StepEntry(s2, u, []), StepEntry(s1, t[:100], range(100))])
    rest = [eng.step([StepEntry(s2, [5], []), StepEntry(s1, [x], [0])]) for x in t[100:]]
    eng.release(s1)
    eng.release(s2)
    assert torch.equal(torch.cat([first] + rest), whole)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(cases, graphs):
    case = cases("a", "float32")
    reqs, wants = vc.greedy(case, n_new=12, prompts=5)
    res = lq.generate(case.eng, reqs, max_new_tokens=12, max_batch=3, stop_ids=[], use_graphs=graphs)
    assert res.tokens == wants
    case.assert_idle()


def test_generation_in_bfloat16_captured_and_direct_steps_agree_and_stop_ids_end_requests(cases):
    case = cases("b", "bfloat16")
    assert case.eng.graph_safe
    reqs = [vc.tokens(n, case.vocab, 40 + n) for n in (3, 70, 9, 1, 130, 20)]
    direct = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[], use_graphs=False)
    stop = direct.tokens[1][7]
    a = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=False)
    b = lq.generate(case.eng, reqs, max_new_tokens=40, max_batch=4, stop_ids=[stop], use_graphs=True)
    assert a.tokens == b.tokens and a.finish == b.finish and "stop" in a.finish
    case.assert_idle()


def test_command_line_and_trace_replay(cases, tmp_path):
    case = cases("c", "float32")
    reqs, wants = vc.greedy(case, n_new=5, prompts=1)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "quarrel"), "-model", case.folder, "-dtype", "float32",
                          "-prompt", " ".join(map(str, reqs[0])), "-n", "5", "-temp", "0", "-penalty", "1"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Architecture: Vafodra" in out.stdout
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in wants[0]]
    # the replay: two requests start together with different lengths, go on token by token, one ends earlier
    a, b = vc.tokens(70, case.vocab, 1), vc.tokens(9, case.vocab, 2)
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
    assert vc.err(read(0), torch.stack([wa[0], wa[65], wb[6]])) < TOL_F32
    assert vc.err(read(1), wa[66:67]) < TOL_F32 and vc.err(read(2), wb[8:9]) < TOL_F32
    assert vc.err(read(3), wa[69:70]) < TOL_F32
