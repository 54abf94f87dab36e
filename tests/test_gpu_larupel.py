"""Larupel on the GPU: the kernels it brought, each against a plain float32 computation in torch,
and the model in both dtypes against the plain implementation in tests/plain/larupel_plain.py: every
cutting, mixed batches on reused pages and slots, contexts long enough for the attention kernels to
cut their keys into runs, captured decode steps, generation, and the programs a user starts."""

from __future__ import annotations

import json
import math
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces
from larupel_configs import LARUPEL, attention, delta, dense, general_delta, layer, model, moe, write_larupel
from plain import larupel_plain as plain
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
DEV = "cuda:0"
# 32-bit: a row's largest error over its largest logit; the norm behind a head's read-out that nearly
# cancels brings its rounding back to size one (4e-5 seen on the host), the median row is at 5e-7.
F32_TOL = 1e-4
# bfloat16, the same measure, against the plain model with its products and activations rounded to
# bfloat16 (``bf16_bars``): the median and the ninth decile of a trace's rows, and how many rows lie far
# out. A single row may be anywhere: in these tiny models a router's close call falls the other way after
# rounding, in the yardstick as in the engine but not at the same token, and moves that row (and, through
# a state, some behind it) by tenths; a mean would follow those few rows.
BF16_FACTOR, BF16_TAIL_FACTOR, BF16_FAR_FACTOR, BF16_FAR_SHARE = 1.5, 2.5, 2.0, 0.03


@pytest.fixture(scope="module")
def ops():
    from prefixserve_amd.kernels.ops import HipOps
    from prefixserve_amd.parts.base import Workspace

    return HipOps(torch.device(DEV), Workspace(torch.device(DEV)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_larupel(tmp_path_factory.mktemp(f"larupel-{name}"), name) for name in LARUPEL}


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def rel(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def runner_for(folder, pages, dtype, slots=4, graphs=False):
    return ModelRunner(folder, dtype=dtype, device=DEV, num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=slots,
                       use_graphs=graphs)


class Step:
    """The few fields of a step's context that the delta rules' kernels read."""

    def __init__(self, lengths, slots):
        starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        self.num_tokens, self.num_items = int(starts[-1]), len(lengths)
        self.item_start = torch.tensor(starts, device=DEV)
        self.slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
        self.tok_item = torch.tensor(np.repeat(np.arange(len(lengths)), lengths).astype(np.int32), device=DEV)


def layer_norm(x, w, b, eps):
    d = x - x.mean(-1, keepdim=True)
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


# ------------------------------------------------------------------ kernels

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t,h", [(1, 64), (7, 100), (130, 72), (40, 1000), (9, 30), (3, 2049)])
def test_layer_norm_around_the_stream(ops, dtype, t, h):
    """stream += norm(delta) with the next norm's output from the same kernel; a delta in float32 slices;
    the norm of picked rows."""
    w1, b1, w2, b2 = (rnd(h, seed=s, scale=0.5) + (1.0 if s % 2 else 0.0) for s in (1, 2, 3, 4))
    stream = rnd(t, h, seed=5, scale=3.0)
    delta_rows = rnd(t, h, dtype=dtype, seed=6)
    got_stream = stream.clone()
    out = torch.empty(t, h, dtype=dtype, device=DEV)
    ops.layernorm_step(got_stream, delta_rows, (w1, b1, 1e-5), (w2, b2, 1e-6), out)
    want_stream = stream + layer_norm(delta_rows.float(), w1, b1, 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert rel(got_stream.cpu(), want_stream.cpu()) < 1e-5
    assert rel(out.float().cpu(), layer_norm(want_stream, w2, b2, 1e-6).cpu()) < tol
    slices = rnd(3, t, h, seed=7)
    got_stream = stream.clone()
    ops.layernorm_step(got_stream, slices, (w1, b1, 1e-5), None, None)
    assert rel(got_stream.cpu(), (stream + layer_norm(slices[0] + slices[1] + slices[2], w1, b1, 1e-5)).cpu()) < 1e-5
    rows = torch.tensor(sorted({0, t - 1, t // 2}), dtype=torch.int32, device=DEV)
    out = torch.empty(rows.numel(), h, dtype=dtype, device=DEV)
    ops.layernorm_step(stream, None, None, (w2, b2, 1e-6), out, rows=rows)
    assert rel(out.float().cpu(), layer_norm(stream[rows.long()], w2, b2, 1e-6).cpu()) < tol


@pytest.mark.parametrize("h", [64, 50, 7])
def test_sinusoid_of_far_positions(ops, h):
    pos = torch.tensor([0, 1, 2, 17, 4095, 100000, 1000003], dtype=torch.int32, device=DEV)
    x = rnd(7, h, seed=1)
    got = x.clone()
    i = torch.arange((h + 1) // 2, dtype=torch.float64)
    freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * i / h)
    ops.add_sinusoid(got, pos, freq.to(DEV))
    want = x.cpu().double() + torch.from_numpy(plain.sinusoid(pos.cpu().numpy(), h))
    assert float((got.cpu().double() - want).abs().max()) < 5e-7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,groups,dim,vdim,taps", [(4, 2, 8, 12, 3), (1, 1, 40, 16, 1), (6, 6, 64, 64, 4), (2, 1, 130, 20, 7)])
def test_gated_delta_rule_continues_from_its_slot(ops, dtype, heads, groups, dim, vdim, taps):
    """Convolution, operands, recurrence and the gated norm behind it over three steps: requests in
    slots full of junk except where they start, continued by a single token, by fewer tokens than
    taps, and by a long portion, beside a new request."""
    ks, vs = groups * dim, heads * vdim
    ch = 2 * ks + vs
    tail = (taps - 1) * ch
    conv_w = rnd(ch, taps, seed=1, scale=0.6)
    a_log, dt_bias, norm_w = rnd(heads, seed=2, scale=0.5) - 2.0, rnd(heads, seed=3, scale=0.5), rnd(vdim, seed=4, scale=0.3) + 1.0
    state = torch.full((5, tail + heads * vdim * dim), 1e30, device=DEV)
    seqs = {s: (rnd(n, ch + vs, dtype=dtype, seed=10 + s), rnd(n, 2 * heads, seed=20 + s)) for s, n in ((4, 109), (1, 14), (2, 70), (0, 5))}

    def plain_run(rows, gates):
        n = rows.shape[0]
        x = torch.cat([torch.zeros(taps - 1, ch, device=DEV), rows[:, :ch].float()])
        u = sum(conv_w[:, j] * x[j: j + n] for j in range(taps))
        u = u * torch.sigmoid(u)
        q, k, v = u[:, :ks].view(n, groups, dim), u[:, ks: 2 * ks].view(n, groups, dim), u[:, 2 * ks:].view(n, heads, vdim)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        b = torch.sigmoid(gates[:, :heads])
        g = torch.exp(-torch.exp(a_log) * torch.nn.functional.softplus(gates[:, heads:] + dt_bias))
        s = torch.zeros(heads, dim, vdim, device=DEV, dtype=torch.float64)
        q, k, v, b, g = (z.double() for z in (q, k, v, b, g))
        out = []
        for t in range(n):
            kk, qq = (z[t].repeat_interleave(heads // groups, dim=0) for z in (k, q))
            s = g[t][:, None, None] * s
            write = b[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", s, kk))
            s = s + kk[:, :, None] * write[:, None, :]
            out.append(torch.einsum("hdv,hd->hv", s, qq))
        o = torch.stack(out).float()
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + 1e-5) * norm_w
        z = rows[:, ch:].float()
        return o.reshape(n, vs) * z * torch.sigmoid(z)

    def step(pieces):
        ctx = Step([p[0].shape[0] for _, p in pieces], [s for s, _ in pieces])
        rows = torch.cat([p[0] for _, p in pieces]).contiguous()
        gates = torch.cat([p[1] for _, p in pieces]).contiguous()
        t = ctx.num_tokens
        u = torch.empty(t, ch, device=DEV)
        ops.short_conv(rows, 0, conv_w, u, state, 0, ctx, silu=True)
        coef = torch.empty(t, 3 * heads, device=DEV)
        ops.gated_delta_prepare(u, groups, dim, gates, a_log, dt_bias, coef, dim ** -0.5, 1e-6)
        o = torch.empty(t, vs, device=DEV)
        ops.delta_scan(keys=(u, ks), directions=(u, ks), removals=(u, ks), queries=(u, 0), key_groups=groups, decay_vectors=None,
                       decay=(coef, 0), removal_scale=(coef, heads), value_scale=(coef, 2 * heads), values=(u, 2 * ks), out=o,
                       state=state, state_offset=tail, ctx=ctx, heads=heads, dim=dim, vdim=vdim, reads_decayed=True)
        out = torch.empty(t, vs, dtype=dtype, device=DEV)
        ops.heads_norm_gate(o, heads, vdim, norm_w, False, 1e-5, rows, ch, "silu", out)
        return out.float()

    def cut(s, a, b=None):
        return (seqs[s][0][a:b], seqs[s][1][a:b])

    for s in (4, 1, 2):
        state[s].zero_()                                   # what the runner does for a request at position 0
    first = step([(4, cut(4, 0, 7)), (1, cut(1, 0, 3)), (2, cut(2, 0))])
    state[0].zero_()
    second = step([(1, cut(1, 3, 4)), (0, cut(0, 0)), (4, cut(4, 7))])
    third = step([(1, cut(1, 4, 6))])                      # two tokens behind a single one: fewer than most taps
    fourth = step([(1, cut(1, 6))])
    got = {4: torch.cat([first[:7], second[6:]]), 1: torch.cat([first[7:10], second[:1], third, fourth]), 2: first[10:], 0: second[1:6]}
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    for s, (rows, gates) in seqs.items():
        assert rel(got[s].cpu(), plain_run(rows, gates).cpu()) < tol, s
    assert bool((state[3] == 1e30).all())                  # a slot nobody used


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rank", [(2, 16, 5), (1, 40, 1), (4, 64, 16), (3, 200, 9)])
def test_generalized_delta_rule_continues_from_its_slot(ops, dtype, heads, dim, rank):
    s_ = heads * dim
    width = 5 * s_ + rank
    a_bias, w2, w0, norm_w = rnd(s_, seed=1, scale=0.5), rnd(s_, rank, seed=2, scale=0.5), rnd(s_, seed=3), rnd(s_, seed=4, scale=0.3) + 1.0
    floor = math.exp(-0.5)
    state = torch.full((4, s_ * dim), 1e30, device=DEV)
    seqs = {s: rnd(n, width, dtype=dtype, seed=10 + s) for s, n in ((3, 90), (1, 9), (0, 33))}

    def plain_run(rows):
        n = rows.shape[0]
        x = rows.double()
        r, k, v, gate, a_in = (x[:, i * s_: (i + 1) * s_].view(n, heads, dim) for i in range(5))
        low = torch.tanh(x[:, 5 * s_:]) @ w2.double().T + w0.double()
        w = torch.exp(-floor * torch.sigmoid(low)).view(n, heads, dim)
        a = torch.sigmoid(a_in + a_bias.double().view(heads, dim))
        c = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        s = torch.zeros(heads, dim, dim, device=DEV, dtype=torch.float64)
        out = []
        for t in range(n):
            seen = torch.einsum("hd,hdv->hv", c[t], s)
            s = w[t][:, :, None] * s - (a[t] * c[t])[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
            out.append(torch.einsum("hdv,hd->hv", s, r[t]))
        o = torch.stack(out)
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + 1e-5)
        return (o.reshape(n, s_) * norm_w.double() * torch.sigmoid(gate.reshape(n, s_))).float()

    def step(pieces):
        ctx = Step([p.shape[0] for _, p in pieces], [s for s, _ in pieces])
        rows = torch.cat([p for _, p in pieces]).contiguous()
        t = ctx.num_tokens
        operands = torch.empty(t, 6 * s_, device=DEV)
        ops.general_delta_prepare(rows, 0, s_, 2 * s_, 4 * s_, 5 * s_, a_bias, w2.t().contiguous(), w0, operands, heads, dim, floor, 1e-6)
        o = torch.empty(t, s_, device=DEV)
        ops.delta_scan(keys=(operands, s_), directions=(operands, 5 * s_), removals=(operands, 4 * s_), queries=(operands, 0),
                       key_groups=heads, decay_vectors=(operands, 3 * s_), decay=None, removal_scale=None, value_scale=None,
                       values=(operands, 2 * s_), out=o, state=state, state_offset=0, ctx=ctx, heads=heads, dim=dim, vdim=dim,
                       reads_decayed=False)
        out = torch.empty(t, s_, dtype=dtype, device=DEV)
        ops.heads_norm_gate(o, heads, dim, norm_w, True, 1e-5, rows, 3 * s_, "sigmoid", out)
        return out.float()

    state[3].zero_()
    state[1].zero_()
    first = step([(3, seqs[3][:40]), (1, seqs[1][:1])])
    state[0].zero_()
    second = step([(1, seqs[1][1:2]), (0, seqs[0]), (3, seqs[3][40:42])])
    third = step([(3, seqs[3][42:]), (1, seqs[1][2:])])
    got = {3: torch.cat([first[:40], second[34:], third[:48]]), 1: torch.cat([first[40:], second[:1], third[48:]]), 0: second[1:34]}
    tol = 3e-5 if dtype == torch.float32 else 2e-2
    for s, rows in seqs.items():
        assert rel(got[s].cpu(), plain_run(rows).cpu()) < tol, s
    assert bool((state[2] == 1e30).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("t", [1, 5, 40, 300])
@pytest.mark.parametrize("experts,top,k,f", [(8, 4, 64, 24), (5, 1, 40, 16), (6, 6, 72, 8), (32, 3, 128, 64)])
def test_experts_weighted_on_their_output_by_the_softmax_over_the_chosen(ops, dtype, t, experts, top, k, f):
    """Router with a bias, the largest logits, softmax over those alone; the weight on the expert's output;
    the shared expert's gate per token. Every size of step: the fused router, the product + choice, the
    experts row by row and grouped on the matrix cores."""
    x = rnd(t, k, dtype=dtype, seed=1)
    w_router, bias = rnd(experts, k, seed=2, scale=0.4), rnd(experts, seed=3)
    gate_up, down = rnd(experts, 2 * f, k, dtype=dtype, seed=4, scale=0.2), rnd(experts, k, f, dtype=dtype, seed=5, scale=0.2)
    chosen = torch.empty(t, top, dtype=torch.int32, device=DEV)
    weight = torch.empty(t, top, device=DEV)
    router_act = w_router if dtype == torch.float32 else w_router.to(dtype)
    router32 = router_act.float()                          # what both forms of the router multiply with
    ops.moe_route(x, router32.contiguous(), chosen, weight, router_act.contiguous(), bias=bias, mode=1)
    logits = x.float() @ router32.T + bias
    order = torch.argsort(-logits, dim=-1, stable=True)[:, :top]
    picked = torch.gather(logits, 1, order)
    close_call = (torch.sort(logits, dim=-1, descending=True).values[:, top - 1] -
                  (torch.sort(logits, dim=-1, descending=True).values[:, top] if top < experts else -1e30)) < 1e-4
    sure = ~close_call
    assert torch.equal(chosen[sure].long(), order[sure])
    assert rel(weight[sure].cpu(), torch.softmax(picked, dim=-1)[sure].cpu()) < 1e-5
    act = torch.empty(t * top, f, dtype=dtype, device=DEV)
    out = torch.full((top, t, k), 7.0, device=DEV)
    ops.moe_experts(x, chosen, weight, gate_up, down, act, out, 1.0, float("inf"), 0.0, weight_on_output=True)
    want = torch.zeros(top, t, k, device=DEV)
    for j in range(top):
        for e in range(experts):
            rows = (chosen[:, j] == e).nonzero().view(-1)
            if rows.numel():
                gu = x[rows].float() @ gate_up[e].float().T
                h = (gu[:, :f] * torch.sigmoid(gu[:, :f]) * gu[:, f:])
                if dtype == torch.bfloat16:
                    h = h.to(dtype).float()
                want[j, rows] = weight[rows, j: j + 1] * (h @ down[e].float().T)
    assert rel(out.cpu(), want.cpu()) < (1e-5 if dtype == torch.float32 else 1e-2)
    sg = rnd(k, seed=6, scale=0.3)
    shared = rnd(t, k, seed=7)
    got = shared.clone()
    ops.row_gate(got, x, sg)
    assert rel(got.cpu(), (shared * torch.sigmoid(x.float() @ sg)[:, None]).cpu()) < 1e-5


# ------------------------------------------------------------------ whole models

LENGTHS = [70, 33, 97, 18, 64, 45, 1, 52, 2, 81, 29, 3]


def bf16_bars(folder, truth, reqs, last=0):
    """(median, ninth decile, 99th percentile) of the rows (the ``last`` ones of each request, or all) of a
    plain bfloat16 run against the plain model in float64."""
    rough = plain.PlainLarupel.from_dir(folder, bf16=True)
    rows = np.concatenate([np.abs(rough.logits(t)[-last:] - w[-last:]).max(-1) / np.abs(w[-last:]).max(-1) for t, w in zip(reqs, truth)])
    return tuple(float(np.quantile(rows, q)) for q in (0.5, 0.9, 0.99))


def check_rows(errors, dtype, bars=None):
    if dtype == "float32":
        assert max(errors) < F32_TOL, max(errors)
    else:
        e = np.asarray(errors)
        far = int((e > BF16_FAR_FACTOR * bars[2]).sum())
        assert np.isfinite(e).all() and np.median(e) < BF16_FACTOR * bars[0] and np.quantile(e, 0.9) < BF16_TAIL_FACTOR * bars[1] \
            and far <= max(1, BF16_FAR_SHARE * len(e)), (float(np.median(e)), float(np.quantile(e, 0.9)), far, len(e), bars, float(e.max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(LARUPEL))
def test_every_cutting_matches_the_plain_model(name, dtype, folders):
    rng = np.random.default_rng(4)
    reqs = [rng.integers(0, LARUPEL[name]["vocab"], n).tolist() for n in LENGTHS]
    pm = plain.PlainLarupel.from_dir(folders[name])
    truth = [pm.logits(t) for t in reqs]
    bars = bf16_bars(folders[name], truth, reqs) if dtype == "bfloat16" else None
    runner = runner_for(folders[name], 32, dtype)
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        errors: list = []
        traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, 1.0, errors)
        check_rows(errors, dtype, bars)
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=2)
    small = runner_for(folders[name], peak // 16, dtype, slots=3)
    for t in small.pools.tensors:
        t.fill_(3e4)                                        # a page that is used again never holds zeros
    for s in small.states.values():
        s.fill_(1e30)
    rp = TraceReplayer(small)
    errors = []
    traces.compare(rp.run_step, steps, expect, truth, 1.0, errors)
    check_rows(errors, dtype, bars)
    assert all(rp.cache.num_free(g) == peak // 16 for g in range(rp.cache.num_groups))


def test_cuttings_agree_with_each_other_in_32_bit(folders):
    """A position's 32-bit logits do not depend on how its prompt was cut, beyond rounding."""
    toks = np.random.default_rng(8).integers(0, 70, 90).tolist()
    runner = runner_for(folders["C"], 16, "float32")
    rows = {}
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build([toks])
        rp = TraceReplayer(runner)
        got = np.concatenate([r for r in (rp.run_step(s) for s in steps) if r is not None])
        rows[build.__name__] = {p: got[k] for k, (_, p) in enumerate(e for exp in expect for e in exp)}
    for p in rows["decode_tail"]:
        assert rel(rows["decode_tail"][p], rows["whole"][p]) < 2e-5 and rel(rows["portions"][p], rows["whole"][p]) < 2e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_contexts_and_far_keys(dtype, tmp_path):
    """2,100 keys, so that the decode attention and the attention of a short portion cut their keys
    into runs, under a score scale with which single keys hundreds of tokens back carry the weight;
    a reader of the same keys behind it; and both delta rules over as many tokens with slow decays."""
    def slow(tensors):
        for name, t in tensors.items():
            if name.endswith(".A_log"):
                t.fill_(-5.0)
            if name.endswith(".w0"):
                t.fill_(-4.0)

    cfgs = [model(80, 64, 1e-5, [layer(attention(4, 2, 32, 32, 3.0), dense(32)), layer(attention(4, 2, 32, 32, 3.0, kv_from=0), None)]),
            model(80, 64, 1e-5, [layer(delta(2, 1, 16, 24, 4), dense(32)), layer(general_delta(2, 24, 6), None)])]
    for k, cfg in enumerate(cfgs):
        folder = write_larupel(tmp_path / f"m{k}", cfg, seed=3 + k, std=0.3, edit=slow)
        toks = np.random.default_rng(5).integers(0, 80, 2110).tolist()
        pm = plain.PlainLarupel.from_dir(folder)
        truth = pm.logits(toks)
        runner = runner_for(folder, 140, dtype)
        steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:2080], "want": [100, 2079]}], "end": []},
                 {"step": 1, "entries": [{"id": "a", "tokens": toks[2080:2100], "want": list(range(20))}], "end": []}]
        steps += [{"step": 2 + i, "entries": [{"id": "a", "tokens": [toks[2100 + i]], "want": [0]}], "end": []} for i in range(10)]
        expect = [[(0, 100), (0, 2079)], [(0, p) for p in range(2080, 2100)]] + [[(0, 2100 + i)] for i in range(10)]
        errors: list = []
        traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], 1.0, errors)
        check_rows(errors, dtype, bf16_bars(folder, [truth], [toks], last=40) if dtype == "bfloat16" else None)
        far = np.abs(pm.logits(toks[1500:])[-1] - truth[-1]).max() / np.abs(truth[-1]).max()
        assert far > 100 * F32_TOL                          # what lies far back matters to the last row


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_at_the_kernels_limits(dtype, tmp_path):
    """Keys of 256 in both delta rules (sixteen state entries per lane), a value head of 200, sixteen
    taps, an attention head of 256 beside a value of 40, 64 experts of which one is used."""
    cfg = model(90, 128, 1e-5, [layer(delta(2, 1, 256, 200, 16), moe(64, 1, 16)), layer(general_delta(1, 256, 32), None),
                                layer(attention(2, 1, 256, 40, 0.05), dense(40))])
    folder = write_larupel(tmp_path, cfg, seed=9)
    toks = np.random.default_rng(5).integers(0, 90, 60).tolist()
    truth = plain.PlainLarupel.from_dir(folder).logits(toks)
    steps, expect = traces.decode_tail([toks], tail=12)
    errors: list = []
    traces.compare(TraceReplayer(runner_for(folder, 8, dtype)).run_step, steps, expect, [truth], 1.0, errors)
    check_rows(errors, dtype, bf16_bars(folder, [truth], [toks]) if dtype == "bfloat16" else None)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_multiples_of_nothing(dtype, tmp_path):
    """A width of 90, a vocabulary of 77, inner sizes of 50, 13 and 7, heads of 5, 9 and 11 numbers, a rank
    of 3: the products' and the norms' narrow forms, rows that start at odd addresses."""
    cfg = model(77, 90, 1e-6, [layer(delta(3, 1, 5, 9, 2), moe(3, 2, 13, shared=7)), layer(attention(3, 3, 11, 5, 0.4), dense(50)),
                               layer(general_delta(2, 9, 3), moe(5, 5, 7)), layer(attention(3, 3, 11, 5, 0.4, kv_from=1), None)])
    folder = write_larupel(tmp_path, cfg, seed=13)
    rng = np.random.default_rng(5)
    reqs = [rng.integers(0, 77, n).tolist() for n in (75, 40, 9)]
    pm = plain.PlainLarupel.from_dir(folder)
    truth = [pm.logits(t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=1)
    errors: list = []
    traces.compare(TraceReplayer(runner_for(folder, peak // 16, dtype, slots=3)).run_step, steps, expect, truth, 1.0, errors)
    check_rows(errors, dtype, bf16_bars(folder, truth, reqs) if dtype == "bfloat16" else None)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_through_graphs(dtype, folders):
    """The delta rules' kernels read slots and item boundaries from device memory, so decode steps are
    captured; the capture puts the state back before its first replay. Two requests decode side by
    side, then one alone (another graph), in slots that held junk."""
    rng = np.random.default_rng(3)
    reqs = [rng.integers(0, 96, n).tolist() for n in (60, 75)]
    pm = plain.PlainLarupel.from_dir(folders["A"])
    truth = [pm.logits(t) for t in reqs]
    runner = runner_for(folders["A"], 16, dtype, graphs=True)
    assert runner.use_graphs and runner.states
    for s in runner.states.values():
        s.fill_(1e30)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": reqs[0][:20], "want": [19]}, {"id": "b", "tokens": reqs[1][:31], "want": [30]}], "end": []}]
    expect = [[(0, 19), (1, 30)]]
    for k in range(40):
        steps.append({"step": len(steps), "entries": [{"id": "a", "tokens": [reqs[0][20 + k]], "want": [0]},
                                                     {"id": "b", "tokens": [reqs[1][31 + k]], "want": [0]}], "end": ["a"] if k == 39 else []})
        expect.append([(0, 20 + k), (1, 31 + k)])
    for k in range(71, 75):
        steps.append({"step": len(steps), "entries": [{"id": "b", "tokens": [reqs[1][k]], "want": [0]}], "end": ["b"] if k == 74 else []})
        expect.append([(1, k)])
    errors: list = []
    traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, 1.0, errors)
    check_rows(errors, dtype, bf16_bars(folders["A"], truth, reqs) if dtype == "bfloat16" else None)
    assert len(runner._graphs) == 2


def test_greedy_generation_through_the_entry_point(folders):
    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import generate

    pm = plain.PlainLarupel.from_dir(folders["A"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 96, n).tolist() for n in (5, 23, 40, 9, 31)]
    eng = Engine(EngineConfig(model_path=str(folders["A"]), dtype="float32", max_num_seqs=3, max_prefill_tokens=16,
                              max_seq_len=128, num_blocks=14))
    outs, _ = generate(eng, prompts, 12, temperature=0.0, ignore_eos=True)
    for p, o in zip(prompts, outs):
        assert list(o.tokens) == pm.greedy(p, 12)


def test_trace_run_and_the_command_line_as_programs(folders, tmp_path):
    rng = np.random.default_rng(7)
    reqs = [rng.integers(0, 130, n).tolist() for n in (40, 70, 25, 90, 33)]
    pm = plain.PlainLarupel.from_dir(folders["B"])
    truth = [pm.logits(t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=5)
    env = {k: v for k, v in os.environ.items()}
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out-{dtype}"
        proc = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(folders["B"]), "--dtype", dtype, "--out", str(out),
                               "--max-tokens", str(peak)], input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                              capture_output=True, env=env, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        errors = []
        for s, exp in zip(steps, expect):
            if exp:
                got = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(exp), -1)
                errors += [rel(row, truth[i][p]) for row, (i, p) in zip(got, exp)]
        check_rows(errors, dtype, bf16_bars(folders["B"], truth, reqs) if dtype == "bfloat16" else None)
    prompt = [5, 17, 3, 90, 41, 7, 7, 19, 0, 64, 11]
    proc = subprocess.run(
        [sys.executable, "-m", "prefixserve_amd.cli", "generate", "--model", str(folders["B"]), "--dtype", "float32",
         "--max-seq-len", "128", "--num-blocks", "16", "--max-running-requests", "2", "--chunked-prefill-size", "5",
         "--max-tokens", "6", "--ignore-eos", "--prompt-ids", ",".join(map(str, prompt))],
        capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert json.loads(proc.stdout.strip().splitlines()[-1])["outputs"][0]["tokens"] == pm.greedy(prompt, 6)


def random_larupel(rng) -> dict:
    """A configuration drawn at random: widths that are no multiples of 16, two to six layers of every
    kind in any order, readers of earlier attention layers, every kind of feed-forward or none."""
    width = int(rng.choice([40, 72, 100, 136]))
    layers, sources = [], {}
    for i in range(int(rng.integers(2, 7))):
        kind = int(rng.integers(0, 4))
        if kind == 3 and not sources:
            kind = 2
        if kind == 0:
            g = int(rng.choice([1, 2, 3]))
            mixer = delta(g * int(rng.choice([1, 2, 4])), g, int(rng.choice([4, 16, 24, 64, 100])), int(rng.choice([6, 16, 40, 64])),
                          int(rng.choice([1, 2, 4, 6])))
        elif kind == 1:
            mixer = general_delta(int(rng.choice([1, 2, 5])), int(rng.choice([8, 20, 64, 72])), int(rng.choice([1, 4, 16, 40])))
        elif kind == 2:
            g = int(rng.choice([1, 2, 3]))
            sizes = dict(heads=g * int(rng.choice([1, 2, 4])), kv_heads=g, dim=int(rng.choice([8, 20, 32, 48, 72])),
                         vdim=int(rng.choice([8, 16, 40, 64])), scale=float(rng.choice([0.05, 0.3, 1.0])))
            sources[i] = sizes
            mixer = attention(**sizes)
        else:
            j = int(rng.choice(sorted(sources)))
            mixer = attention(**sources[j], kv_from=j)
        ff = int(rng.integers(0, 4))
        experts = int(rng.choice([2, 5, 8, 16]))
        mlp = (None, dense(int(rng.choice([12, 40, 64]))), moe(experts, int(rng.integers(1, experts + 1)), int(rng.choice([8, 24, 40]))),
               moe(experts, int(rng.integers(1, experts + 1)), int(rng.choice([8, 24, 40])), shared=int(rng.choice([8, 20, 64]))))[ff]
        layers.append(layer(mixer, mlp))
    return model(int(rng.choice([50, 131, 256])), width, float(rng.choice([1e-5, 1e-6])), layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_in_both_dtypes(seed, tmp_path):
    rng = np.random.default_rng(200 + seed)
    cfg = random_larupel(rng)
    folder = write_larupel(tmp_path, cfg, seed=seed)
    reqs = [rng.integers(0, cfg["vocab"], n).tolist() for n in (90, 17, 45, 3)]
    pm = plain.PlainLarupel.from_dir(folder)
    truth = [pm.logits(t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=seed)
    for dtype in ("float32", "bfloat16"):
        errors: list = []
        traces.compare(TraceReplayer(runner_for(folder, peak // 16, dtype, slots=3)).run_step, steps, expect, truth, 1.0, errors)
        if dtype == "float32":
            assert max(errors) < F32_TOL, (cfg, max(errors))
        else:
            check_rows(errors, dtype, bf16_bars(folder, truth, reqs))
