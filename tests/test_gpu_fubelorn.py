"""Fubelorn on the GPU: the kernels it brought, each against the same computation in plain float32 torch
(the host stand-in of the kernel library, which is nothing else), and the model in both dtypes against
the plain implementation in tests/plain/fubelorn_plain.py: every cutting, mixed batches on reused pages
and slots, windows and pooled blocks long enough for the attention kernel's rounds of keys, captured
decode steps, generation, and the programs a user starts."""

from __future__ import annotations

import json
import os
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces
from emulated_ops import EmulatedOps
from fubelorn_configs import FUBELORN, attention, delta, layer, mamba2, memory, model, side_by_side, write_fubelorn
from plain import fubelorn_plain as plain
from prefixserve_amd.engine.batch import GroupMeta, StepItem, StepPacker
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent
DEV = "cuda:0"
F32_TOL = 1e-4
# bfloat16: a row's largest error over its largest logit, against the plain model with its products and
# activations rounded to bfloat16: the median and the ninth decile of a trace's rows, and how many lie far out.
BF16_FACTOR, BF16_TAIL_FACTOR, BF16_FAR_FACTOR, BF16_FAR_SHARE = 1.5, 2.5, 2.0, 0.03


@pytest.fixture(scope="module")
def ops():
    from prefixserve_amd.kernels.ops import HipOps
    from prefixserve_amd.parts.base import Workspace

    return HipOps(torch.device(DEV), Workspace(torch.device(DEV)))


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_fubelorn(tmp_path_factory.mktemp(f"fubelorn-{name}"), name) for name in FUBELORN}


class _OnDevice:
    """The host stand-in with its new tensors made on the device."""

    def __init__(self, inner):
        self.inner = inner

    def __getattr__(self, name):
        fn = getattr(self.inner, name)

        def call(*args, **kwargs):
            with torch.device(DEV):
                return fn(*args, **kwargs)

        return call


PLAIN = _OnDevice(EmulatedOps(DEV))


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def rel(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    if want.size == 0:
        return 0.0
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-30))


def same(got, want, dtype=torch.float32):
    return rel(got.float().cpu(), want.float().cpu()) < (2e-5 if dtype == torch.float32 else 1e-2)


def runner_for(folder, pages, dtype, slots=4, graphs=False):
    return ModelRunner(folder, dtype=dtype, device=DEV, num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=slots,
                       use_graphs=graphs)


class Step:
    """The few fields of a step's context that the recurrences' kernels read."""

    def __init__(self, lengths, slots):
        starts = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
        self.num_tokens, self.num_items = int(starts[-1]), len(lengths)
        self.item_start = torch.tensor(starts, device=DEV)
        self.slots = torch.tensor(slots, dtype=torch.int32, device=DEV)
        self.tok_item = torch.tensor(np.repeat(np.arange(len(lengths)), lengths).astype(np.int32), device=DEV)


# ------------------------------------------------------------------ kernels

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("s,t,h", [(1, 1, 64), (4, 7, 100), (3, 130, 72), (16, 9, 30), (2, 3, 2049)])
def test_streams_are_read_and_written(ops, dtype, s, t, h):
    streams = rnd(s, t, h, seed=1, scale=2.0)
    read, write, mix = rnd(s, seed=2), rnd(s, seed=3), rnd(s, s, seed=4, scale=0.5) + torch.eye(s, device=DEV)
    weight, factor = rnd(h, seed=5, scale=0.2) + 1.0, rnd(h, seed=6)
    for fac in (None, factor):
        for out_dtype in (torch.float32, dtype):
            got, want = (torch.empty(t, h, dtype=out_dtype, device=DEV) for _ in range(2))
            ops.hyper_read(streams, read, weight, 1e-5, got, factor=fac)
            PLAIN.hyper_read(streams, read, weight, 1e-5, want, factor=fac)
            assert same(got, want, out_dtype)
    for delta_rows in (rnd(t, h, dtype=dtype, seed=7), rnd(3, t, h, seed=8), rnd(1, t, h, seed=9)):
        got, want = streams.clone(), streams.clone()
        ops.hyper_write(got, mix, write, delta_rows)
        PLAIN.hyper_write(want, mix, write, delta_rows)
        assert same(got, want)
    a, b = rnd(t, h, dtype=dtype, seed=10), rnd(2, t, h, seed=11)
    got, want = streams.clone(), streams.clone()
    ops.hyper_write(got, mix, write, a, 0.8, b, -1.5)                      # the weighted sum of two outputs
    PLAIN.hyper_write(want, mix, write, a, 0.8, b, -1.5)
    assert same(got, want)
    got, want = (torch.empty(t, h, device=DEV) for _ in range(2))
    ops.weighted_sum(a, 0.8, b, -1.5, got)
    PLAIN.weighted_sum(a, 0.8, b, -1.5, want)
    assert same(got, want)
    x = rnd(t, h, seed=12, scale=3.0)
    got = x.clone()
    ops.stream_rms_norm(got, weight, 1e-6)
    assert same(got, weight * x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_activations_in_place(ops, dtype):
    x = rnd(37, 101, dtype=dtype, seed=1, scale=2.5)
    for kind in ("gelu", "gelu_tanh", "silu", "relu"):
        got, want = x.clone(), x.clone()
        ops.activation(got, kind)
        PLAIN.activation(want, kind)
        assert same(got, want, dtype)
    z = torch.linspace(-6, 6, 1001, device=DEV)
    got = z.clone()
    ops.activation(got, "gelu")
    assert float((got.double() - 0.5 * z.double() * (1 + torch.erf(z.double() / 2 ** 0.5))).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,channels", [(1, 40), (4, 320), (3, 77), (16, 9)])
def test_convolution_with_a_bias_and_an_output_of_either_type(ops, dtype, taps, channels):
    """Float rows into rows of the activation type (what a sub-layer reads), and rows of the activation type with a bias
    into float rows (the state space layer's), continued from a slot: a single token, fewer than taps, a long portion."""
    w, bias = rnd(channels, taps, seed=1, scale=0.5), rnd(channels, seed=2)
    tail = (taps - 1) * channels
    for rows_dtype, out_dtype, b, silu in ((torch.float32, dtype, None, False), (dtype, torch.float32, bias, True)):
        got_state = torch.full((3, 5 + tail + 3), 1e30, device=DEV)
        got_state[:, 5: 5 + tail] = rnd(3, tail, seed=3)
        want_state = got_state.clone()
        for k, lengths in enumerate([(1, 2, 40), (3, 1, 1), (70, 2, 5)]):
            step = Step(lengths, [2, 0, 1])
            rows = rnd(step.num_tokens, channels + 6, dtype=rows_dtype, seed=10 + k)
            got, want = (torch.empty(step.num_tokens, channels, dtype=out_dtype, device=DEV) for _ in range(2))
            ops.short_conv(rows, 4, w, got, got_state, 5, step, silu=silu, bias=b)
            PLAIN.short_conv(rows, 4, w, want, want_state, 5, step, silu=silu, bias=b)
            assert same(got, want, out_dtype) and same(got_state[:, 5: 5 + tail], want_state[:, 5: 5 + tail])
        assert bool((got_state[:, :5] == 1e30).all()) and bool((got_state[:, 5 + tail:] == 1e30).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim,n,groups,parts", [(4, 8, 12, 2, 2), (1, 20, 3, 1, 1), (8, 64, 128, 1, 4), (6, 10, 256, 3, 5)])
def test_state_space_layer_through_the_delta_scan(ops, dtype, heads, vdim, n, groups, parts):
    """Step sizes and decays, the recurrence over three steps from slots of junk, the skip, gate and norm in parts."""
    inner, ch = heads * vdim, heads * vdim + 2 * groups * n
    dt_bias, a_log, skip, norm_w = rnd(heads, seed=1), rnd(heads, seed=2, scale=0.5) - 1.0, rnd(heads, seed=3), rnd(inner, seed=4, scale=0.2) + 1.0
    got_state = torch.full((3, 7 + inner * n), 1e30, device=DEV)
    got_state[:, 7:] = 0.0
    want_state = got_state.clone()
    for k, lengths in enumerate([(33, 2), (1, 1), (5, 70)]):
        step = Step(lengths, [2, 0])
        t = step.num_tokens
        u, dt, z = rnd(t, ch, seed=10 + k), rnd(t, heads, seed=20 + k), rnd(t, inner + 3, dtype=dtype, seed=30 + k)
        outs = []
        for o, state in ((ops, got_state), (PLAIN, want_state)):
            coef = torch.empty(t, 3 * heads, device=DEV)
            o.state_space_prepare(dt, dt_bias, a_log, coef)
            y = torch.empty(t, inner, device=DEV)
            o.delta_scan(keys=(u, inner), directions=(u, inner), removals=(u, inner), queries=(u, inner + groups * n),
                         key_groups=groups, decay_vectors=None, decay=(coef, 0), removal_scale=(coef, heads), value_scale=(coef, 2 * heads),
                         values=(u, 0), out=y, state=state, state_offset=7, ctx=step, heads=heads, dim=n, vdim=vdim, reads_decayed=True, no_removal=True)
            out = torch.empty(t, inner, dtype=dtype, device=DEV)
            o.gated_group_norm(y, u, 0, skip, heads, z, 3, norm_w, parts, 1e-5, out)
            outs.append((coef, y, out))
        assert same(outs[0][0], outs[1][0]) and same(outs[0][1], outs[1][1]) and same(outs[0][2], outs[1][2], dtype)
        assert same(got_state[[0, 2], 7:], want_state[[0, 2], 7:])
    assert bool((got_state[:, :7] == 1e30).all())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim,cap", [(2, 12, 8, 10.0), (1, 18, 5, 2.0), (4, 64, 64, 15.0), (3, 256, 15, 30.0)])
def test_matrix_memory_through_the_delta_scan(ops, dtype, heads, dim, vdim, cap):
    """Gates with their running maximum, operands, the recurrence with n as one more column, and the read-out with its
    denominator, norm and gate, over three steps from slots of junk."""
    ks, vs, vd = heads * dim, heads * vdim, vdim + 1
    bias, norm_w = rnd(2 * heads, seed=1), rnd(vs, seed=2, scale=0.2) + 1.0
    size = heads * vd * dim + heads
    got_state = torch.full((3, 4 + size), 1e30, device=DEV)
    got_state[:, 4:] = 0.0
    want_state = got_state.clone()
    for k, lengths in enumerate([(40, 3), (1, 1), (2, 66)]):
        step = Step(lengths, [1, 2])
        t = step.num_tokens
        rows, gates = rnd(t, 2 * ks + 2 * vs, dtype=dtype, seed=10 + k), rnd(t, 2 * heads, seed=20 + k, scale=3.0)
        outs = []
        for o, state in ((ops, got_state), (PLAIN, want_state)):
            coef = torch.empty(t, 4 * heads, device=DEV)
            o.matrix_memory_gates(gates, bias, cap, coef, state, 4 + heads * vd * dim, step)
            u, vals = torch.empty(t, 2 * ks, device=DEV), torch.empty(t, heads * vd, device=DEV)
            o.matrix_memory_operands(rows, 0, ks, 2 * ks, heads, dim, vdim, dim ** -0.5, u, vals)
            raw = torch.empty(t, heads * vd, device=DEV)
            o.delta_scan(keys=(u, ks), directions=(u, ks), removals=(u, ks), queries=(u, 0), key_groups=heads, decay_vectors=None,
                         decay=(coef, 0), removal_scale=(coef, heads), value_scale=(coef, 2 * heads), values=(vals, 0), out=raw,
                         state=state, state_offset=4, ctx=step, heads=heads, dim=dim, vdim=vd, reads_decayed=True, no_removal=True)
            out = torch.empty(t, vs, dtype=dtype, device=DEV)
            o.memory_read_norm_gate(raw, coef, 3 * heads, heads, vdim, 1e-6, norm_w, 1e-5, rows, 2 * ks + vs, out)
            outs.append((coef, u, vals, raw, out))
        for a, b in zip(outs[0][:4], outs[1][:4]):
            assert same(a, b)
        assert same(outs[0][4], outs[1][4], dtype)
        assert same(got_state[[1, 2], 4:], want_state[[1, 2], 4:])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d,window,keep,block", [(4, 2, 32, 9, 0, 4), (3, 3, 16, 6, 3, 0), (2, 1, 48, 70, 20, 16), (2, 2, 64, 3, 0, 7),
                                                        (8, 2, 128, 40, 18, 1), (2, 1, 160, 30, 3, 5), (4, 2, 192, 50, 8, 12), (1, 1, 512, 5, 2, 3)])
def test_attention_with_kept_tokens_pooled_blocks_and_a_gate(ops, dtype, hq, hkv, d, window, keep, block):
    """Block means are written as their last token runs; then a portion, a single token and a new request see the window,
    the kept first tokens and the blocks wholly in front of the window, from pages in a scrambled order."""
    pages = 24
    win = max(window, block) if block else window
    packer = StepPacker(torch.device(DEV), [GroupMeta(pages, win, keep, 1), GroupMeta(pages, None, 0, max(block, 1))], 100, pages * 16, 4, 64)
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(5)).tolist()
    tables = {0: [order[:14], order[10:]], 1: [order[14:][::-1], order[:10][::-1]]}      # 191 and 128 tokens at most
    kv = [rnd(pages, 2, hkv, 16 * d, dtype=dtype, seed=1) for _ in range(2)]
    pool = [torch.full((pages, 2, hkv, 16 * d), 3e4, dtype=dtype, device=DEV) for _ in range(2)]
    done = {0: 0, 1: 0}
    for k, portions in enumerate([{0: 150}, {0: 1, 1: 37}, {0: 40, 1: 1}, {1: 90}]):
        items = [StepItem(key=r, tokens=[1] * n, start=done[r], block_tables=tables[r], slot=r, want=[]) for r, n in portions.items()]
        ctx = packer.pack(items)
        torch.cuda.synchronize()
        t = ctx.num_tokens
        qkv = rnd(t, hq * d + 5, dtype=dtype, seed=20 + k, scale=0.5)
        gate = rnd(t, hq, seed=30 + k)
        outs = []
        for o, pl in ((ops, pool[0]), (PLAIN, pool[1])):
            if block:
                o.pool_kv_append(kv[0], pl, ctx, 0, 1, hkv, d, block)
            out = torch.empty(t, hq * d, dtype=dtype, device=DEV)
            o.paged_attention(qkv, out, kv[0], ctx, 0, hq, hkv, d, 0.4, window, keep_first=keep, exact_weights=k >= 2,
                              pooled=(pl, 1, block) if block else None, head_gate=gate if k % 2 == 0 else None)
            outs.append(out)
        assert same(outs[0], outs[1], dtype), (k, rel(outs[0].float().cpu(), outs[1].float().cpu()))
        if block:
            assert same(pool[0], pool[1], dtype)
        for r, n in portions.items():
            done[r] += n


# ------------------------------------------------------------------ whole models

LENGTHS = [70, 33, 97, 18, 64, 45, 1, 52, 2, 81, 29, 3]


def truth_of(folder, toks, **kw):
    cfg, tensors = plain.load(folder)
    return plain.forward(cfg, tensors, toks, **kw)


def bf16_bars(folder, truth, reqs, last=10 ** 9):
    rows = np.concatenate([np.abs(truth_of(folder, t, bf16=True)[-last:] - w[-last:]).max(-1) / np.abs(w[-last:]).max(-1)
                           for t, w in zip(reqs, truth)])
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
@pytest.mark.parametrize("name", list(FUBELORN))
def test_every_cutting_matches_the_plain_model(name, dtype, folders):
    rng = np.random.default_rng(4)
    lengths = LENGTHS + ([190] if name == "C" else [])
    reqs = [rng.integers(0, FUBELORN[name]["vocab"], n).tolist() for n in lengths]
    truth = [truth_of(folders[name], t) for t in reqs]
    bars = bf16_bars(folders[name], truth, reqs) if dtype == "bfloat16" else None
    runner = runner_for(folders[name], 40, dtype)
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
    toks = np.random.default_rng(8).integers(0, 64, 150).tolist()
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
def test_long_contexts_windows_and_blocks_of_real_sizes(dtype, tmp_path):
    """1,300 tokens through a window of 200 that keeps 40 first tokens and one of 300 with blocks of 32, heads of 64,
    slow decays: a long portion, a short one, single tokens; what lies far back matters to the last rows."""
    def slow(tensors):
        for name, t in tensors.items():
            if name.endswith(".A_log"):
                t.fill_(-5.0)
            if name.endswith(".f.b"):
                t.fill_(5.0)
            if name.endswith("left.q") or name.endswith("left.k"):
                # single keys carry the first layer's softmax (a kept token can); the last layer's is flat, so that
                # the means over blocks, which are short vectors, have their share
                t.mul_(3.0 if name.startswith("l0.") else 0.2)

    cfg = model(80, 64, 1e-5, [
        layer(side_by_side("parallel", attention(4, 2, 64, 64, 0.5, 200, keep_first=40), delta(2, 1, 16, 24, 4), 1.0, 0.5), 32),
        layer(mamba2(2, 32, 64, 1, 4, 1), None),
        layer(side_by_side("parallel_2", attention(4, 2, 64, 32, 0.2, 300, pool=32, rot={"dims": 32, "base": 10000.0}),
                           memory(2, 32, 32, 15.0), 1.0, 0.5), 32),
    ], streams=2, taps=4, mult=0.5)
    folder = write_fubelorn(tmp_path, cfg, seed=3, std=0.3, edit=slow)
    toks = np.random.default_rng(5).integers(0, 80, 1310).tolist()
    raw, tensors = plain.load(folder)
    truth = plain.forward(raw, tensors, toks)
    runner = runner_for(folder, 90, dtype)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:1280], "want": [100, 1279]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[1280:1300], "want": list(range(20))}], "end": []}]
    steps += [{"step": 2 + i, "entries": [{"id": "a", "tokens": [toks[1300 + i]], "want": [0]}], "end": []} for i in range(10)]
    expect = [[(0, 100), (0, 1279)], [(0, p) for p in range(1280, 1300)]] + [[(0, 1300 + i)] for i in range(10)]
    errors: list = []
    traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], 1.0, errors)
    check_rows(errors, dtype, bf16_bars(folder, [truth], [toks], last=40) if dtype == "bfloat16" else None)
    for i, key in ((0, "keep_first"), (2, "pool")):
        other = json.loads(json.dumps(raw))
        other["layers"][i]["mixer"]["left"]["mask"][key] = 0
        assert rel(plain.forward(other, tensors, toks)[-1], truth[-1]) > 50 * F32_TOL


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sizes_that_are_multiples_of_nothing(dtype, tmp_path):
    """A width of 90, a vocabulary of 77, inner sizes of 50 and 13, heads of 5, 9 and 11 numbers, a state of 7, a block of 5."""
    cfg = model(77, 90, 1e-6, [
        layer(mamba2(3, 5, 7, 3, 2, 3), 13),
        layer(side_by_side("parallel_2", attention(3, 3, 11, 5, 0.4, 13, pool=5, rot={"dims": 6, "base": 77.0}), memory(2, 9, 5, 3.0), 0.9, 1.1), 50),
        layer(side_by_side("parallel", attention(3, 1, 9, 11, 0.4, 7, keep_first=5), delta(3, 1, 5, 9, 2), 1.2, 0.4), None),
    ], streams=5, taps=2, mult=0.3)
    folder = write_fubelorn(tmp_path, cfg, seed=13)
    rng = np.random.default_rng(5)
    reqs = [rng.integers(0, 77, n).tolist() for n in (75, 40, 9)]
    truth = [truth_of(folder, t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=1)
    errors: list = []
    traces.compare(TraceReplayer(runner_for(folder, peak // 16, dtype, slots=3)).run_step, steps, expect, truth, 1.0, errors)
    check_rows(errors, dtype, bf16_bars(folder, truth, reqs) if dtype == "bfloat16" else None)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_through_graphs(dtype, folders):
    """Every kernel of the design reads slots, positions and tables from device memory, so decode steps are captured;
    the capture puts the state back before its first replay. Two requests decode side by side, then one alone
    (another graph), in slots that held junk; blocks are completed and windows pass page borders on the way."""
    rng = np.random.default_rng(3)
    reqs = [rng.integers(0, 90, n).tolist() for n in (60, 75)]
    truth = [truth_of(folders["A"], t) for t in reqs]
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

    cfg, tensors = plain.load(folders["A"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 90, n).tolist() for n in (5, 23, 40, 9, 31)]
    eng = Engine(EngineConfig(model_path=str(folders["A"]), dtype="float32", max_num_seqs=3, max_prefill_tokens=16,
                              max_seq_len=128, num_blocks=14))
    outs, _ = generate(eng, prompts, 12, temperature=0.0, ignore_eos=True)
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(np.argmax(plain.forward(cfg, tensors, seq)[-1])))
        assert list(o.tokens) == seq[len(p):]


def test_trace_run_and_the_command_line_as_programs(folders, tmp_path):
    rng = np.random.default_rng(7)
    reqs = [rng.integers(0, 64, n).tolist() for n in (40, 170, 25, 90, 33)]
    truth = [truth_of(folders["C"], t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=5)
    env = {k: v for k, v in os.environ.items()}
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out-{dtype}"
        proc = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(folders["C"]), "--dtype", dtype, "--out", str(out),
                               "--max-tokens", str(peak)], input="".join(json.dumps(s) + "\n" for s in steps), text=True,
                              capture_output=True, env=env, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        errors = []
        for s, exp in zip(steps, expect):
            if exp:
                got = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(exp), -1)
                errors += [rel(row, truth[i][p]) for row, (i, p) in zip(got, exp)]
        check_rows(errors, dtype, bf16_bars(folders["C"], truth, reqs) if dtype == "bfloat16" else None)
    prompt = [5, 17, 3, 60, 41, 7, 7, 19, 0, 63, 11]
    cfg, tensors = plain.load(folders["C"])
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(np.argmax(plain.forward(cfg, tensors, seq)[-1])))
    proc = subprocess.run(
        [sys.executable, "-m", "prefixserve_amd.cli", "generate", "--model", str(folders["C"]), "--dtype", "float32",
         "--max-seq-len", "128", "--num-blocks", "16", "--max-running-requests", "2", "--chunked-prefill-size", "5",
         "--max-tokens", "6", "--ignore-eos", "--prompt-ids", ",".join(map(str, prompt))],
        capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert json.loads(proc.stdout.strip().splitlines()[-1])["outputs"][0]["tokens"] == seq[len(prompt):]


def random_fubelorn(rng) -> dict:
    """A configuration drawn at random: widths that are no multiples of 16, two to five layers of every kind in any order,
    with and without several streams, taps, kept tokens, blocks, rotation, feed-forwards."""
    width = int(rng.choice([40, 72, 100, 136]))
    layers = []
    for _ in range(int(rng.integers(2, 6))):
        kind = int(rng.integers(0, 3))
        g = int(rng.choice([1, 2, 3]))
        heads, dim, vdim = g * int(rng.choice([1, 2, 4])), int(rng.choice([8, 20, 32, 48, 72])), int(rng.choice([8, 16, 40, 64]))
        size = int(rng.choice([3, 17, 40, 100]))
        if kind == 0:
            groups = int(rng.choice([1, 2]))
            mixer = mamba2(groups * int(rng.choice([1, 3])), int(rng.choice([4, 16, 40])), int(rng.choice([3, 16, 64, 100])), groups,
                           int(rng.choice([1, 2, 4])), 1)
        elif kind == 1:
            keep = int(rng.choice([0, 1, 5, 30]))
            left = attention(heads, g, dim, vdim, float(rng.choice([0.1, 0.3])), size, keep_first=keep if keep else None)
            mixer = side_by_side("parallel", left, delta(g * int(rng.choice([1, 2])), g, int(rng.choice([4, 16, 24, 64])),
                                                         int(rng.choice([6, 16, 40])), int(rng.choice([1, 2, 4]))), 0.9, 0.7)
        else:
            pool = int(rng.choice([0, 1, 6, 16, 50]))
            dims = int(rng.choice([0, 4, dim - dim % 2]))
            rot = {"dims": dims, "base": 1000.0}
            if rng.random() < 0.5:
                rot["scaling"] = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
            left = attention(heads, g, dim, vdim, float(rng.choice([0.1, 0.3])), size, pool=pool if pool else None, rot=rot if dims else None)
            mixer = side_by_side("parallel_2", left, memory(int(rng.choice([1, 2, 5])), int(rng.choice([8, 20, 64])),
                                                            int(rng.choice([8, 24, 40])), float(rng.choice([2.0, 15.0]))), 0.8, 0.5)
        layers.append(layer(mixer, (None, int(rng.choice([12, 40, 64])))[int(rng.integers(0, 2))]))
    streams, taps = int(rng.choice([1, 2, 4])), int(rng.choice([0, 1, 2, 4]))
    return model(int(rng.choice([50, 131, 256])), width, float(rng.choice([1e-5, 1e-6])), layers, streams=streams if streams > 1 else None,
                 taps=taps if taps else None, mult=float(rng.choice([0.3, 1.0])))


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations_in_both_dtypes(seed, tmp_path):
    rng = np.random.default_rng(300 + seed)
    cfg = random_fubelorn(rng)
    folder = write_fubelorn(tmp_path, cfg, seed=seed)
    reqs = [rng.integers(0, cfg["vocab"], n).tolist() for n in (140, 17, 45, 3)]
    truth = [truth_of(folder, t) for t in reqs]
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=seed)
    for dtype in ("float32", "bfloat16"):
        errors: list = []
        traces.compare(TraceReplayer(runner_for(folder, peak // 16, dtype, slots=3)).run_step, steps, expect, truth, 1.0, errors)
        if dtype == "float32":
            assert max(errors) < F32_TOL, (cfg, max(errors))
        else:
            check_rows(errors, dtype, bf16_bars(folder, truth, reqs))
