"""Fubelorn on the host: its configuration, the model built from it, and the whole engine path
(packing, pages of a window that keeps the first tokens, pages of means over blocks, state slots,
several residual streams, replay, scheduler, generation) with the kernel library's CPU stand-in,
against the plain implementation in tests/plain/fubelorn_plain.py."""

from __future__ import annotations

import copy
import math

import numpy as np
import pytest
import torch

import traces
from emulated_ops import EmulatedOps
from fubelorn_configs import FUBELORN, attention, delta, layer, mamba2, memory, model, side_by_side, write_fubelorn
from plain import fubelorn_plain as plain
from prefixserve_amd.cache.manager import CacheManager
from prefixserve_amd.config import UnsupportedModelError
from prefixserve_amd.config.fubelorn import FubelornConfig
from prefixserve_amd.engine.batch import StepItem
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.models.fubelorn import build_fubelorn_spec

# 32-bit against the float64 oracle, per row relative to its largest logit.
TOL = 1e-4


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_fubelorn(tmp_path_factory.mktemp(f"fubelorn-{name}"), name) for name in FUBELORN}


def runner_for(folder, pages, dtype="float32", slots=4):
    return ModelRunner(folder, dtype=dtype, device="cpu", num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=slots,
                       use_graphs=False, ops=EmulatedOps())


def whole(runner, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    rp = TraceReplayer(runner)
    return rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": list(toks), "want": want}], "end": ["a"]})


def truth_of(folder, toks, **kw):
    cfg, tensors = plain.load(folder)
    return plain.forward(cfg, tensors, toks, **kw)


def close(got, want, tol=TOL):
    return float(np.abs(got - want).max()) <= tol * float(np.abs(want).max())


# ------------------------------------------------------------------ configuration and spec

def test_configuration_reads_every_key_and_refuses_what_it_does_not_know():
    cfg = FubelornConfig.from_dicts(FUBELORN["A"])
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps, cfg.streams, cfg.canon_taps, cfg.residual_mult) == (90, 48, 1e-5, 3, 3, 0.4)
    p2, ssm, p1 = (l.mixer for l in cfg.layers)
    a = p2.left
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.window, a.keep_first, a.pool) == (4, 2, 12, 20, 0.3, 9, 0, 4)
    assert (a.rot.dims, a.rot.base, a.rot.scaling.factor, a.rot.scaling.original) == (8, 10000.0, 4.0, 32)
    assert (p2.right.heads, p2.right.dim, p2.right.vdim, p2.right.gate_cap, p2.left_scale, p2.right_scale) == (2, 12, 8, 10.0, 0.8, 0.6)
    assert (ssm.heads, ssm.vdim, ssm.state, ssm.groups, ssm.conv, ssm.norm_groups) == (4, 8, 12, 2, 4, 2)
    assert (p1.left.keep_first, p1.left.window, p1.left.rot, p1.right.kv_heads, p1.right.conv) == (3, 6, None, 2, 2)
    assert cfg.layers[1].mlp is None and cfg.layers[0].mlp.ff == 64
    assert FubelornConfig.from_dicts(cfg.to_config_json()) == cfg
    lean = FubelornConfig.from_dicts(FUBELORN["B"])
    assert (lean.streams, lean.canon_taps, lean.residual_mult) == (1, 0, 1.0)
    for path, value in [(("layers", 0, "type"), "parallel_3"), (("layers", 0, "mlp", "kind"), "glu"), (("layers", 1, "mixer", "window"), 8),
                        (("layers", 0, "mixer", "left", "kv_heads"), 3), (("layers", 0, "mixer", "left", "mask", "size"), 0),
                        (("layers", 0, "mixer", "left", "rot", "dims"), 14), (("layers", 0, "mixer", "left", "rot", "kind"), "x"),
                        (("layers", 1, "mixer", "groups"), 3), (("layers", 1, "mixer", "norm_groups"), 5), (("layers", 2, "mixer", "right", "conv"), 0),
                        (("layers", 0, "mixer", "right", "gate_cap"), 0.0), (("streams",), 0), (("canon", "taps"), 17), (("tie",), True),
                        (("norm", "kind"), "rms")]:
        raw = copy.deepcopy(FUBELORN["A"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(UnsupportedModelError):
            FubelornConfig.from_dicts(raw)


def test_the_spec_lays_out_pages_states_and_streams(folders):
    spec = build_fubelorn_spec(FubelornConfig.from_dicts(FUBELORN["A"]))
    assert spec.streams == 3 and [l.block for l in spec.layers] == ["hyper"] * 3
    runner = runner_for(folders["A"], 8)
    needs = runner.model.cache_needs()
    # layer 0: tokens in a window that outlasts a block of 4 (9 > 4), its pooled means at a stride of 4; layer 2: three kept tokens
    assert (needs[0].window, needs[0].keep_first, needs[0].stride) == (9, 0, 1)
    assert (needs[2].window, needs[2].keep_first) == (6, 3)
    pool = [n for n in needs.values() if n.stride == 4]
    assert len(pool) == 1 and pool[0].window is None and sorted(runner.strides) == [1, 1, 4]
    # a run's state: saved inputs of both sub-layers' convolutions (2 x 2 x 48; the layer without a feed-forward: 1 x 2 x 48),
    # then the mixer's own
    sizes = {i: int(s.shape[1]) for i, s in runner.states.items()}
    assert sizes[0] == 2 * 2 * 48 + 2 * ((8 + 1) * 12 + 1)
    assert sizes[1] == 2 * 48 + 3 * (32 + 2 * 2 * 12) + 4 * 8 * 12
    assert sizes[2] == 2 * 2 * 48 + (2 - 1) * (2 * 2 * 8 + 4 * 6) + 4 * 6 * 8
    lone = runner_for(folders["B"], 8)
    assert lone.spec.streams == 1 and int(lone.states[0].shape[1]) == 2 * 10 * 5      # one tap: no saved inputs at all


def test_a_window_keeps_the_pages_of_the_first_tokens_and_a_stride_group_needs_fewer():
    cache = CacheManager([16, 16], [40, None], keep_first=[20, 0], strides=[1, 16], enable_prefix_cache=False)
    assert [cache.blocks_for_group(1, n) for n in (15, 16, 255, 256, 271, 272)] == [0, 1, 1, 1, 1, 2]
    tables = cache.allocate([10, 1])
    assert tables is not None
    freed = cache.trim_windows(tables, 150)              # first visible position 111: pages 0 .. 5 lie in front, 0 and 1 stay
    assert freed == 4 and tables[0][:7] == [tables[0][0], tables[0][1], -1, -1, -1, -1, tables[0][6]] and tables[0][0] >= 0
    assert cache.trim_windows(tables, 160) == 1 and tables[0][6] == -1
    cache.release(tables)
    assert cache.num_free(0) == 16 and cache.num_free(1) == 16


# ------------------------------------------------------------------ mechanisms of the plain model, entry by entry

def test_plain_functions_follow_their_equations():
    rng = np.random.default_rng(0)
    # convolution: the last column meets the token itself
    h, w = rng.normal(size=(6, 3)), rng.normal(size=(3, 4))
    out = plain.causal_conv(h, w)
    assert np.allclose(out[0], w[:, 3] * h[0]) and np.allclose(out[5], sum(w[:, j] * h[2 + j] for j in range(4)))
    # scaled frequencies: short waves kept, long ones divided, the band between blended
    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f0, f = plain.rotary_frequencies(16, 100.0, None), plain.rotary_frequencies(16, 100.0, sc)
    waves = 2 * math.pi / f0
    assert np.allclose(f[waves < 16], f0[waves < 16]) and np.allclose(f[waves > 64], f0[waves > 64] / 8.0)
    mid = (waves >= 16) & (waves <= 64)
    assert mid.any() and np.all(f[mid] <= f0[mid]) and np.all(f[mid] >= f0[mid] / 8.0)
    # rotation of a part of the head
    x = rng.normal(size=(3, 1, 10))
    y = plain.rotate(x, np.array([0, 5, 9]), 6, f0[:3])
    assert np.allclose(y[0], x[0]) and np.allclose(y[..., 6:], x[..., 6:])
    a = 5 * f0[1]
    assert np.allclose(y[1, 0, 1], x[1, 0, 1] * math.cos(a) - x[1, 0, 4] * math.sin(a))
    assert np.allclose(y[1, 0, 4], x[1, 0, 4] * math.cos(a) + x[1, 0, 1] * math.sin(a))
    # window with kept first tokens and with pooled blocks: query 9, window 3
    q, k, v = rng.normal(size=(10, 1, 4)), rng.normal(size=(10, 1, 4)), rng.normal(size=(10, 1, 2))
    seen = [0, 1, 7, 8, 9]
    s = np.array([q[9, 0] @ k[j, 0] for j in seen]) * 0.5
    p = np.exp(s - s.max())
    assert np.allclose(plain.window_attention(q, k, v, 0.5, 3, keep_first=2)[9, 0], (p / p.sum()) @ v[seen, 0])
    keys = [k[7, 0], k[8, 0], k[9, 0], k[0:3, 0].mean(0), k[3:6, 0].mean(0)]       # block 2 (6 .. 8) is not wholly in front
    vals = [v[7, 0], v[8, 0], v[9, 0], v[0:3, 0].mean(0), v[3:6, 0].mean(0)]
    s = np.array([q[9, 0] @ key for key in keys]) * 0.5
    p = np.exp(s - s.max())
    assert np.allclose(plain.window_attention(q, k, v, 0.5, 3, pool=3)[9, 0], (p / p.sum()) @ np.stack(vals))
    # query 8: block 1 (3 .. 5) ends at 5 = 8 - 3 and is seen, together with the window 6 .. 8 and block 0
    keys = [k[6, 0], k[7, 0], k[8, 0], k[0:3, 0].mean(0), k[3:6, 0].mean(0)]
    vals = [v[6, 0], v[7, 0], v[8, 0], v[0:3, 0].mean(0), v[3:6, 0].mean(0)]
    assert np.allclose(plain.window_attention(q, k, v, 0.5, 3, pool=3)[8, 0],
                       plain.softmax_rows(np.array([q[8, 0] @ key for key in keys]) * 0.5, np.stack(vals)))
    # query 7: block 1 ends at 5 > 7 - 3 and is not seen yet; tokens 3 and 4 are seen by nobody
    assert np.allclose(plain.window_attention(q, k, v, 0.5, 3, pool=3)[7, 0],
                       plain.softmax_rows(np.array([q[7, 0] @ key for key in (k[5, 0], k[6, 0], k[7, 0], k[0:3, 0].mean(0))]) * 0.5,
                                          np.stack([v[5, 0], v[6, 0], v[7, 0], v[0:3, 0].mean(0)])))
    # matrix memory: two tokens by hand
    q, k, v = rng.normal(size=(2, 1, 3)), rng.normal(size=(2, 1, 3)), rng.normal(size=(2, 1, 2))
    il, fl = np.array([[0.3], [-0.2]]), np.array([[-0.5], [-0.1]])
    m1 = max(-0.5 + 0.0, 0.3)
    s1, n1 = math.exp(0.3 - m1) * np.outer(k[0, 0], v[0, 0]), math.exp(0.3 - m1) * k[0, 0]
    m2 = max(-0.1 + m1, -0.2)
    s2 = math.exp(-0.1 + m1 - m2) * s1 + math.exp(-0.2 - m2) * np.outer(k[1, 0], v[1, 0])
    n2 = math.exp(-0.1 + m1 - m2) * n1 + math.exp(-0.2 - m2) * k[1, 0]
    got = plain.matrix_memory(q, k, v, il, fl)
    assert np.allclose(got[0, 0], s1.T @ q[0, 0] / (max(abs(n1 @ q[0, 0]), math.exp(-m1)) + 1e-6))
    assert np.allclose(got[1, 0], s2.T @ q[1, 0] / (max(abs(n2 @ q[1, 0]), math.exp(-m2)) + 1e-6))
    # state space: two tokens by hand, two heads on one group
    x, b, c = rng.normal(size=(2, 2, 3)), rng.normal(size=(2, 1, 4)), rng.normal(size=(2, 1, 4))
    dt, a_log, skip = np.array([[0.5, 0.2], [0.1, 0.9]]), np.array([0.1, -0.3]), np.array([2.0, -1.0])
    got = plain.ssd(x, b, c, dt, a_log, skip)
    s0 = dt[0, 1] * np.outer(b[0, 0], x[0, 1])
    s1 = math.exp(-math.exp(-0.3) * 0.9) * s0 + 0.9 * np.outer(b[1, 0], x[1, 1])
    assert np.allclose(got[1, 1], s1.T @ c[1, 0] - x[1, 1])
    # delta rule: the read-out sees the token's own write
    q, k, v = rng.normal(size=(1, 1, 3)), rng.normal(size=(1, 1, 3)), rng.normal(size=(1, 1, 2))
    assert np.allclose(plain.gated_delta(q, k, v, np.array([[0.7]]), np.array([[0.9]]))[0, 0], (q[0, 0] @ k[0, 0]) * 0.7 * v[0, 0])
    # several streams: every copy from the old ones
    streams = rng.normal(size=(2, 3, 4))
    hc = {"in": np.array([0.5, 2.0]), "out": np.array([1.0, -1.0]), "mix": np.array([[1.0, 0.2], [0.0, 3.0]])}
    new = plain.hyper_sublayer(streams, lambda name: hc[name], 1.5, None, 1e-6, 0.3, lambda h: 2.0 * h, lambda x: x)
    u = 0.5 * streams[0] + 2.0 * streams[1]
    y = 2.0 * 1.5 * u / np.sqrt((u * u).mean(-1, keepdims=True) + 1e-6)
    assert np.allclose(new[0], streams[0] + 0.3 * y) and np.allclose(new[1], 0.2 * streams[0] + 3.0 * streams[1] - 0.3 * y)


# ------------------------------------------------------------------ one mixer at a time

ONE_LAYER = {
    "state-space": mamba2(4, 8, 12, 2, 4, 2),
    "state-space-one-head-one-tap": mamba2(1, 20, 3, 1, 1, 1),
    "window-kept+delta": side_by_side("parallel", attention(3, 3, 8, 12, 0.35, 6, keep_first=3), delta(4, 2, 8, 6, 2), 1.1, 0.5),
    "window-alone+delta-one-head": side_by_side("parallel", attention(1, 1, 24, 8, 0.2, 4), delta(1, 1, 10, 14, 5), 0.5, 2.0),
    "kept-more-than-window+delta": side_by_side("parallel", attention(4, 1, 8, 8, 0.5, 3, keep_first=18), delta(2, 2, 6, 6, 1), 1.0, 1.0),
    "window-pooled+memory": side_by_side("parallel_2", attention(4, 2, 12, 20, 0.3, 9, pool=4,
                                         rot={"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}}),
                                         memory(2, 12, 8, 10.0), 0.8, 0.6),
    "block-longer-than-window+memory-one-head": side_by_side("parallel_2", attention(2, 2, 8, 8, 0.4, 3, pool=7, rot={"dims": 8, "base": 50.0}),
                                                             memory(1, 18, 5, 2.0), 1.0, 1.0),
    "blocks-of-one+memory": side_by_side("parallel_2", attention(2, 1, 8, 10, 0.4, 5, pool=1), memory(3, 4, 4, 30.0), 0.3, 1.5),
}


@pytest.mark.parametrize("kind", list(ONE_LAYER))
@pytest.mark.parametrize("shape", ["plain", "streams", "streams+taps"])
def test_each_mixer_alone(kind, shape, tmp_path):
    """A model of one layer: whatever differs from the plain model is that mixer's (or the block's)."""
    extra = {"plain": {}, "streams": {"streams": 4, "mult": 0.5}, "streams+taps": {"streams": 2, "taps": 4, "mult": 1.5}}[shape]
    ff = None if shape == "plain" else 24
    folder = write_fubelorn(tmp_path, model(50, 32, 1e-5, [layer(ONE_LAYER[kind], ff)], **extra), seed=8)
    toks = np.random.default_rng(1).integers(0, 50, 45).tolist()
    assert close(whole(runner_for(folder, 4), toks), truth_of(folder, toks))


# ------------------------------------------------------------------ whole models

LENGTHS = [70, 33, 97, 18, 64, 45, 1, 52, 2, 81, 29, 3]


@pytest.mark.parametrize("name", list(FUBELORN))
def test_every_cutting_matches_the_plain_model_on_the_host(name, folders):
    rng = np.random.default_rng(4)
    lengths = LENGTHS + ([190] if name == "C" else [])           # past the long window and more than a page of pooled blocks
    reqs = [rng.integers(0, FUBELORN[name]["vocab"], n).tolist() for n in lengths]
    truth = [truth_of(folders[name], t) for t in reqs]
    runner = runner_for(folders[name], 40)
    for build in (traces.whole, traces.decode_tail, traces.portions):
        steps, expect = build(reqs)
        assert traces.compare(TraceReplayer(runner).run_step, steps, expect, truth, TOL) < TOL
    steps, expect, peak = traces.mixed(reqs, max_live=3, seed=2)
    assert sum(len(r) for r in reqs) > 1.3 * peak
    small = runner_for(folders[name], peak // 16, slots=3)
    for t in small.pools.tensors:
        t.fill_(1e30)                                       # a page that is used again never holds zeros
    for s in small.states.values():
        s.fill_(1e30)                                       # nor does a state slot
    rp = TraceReplayer(small)
    assert traces.compare(rp.run_step, steps, expect, truth, TOL) < TOL
    assert all(rp.cache.num_free(g) == peak // 16 for g in range(rp.cache.num_groups))


def test_layers_follow_the_plain_model_one_by_one(folders):
    """The sum of the streams behind every layer: a fault shows in the layer that makes it."""
    toks = np.random.default_rng(9).integers(0, 90, 37).tolist()
    want: list = []
    truth_of(folders["A"], toks, layers_out=want)
    runner = runner_for(folders["A"], 8)
    seen = []
    for blk in runner.model.blocks:
        inner = blk.forward

        def forward(residual, *a, _inner=inner, **kw):
            out = _inner(residual, *a, **kw)
            assert out is None and residual.shape[0] == 3       # all streams, nothing pending
            seen.append(residual.sum(0).numpy())
            return out

        blk.forward = forward
    groups = len(runner.num_blocks_per_group)
    runner.step([StepItem(key="a", tokens=toks, start=0, block_tables=[[0, 1, 2]] * groups, slot=0, want=[36])])
    assert len(seen) == len(want) == 3
    for i, (got, exp) in enumerate(zip(seen, want)):
        assert close(got, exp), f"layer {i}"


def test_the_first_tokens_one_at_a_time(folders):
    """Sequences shorter than every convolution's taps, every window and every block, fed token by token."""
    for name in FUBELORN:
        toks = np.random.default_rng(5).integers(0, FUBELORN[name]["vocab"], 5).tolist()
        truth = truth_of(folders[name], toks)
        for n in range(1, 6):
            steps, expect = traces.decode_tail([toks[:n]], tail=n)
            assert traces.compare(TraceReplayer(runner_for(folders[name], 2)).run_step, steps, expect, [truth[:n]], TOL) < TOL


def test_long_decoding_and_a_state_slot_used_three_times(folders):
    toks = np.random.default_rng(6).integers(0, 90, 170).tolist()
    truth = truth_of(folders["A"], toks)
    runner = runner_for(folders["A"], 12, slots=1)
    for _ in range(3):                                       # the one slot and the same pages, each time from their last contents
        steps, expect = traces.decode_tail([toks], tail=150)
        assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], TOL) < TOL


# ------------------------------------------------------------------ faults that would show

def sharp(tensors):
    """Weights under which single keys carry the softmax and states live long: a key that is seen or not
    seen by mistake, or a state that is lost, then moves the logits by far more than rounding."""
    for name, t in tensors.items():
        if name.endswith(".A_log"):
            t.fill_(-4.0)                                    # slow decay: a lost state is a large loss
        if name.endswith("left.q") or name.endswith("left.k"):
            t.mul_(4.0)
        if name.endswith(".f.b"):
            t.fill_(4.0)                                     # the memory forgets slowly


def test_an_edge_that_is_one_token_off_would_show(tmp_path):
    """The engine agrees with the plain model at every position, in prompts and in decoding; the same plain
    model with a window, a count of kept tokens or a block's visibility off by one, a convolution shifted, or a read-out
    before the token's own write is far away."""
    cfg = model(60, 32, 1e-5, [
        layer(side_by_side("parallel", attention(2, 1, 8, 8, 2.0, 7, keep_first=3), delta(2, 1, 8, 8, 3), 1.0, 1.0), 24),
        layer(mamba2(2, 8, 6, 1, 3, 2), None),
        layer(side_by_side("parallel_2", attention(2, 2, 8, 8, 2.0, 6, pool=5, rot={"dims": 4, "base": 100.0}), memory(2, 8, 8, 8.0), 1.0, 1.0), 24),
    ], streams=2, taps=3, mult=0.8)
    folder = write_fubelorn(tmp_path, cfg, seed=2, std=0.3, edit=sharp)
    toks = np.random.default_rng(3).integers(0, 60, 75).tolist()
    raw, tensors = plain.load(folder)
    truth = plain.forward(raw, tensors, toks)
    assert close(whole(runner_for(folder, 5), toks), truth)
    for build in (traces.decode_tail, traces.portions):
        steps, expect = build([toks])
        assert traces.compare(TraceReplayer(runner_for(folder, 5)).run_step, steps, expect, [truth], TOL) < TOL

    def off(change=None, patch=None) -> float:
        other = copy.deepcopy(raw)
        undo = None
        if change is not None:
            change(other)
        if patch is not None:
            name, fn = patch
            undo = getattr(plain, name)
            setattr(plain, name, fn)
        try:
            return float(np.abs(plain.forward(other, tensors, toks) - truth).max() / np.abs(truth).max())
        finally:
            if undo is not None:
                setattr(plain, name, undo)

    def mask_of(i, key, value):
        def change(c):
            c["layers"][i]["mixer"]["left"]["mask"][key] = value
        return change

    def shifted_conv(h, w, bias=None, _inner=plain.causal_conv):
        return _inner(np.concatenate([np.zeros_like(h[:1]), h[:-1]]), w, bias)

    def read_before_write(q, k, v, beta, g):
        t_n, heads, d = q.shape
        out = np.zeros((t_n, heads, v.shape[2]))
        for h in range(heads):
            s = np.zeros((d, v.shape[2]))
            for t in range(t_n):
                s = g[t, h] * s
                out[t, h] = s.T @ q[t, h]
                s = s + np.outer(k[t, h], beta[t, h] * (v[t, h] - s.T @ k[t, h]))
        return out

    def memory_read_before_write(q, k, v, i_log, f_log):
        t_n, heads, d = q.shape
        out = np.zeros((t_n, heads, v.shape[2]))
        for h in range(heads):
            s, n, m = np.zeros((d, v.shape[2])), np.zeros(d), 0.0
            for t in range(t_n):
                m_new = max(f_log[t, h] + m, i_log[t, h])
                keep, write = math.exp(f_log[t, h] + m - m_new), math.exp(i_log[t, h] - m_new)
                out[t, h] = (keep * s.T @ q[t, h]) / (max(abs(keep * n @ q[t, h]), math.exp(-m_new)) + 1e-6)
                s, n, m = keep * s + write * np.outer(k[t, h], v[t, h]), keep * n + write * k[t, h], m_new
        return out

    faults = {
        "window one longer": off(mask_of(0, "size", 8)), "window one shorter": off(mask_of(0, "size", 6)),
        "one more kept": off(mask_of(0, "keep_first", 4)), "one fewer kept": off(mask_of(0, "keep_first", 2)),
        "pooled window one longer": off(mask_of(2, "size", 7)), "pooled window one shorter": off(mask_of(2, "size", 5)),
        "block one longer": off(mask_of(2, "pool", 6)), "no blocks": off(mask_of(2, "pool", 0)),
        "convolutions shifted": off(patch=("causal_conv", shifted_conv)),
        "read-out before the write": off(patch=("gated_delta", read_before_write)),
        "the memory read before its write": off(patch=("matrix_memory", memory_read_before_write)),
        "no scale on the sub-layers": off(lambda c: c.update(residual_mult=1.0)),
    }
    assert all(err > 100 * TOL for err in faults.values()), faults


def test_far_keys_in_kept_tokens_and_pooled_blocks_carry_the_output(tmp_path):
    """Queries hundreds of tokens on whose largest scores are a kept first token's and a pooled block's: the
    output then hangs on pages that were written long ago and on means formed at a block's end."""
    cfg = model(40, 32, 1e-5, [
        layer(side_by_side("parallel", attention(2, 2, 8, 8, 1.0, 20, keep_first=2), delta(1, 1, 8, 8, 2), 1.0, 0.2), None),
        layer(side_by_side("parallel_2", attention(2, 2, 8, 8, 1.0, 24, pool=8), memory(1, 8, 8, 8.0), 1.0, 0.2), None),
    ], streams=1, mult=1.0)
    folder = write_fubelorn(tmp_path, cfg, seed=6, std=0.3)
    toks = np.random.default_rng(8).integers(0, 40, 420).tolist()
    raw, tensors = plain.load(folder)
    truth = plain.forward(raw, tensors, toks)
    steps, expect = traces.portions([toks], sizes=(130, 2, 77, 1, 1, 1, 33, 64))
    assert traces.compare(TraceReplayer(runner_for(folder, 27)).run_step, steps, expect, [truth], TOL) < TOL
    # what is lost when the far part is not seen: the kept tokens, the blocks
    for i, key in ((0, "keep_first"), (1, "pool")):
        other = copy.deepcopy(raw)
        other["layers"][i]["mixer"]["left"]["mask"][key] = 0
        far = plain.forward(other, tensors, toks)[400:]
        assert float(np.abs(far - truth[400:]).max() / np.abs(truth).max()) > 100 * TOL


# ------------------------------------------------------------------ the engine's own entry point

def test_greedy_generation_through_the_engine_and_the_scheduler(folders):
    from prefixserve_amd import Engine, EngineConfig, generate

    for name in ("A", "C"):
        cfg, tensors = plain.load(folders[name])
        rng = np.random.default_rng(11)
        prompts = [rng.integers(0, cfg["vocab"], n).tolist() for n in (19, 40, 7)]
        eng = Engine(EngineConfig(model_path=str(folders[name]), dtype="float32", device="cpu", max_num_seqs=3, max_prefill_tokens=16,
                                  max_seq_len=128, num_blocks=24, use_graphs=False), ops=EmulatedOps())
        outs, _ = generate(eng, prompts, 12, ignore_eos=True)
        for p, o in zip(prompts, outs):
            seq = list(p)
            for _ in range(12):
                seq.append(int(np.argmax(plain.forward(cfg, tensors, seq)[-1])))
            assert o.tokens == seq[len(p):]
