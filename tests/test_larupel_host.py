"""Larupel on the host: its configuration, the model built from it, and the whole engine path
(packing, pages, state slots, layers that read another layer's keys, replay, scheduler,
generation) with the kernel library's CPU stand-in, against the plain implementation in
tests/plain/larupel_plain.py."""

from __future__ import annotations

import copy
import json

import numpy as np
import pytest
import torch

import traces
from emulated_ops import EmulatedOps
from larupel_configs import LARUPEL, attention, delta, dense, general_delta, layer, model, moe, write_larupel
from plain import larupel_plain as plain
from prefixserve_amd.config import UnsupportedModelError, read_model_dir
from prefixserve_amd.config.larupel import LarupelConfig
from prefixserve_amd.engine.batch import StepItem
from prefixserve_amd.engine.replay import TraceReplayer
from prefixserve_amd.engine.runner import ModelRunner
from prefixserve_amd.models.larupel import build_larupel_spec

# 32-bit against the float64 oracle, per row relative to its largest logit. The median row is at 5e-7; a head's
# read-out that nearly cancels is brought back to size one by the norm behind it, its rounding with it (4e-5 seen).
TOL = 1e-4


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: write_larupel(tmp_path_factory.mktemp(f"larupel-{name}"), name) for name in LARUPEL}


def runner_for(folder, pages, dtype="float32", slots=4):
    return ModelRunner(folder, dtype=dtype, device="cpu", num_blocks=pages, max_seq_len=pages * 16, max_num_seqs=slots,
                       use_graphs=False, ops=EmulatedOps())


def whole(runner, toks, want=None):
    want = list(range(len(toks))) if want is None else want
    rp = TraceReplayer(runner)
    return rp.run_step({"step": 0, "entries": [{"id": "a", "tokens": list(toks), "want": want}], "end": ["a"]})


def close(got, want, tol=TOL):
    return float(np.abs(got - want).max()) <= tol * float(np.abs(want).max())


# ------------------------------------------------------------------ configuration and spec

def test_configuration_reads_every_key_and_refuses_what_it_does_not_know():
    cfg = LarupelConfig.from_dicts(LARUPEL["A"])
    assert (cfg.vocab_size, cfg.hidden_size, cfg.norm_eps) == (96, 64, 1e-5)
    g, a, d, r = (cfg.layers[i].mixer for i in range(4))
    assert (g.heads, g.dim, g.decay_rank) == (2, 16, 5)
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.kv_from) == (6, 2, 8, 12, 0.5, None)
    assert (d.heads, d.kv_heads, d.dim, d.vdim, d.conv) == (4, 2, 8, 12, 3)
    assert r.kv_from == 1 and cfg.layers[3].mlp is None
    f0, f1, f2 = (cfg.layers[i].mlp for i in range(3))
    assert (f0.experts, f0.top, f0.ff, f0.shared_ff) == (5, 2, 24, 40) and f1.ff == 80 and f2.shared_ff is None
    assert LarupelConfig.from_dicts(cfg.to_config_json()) == cfg
    lean = copy.deepcopy(LARUPEL["A"])
    for key in ("kv_heads", "dim", "vdim"):
        del lean["layers"][3]["mixer"][key]                  # a reader that leaves its key sizes to its source
    assert LarupelConfig.from_dicts(lean) == cfg
    for path, value in [(("layers", 0, "type"), "conv"), (("layers", 1, "mlp", "kind"), "glu"), (("layers", 1, "mixer", "window"), 8),
                        (("layers", 1, "mixer", "kv_heads"), 4), (("layers", 3, "mixer", "kv_from"), 2),
                        (("layers", 3, "mixer", "kv_from"), 3), (("layers", 3, "mixer", "vdim"), 8), (("layers", 0, "mlp", "router", "top"), 6),
                        (("layers", 2, "mixer", "conv"), 0), (("layers", 2, "mixer", "kv_heads"), 3), (("tie",), True),
                        (("norm", "kind"), "rms")]:
        raw = copy.deepcopy(LARUPEL["A"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        with pytest.raises(UnsupportedModelError):
            LarupelConfig.from_dicts(raw)


def test_the_decay_maps_inner_size_comes_from_the_checkpoint(folders):
    raw = json.loads((folders["A"] / "config.json").read_text())
    assert all("decay_rank" not in entry["mixer"] for entry in raw["layers"])
    with pytest.raises(UnsupportedModelError):
        build_larupel_spec(LarupelConfig.from_dicts(raw))
    arch, cfg, _ = read_model_dir(folders["A"])
    assert arch.name == "Larupel" and cfg.layers[0].mixer.decay_rank == 5
    assert read_model_dir(folders["C"])[1].layers[3].mixer.decay_rank == 3


def test_readers_share_their_source_layers_cache_entry_and_state_is_per_layer(folders):
    spec = build_larupel_spec(read_model_dir(folders["C"])[1])
    assert [(r.layer, r.cache, r.writes_cache) for r in spec.order] == [
        (0, 0, True), (1, 0, False), (2, 2, True), (3, 3, True), (4, 4, True), (5, 4, False), (6, 0, False)]
    assert spec.layers[1].mixer.params["own_kv"] is False and spec.layers[0].mixer.params["own_kv"] is True
    runner = runner_for(folders["C"], 8)
    needs = runner.model.state_needs()
    assert sorted(needs) == [2, 3]
    assert needs[2].shape == ((5 - 1) * (2 * 12 + 2 * 20) + 2 * 20 * 12,) and needs[3].shape == (3 * 8 * 8,)
    assert all(w is None for w in runner.windows)
    # a reader has no key and value tensors
    wanted = runner.model.weights()
    assert "l1.mix.q" in wanted and "l1.mix.q.norm" in wanted and "l1.mix.temp" in wanted
    assert not any(n in wanted for n in ("l1.mix.k", "l1.mix.v", "l1.mix.k.norm"))


# ------------------------------------------------------------------ mechanisms, one at a time

def test_the_plain_mixers_agree_with_their_definitions_written_out():
    """The oracle's own functions against the equations token by token and entry by entry."""
    rng = np.random.default_rng(5)
    n, dim, vdim = 6, 3, 2
    q, k, v = rng.normal(size=(n, dim)), rng.normal(size=(n, dim)), rng.normal(size=(n, vdim))
    b, g = rng.uniform(size=n), rng.uniform(size=n)
    got = plain.gated_delta(q, k, v, b, g)
    s = [[0.0] * vdim for _ in range(dim)]
    for t in range(n):
        s = [[g[t] * s[i][j] for j in range(vdim)] for i in range(dim)]
        seen = [sum(s[i][j] * k[t][i] for i in range(dim)) for j in range(vdim)]
        s = [[s[i][j] + k[t][i] * b[t] * (v[t][j] - seen[j]) for j in range(vdim)] for i in range(dim)]
        assert np.allclose(got[t], [sum(s[i][j] * q[t][i] for i in range(dim)) for j in range(vdim)], rtol=1e-12)
    w, a = rng.uniform(0.5, 1.0, size=(n, dim)), rng.uniform(size=(n, dim))
    got = plain.generalized_delta(q, k, v, w, a)
    s = [[0.0] * vdim for _ in range(dim)]
    for t in range(n):
        length = np.sqrt(sum(x * x for x in k[t]) + 1e-6)
        u = [x / length for x in k[t]]
        seen = [sum(u[i] * s[i][j] for i in range(dim)) for j in range(vdim)]          # the state before this token
        s = [[w[t][i] * s[i][j] - a[t][i] * u[i] * seen[j] + k[t][i] * v[t][j] for j in range(vdim)] for i in range(dim)]
        assert np.allclose(got[t], [sum(s[i][j] * q[t][i] for i in range(dim)) for j in range(vdim)], rtol=1e-12)
    x = rng.normal(size=(5, 2))
    taps = rng.normal(size=(2, 3))
    y = plain.short_conv(x, taps)
    assert np.allclose(y[0], taps[:, 2] * x[0]) and np.allclose(y[1], taps[:, 1] * x[0] + taps[:, 2] * x[1])
    assert np.allclose(y[4], taps[:, 0] * x[2] + taps[:, 1] * x[3] + taps[:, 2] * x[4])
    chosen, weight = plain.route(np.array([[0.1, 2.0, -1.0, 2.0, 0.5]]), 3)
    assert chosen.tolist() == [[1, 3, 4]]
    e = np.exp([2.0, 2.0, 0.5])
    assert np.allclose(weight[0], e / e.sum())
    pos = plain.sinusoid(np.array([0, 3]), 6)
    assert np.allclose(pos[0], [0, 1, 0, 1, 0, 1])
    assert np.allclose(pos[1], [np.sin(3.0), np.cos(3.0), np.sin(3 * 10000 ** (-2 / 6)), np.cos(3 * 10000 ** (-2 / 6)),
                                np.sin(3 * 10000 ** (-4 / 6)), np.cos(3 * 10000 ** (-4 / 6))])
    z = rng.normal(size=(2, 7))
    ln = plain.layer_norm(z, np.full(7, 2.0), np.full(7, 0.5), 0.0)
    assert np.allclose(ln.mean(-1), 0.5) and np.allclose(ln.std(-1), 2.0)
    _, p = plain.causal_softmax_attention(rng.normal(size=(4, 3)), rng.normal(size=(4, 3)), rng.normal(size=(4, 2)), 0.7)
    assert np.allclose(p.sum(-1), 1.0) and np.all(np.triu(p, 1) == 0) and np.all(np.diag(p) > 0)


ONE_LAYER = {
    "delta": delta(4, 2, 8, 12, 3),
    "delta-one-tap-one-head": delta(1, 1, 20, 6, 1),
    "delta-many-taps": delta(3, 3, 6, 6, 7),
    "general_delta": general_delta(2, 16, 5),
    "general_delta-one-head": general_delta(1, 40, 1),
    "attention": attention(6, 2, 8, 12, 0.5),
    "attention-one-head-large-value": attention(1, 1, 12, 40, 0.3),
}
FEED_FORWARDS = {"none": None, "dense": dense(24), "experts": moe(6, 3, 8), "experts-shared": moe(4, 1, 16, shared=8),
                 "all-experts": moe(3, 3, 8, shared=24)}


@pytest.mark.parametrize("kind", list(ONE_LAYER))
@pytest.mark.parametrize("ff", ["none", "dense", "experts-shared"])
def test_each_mixer_alone(kind, ff, tmp_path):
    """A model of one layer: whatever differs from the plain model is that mixer's (or the block's)."""
    folder = write_larupel(tmp_path, model(50, 32, 1e-5, [layer(ONE_LAYER[kind], FEED_FORWARDS[ff])]), seed=8)
    toks = np.random.default_rng(1).integers(0, 50, 45).tolist()
    want = plain.PlainLarupel.from_dir(folder).logits(toks)
    assert close(whole(runner_for(folder, 4), toks), want)


@pytest.mark.parametrize("ff", list(FEED_FORWARDS))
def test_each_feed_forward_alone(ff, tmp_path):
    folder = write_larupel(tmp_path, model(40, 24, 1e-6, [layer(attention(2, 1, 8, 8, 0.4), FEED_FORWARDS[ff])]), seed=5, std=0.3)
    toks = np.random.default_rng(2).integers(0, 40, 50).tolist()
    assert close(whole(runner_for(folder, 4), toks), plain.PlainLarupel.from_dir(folder).logits(toks))


def test_a_reader_sees_the_keys_as_the_other_layer_normed_them(tmp_path):
    """Two readers of one layer behind it, with head counts of queries that differ from nothing but
    weights: the readers' logits change when the source's key norm weight does."""
    cfg = model(40, 32, 1e-5, [layer(attention(4, 2, 8, 8, 0.6), dense(16)), layer(delta(2, 1, 8, 8, 2), None),
                               layer(attention(4, 2, 8, 8, 0.6, kv_from=0), None), layer(attention(4, 2, 8, 8, 0.6, kv_from=0), dense(16))])
    folder = write_larupel(tmp_path, cfg, seed=4, std=0.3)
    toks = np.random.default_rng(3).integers(0, 40, 40).tolist()
    assert close(whole(runner_for(folder, 4), toks), plain.PlainLarupel.from_dir(folder).logits(toks))


# ------------------------------------------------------------------ whole models

LENGTHS = [70, 33, 97, 18, 64, 45, 1, 52, 2, 81, 29, 3]


@pytest.mark.parametrize("name", list(LARUPEL))
def test_every_cutting_matches_the_plain_model_on_the_host(name, folders):
    rng = np.random.default_rng(4)
    reqs = [rng.integers(0, LARUPEL[name]["vocab"], n).tolist() for n in LENGTHS]
    pm = plain.PlainLarupel.from_dir(folders[name])
    truth = [pm.logits(t) for t in reqs]
    runner = runner_for(folders[name], 32)
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
    """The stream behind every layer: a fault shows in the layer that makes it."""
    toks = np.random.default_rng(9).integers(0, 70, 37).tolist()
    _, want = plain.PlainLarupel.from_dir(folders["C"]).forward(toks, return_layers=True)
    runner = runner_for(folders["C"], 8)
    seen = []
    for blk in runner.model.blocks:
        inner = blk.forward

        def forward(residual, *a, _inner=inner, **kw):
            out = _inner(residual, *a, **kw)
            assert out is None                               # a sandwich block leaves nothing pending
            seen.append(residual.clone().numpy())
            return out

        blk.forward = forward
    groups = len(runner.num_blocks_per_group)
    runner.step([StepItem(key="a", tokens=toks, start=0, block_tables=[[0, 1, 2]] * groups, slot=0, want=[36])])
    assert len(seen) == len(want) == 7
    for i, (got, exp) in enumerate(zip(seen, want)):
        assert close(got, exp), f"layer {i}"


def peaky(tensors):
    """Weights under which single keys carry the softmax, states live long and the router's choice
    matters: a fault in any of them then moves the logits by far more than rounding."""
    for name, t in tensors.items():
        if name.endswith(".temp"):
            t.copy_(torch.linspace(0.5, 3.0, t.numel()).to(t.dtype))
        if name.endswith(".A_log"):
            t.fill_(-4.0)                                    # slow decay: a lost state is a large loss
        if name.endswith(".w0"):
            t.fill_(-3.0)
        if name.endswith("router.b"):
            t.mul_(3.0)
        if name.endswith(".sg"):
            t.mul_(6.0)


def test_a_wrong_source_scale_state_order_or_router_would_show(tmp_path):
    cfg = model(60, 32, 1e-5, [layer(attention(4, 2, 8, 8, 6.0), dense(24)), layer(delta(2, 1, 8, 8, 3), moe(6, 2, 16, shared=8)),
                               layer(attention(4, 2, 8, 8, 6.0), None), layer(general_delta(2, 8, 4), dense(24)),
                               layer(attention(4, 2, 8, 8, 6.0, kv_from=0), None)])
    folder = write_larupel(tmp_path, cfg, seed=2, std=0.3, edit=peaky)
    toks = np.random.default_rng(3).integers(0, 60, 60).tolist()
    truth = plain.PlainLarupel.from_dir(folder).logits(toks)
    assert close(whole(runner_for(folder, 4), toks), truth)
    steps, expect = traces.portions([toks])
    assert traces.compare(TraceReplayer(runner_for(folder, 4)).run_step, steps, expect, [truth], TOL) < TOL

    def wrong(change, patch=None) -> float:
        other = plain.PlainLarupel.from_dir(folder)
        undo = None
        if change is not None:
            change(other)
        if patch is not None:
            name, fn = patch
            undo = getattr(plain, name)
            setattr(plain, name, fn)
        try:
            return float(np.abs(other.logits(toks) - truth).max() / np.abs(truth).max())
        finally:
            if undo is not None:
                setattr(plain, name, undo)

    def read_before_write(q, k, v, strength, decay):
        n, dim = k.shape
        s, out = np.zeros((dim, v.shape[1])), np.zeros_like(v)
        for t in range(n):
            s = decay[t] * s
            out[t] = s.T @ q[t]                              # the read-out misses the token's own write
            s = s + np.outer(k[t], strength[t] * (v[t] - s.T @ k[t]))
        return out

    def removal_reads_decayed(r, k, v, w, a):
        n, dim = k.shape
        s, out, unit = np.zeros((dim, v.shape[1])), np.zeros_like(v), plain.unit_length(k)
        for t in range(n):
            s = w[t][:, None] * s
            s = s - np.outer(a[t] * unit[t], unit[t] @ s) + np.outer(k[t], v[t])
            out[t] = s.T @ r[t]
        return out

    def softmax_over_all(logits, top):
        order, _ = undo_route(logits, top)
        z = np.exp(logits - logits.max(-1, keepdims=True))
        return order, np.take_along_axis(z / z.sum(-1, keepdims=True), order, axis=-1)

    undo_route, undo_sin = plain.route, plain.sinusoid
    changes = [
        (lambda m: m.cfg["layers"][4]["mixer"].update(kv_from=2), None),
        (lambda m: m.w.__setitem__("l0.mix.temp", np.ones(4)), None),
        (lambda m: m.w.__setitem__("l4.mix.q.norm", np.ones(8)), None),
        (lambda m: m.w.__setitem__("l0.mix.k.norm", np.ones(8)), None),
        (lambda m: m.cfg["layers"][0]["mixer"].update(scale=5.0), None),
        (lambda m: m.w.__setitem__("l1.mix.q.conv", np.roll(m.w["l1.mix.q.conv"], 1, axis=1)), None),
        (lambda m: m.w.__setitem__("l1.mix.dt_bias", m.w["l1.mix.dt_bias"] * 0), None),
        (lambda m: m.w.__setitem__("l3.mix.a.b", m.w["l3.mix.a.b"] * 0), None),
        (lambda m: m.w.__setitem__("l1.mlp.router.b", m.w["l1.mlp.router.b"] * 0), None),
        (lambda m: m.w.__setitem__("l1.mlp.shared.sg", m.w["l1.mlp.shared.sg"] * 0), None),
        (lambda m: m.w.__setitem__("l2.norm1b.b", m.w["l2.norm1b.b"] * 0), None),
        (None, ("gated_delta", read_before_write)),
        (None, ("generalized_delta", removal_reads_decayed)),
        (None, ("route", softmax_over_all)),
        (None, ("sinusoid", lambda p, width: np.roll(undo_sin(p, width), 1, axis=-1))),      # cos where sin belongs
    ]
    for change, patch in changes:
        assert wrong(change, patch) > 100 * TOL, (change, patch)


def test_one_far_key_carries_the_softmax_across_many_pages(tmp_path):
    """Hundreds of keys, a large score scale: almost all weight of late queries sits on single keys
    far back, in a prompt, in portions and decoded; pages are 16 tokens, so every offset in a page occurs."""
    cfg = model(48, 32, 1e-5, [layer(attention(2, 1, 16, 16, 8.0), None), layer(attention(2, 1, 16, 16, 8.0, kv_from=0), dense(16))])
    folder = write_larupel(tmp_path, cfg, seed=6, std=0.3)
    rng = np.random.default_rng(8)
    toks = rng.integers(0, 48, 420).tolist()
    pm = plain.PlainLarupel.from_dir(folder)
    truth = pm.logits(toks)
    h = pm.norm(pm.w["embed"][np.asarray(toks)] + plain.sinusoid(np.arange(420), 32), "l0.norm1")
    k, v = pm.keys_values(h, "l0.mix.", cfg["layers"][0]["mixer"])
    q = plain.unit_rms((h @ pm.w["l0.mix.q"].T).reshape(420, 2, 16), 1e-5) * pm.w["l0.mix.q.norm"]
    _, p = plain.causal_softmax_attention(q[:, 0], k[:, 0], v[:, 0], 8.0 * pm.w["l0.mix.temp"][0])
    far = [(i, int(np.argmax(p[i]))) for i in range(300, 420) if p[i].max() > 0.5 and i - int(np.argmax(p[i])) > 200]
    assert len(far) >= 5                                     # the weights do what the test is for
    runner = runner_for(folder, 32)
    assert close(whole(runner, toks), truth)
    steps, expect = traces.decode_tail([toks], tail=125)
    assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], TOL) < TOL
    steps, expect = traces.portions([toks])
    assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], TOL) < TOL


def test_first_tokens_and_long_decoding(folders):
    """Sequences of one to five tokens (shorter than the convolutions' taps), and 150 tokens decoded one by one."""
    pm = plain.PlainLarupel.from_dir(folders["C"])
    runner = runner_for(folders["C"], 16)
    rng = np.random.default_rng(6)
    for n in (1, 2, 3, 4, 5):
        toks = rng.integers(0, 70, n).tolist()
        assert close(whole(runner, toks), pm.logits(toks))
        steps, expect = traces.decode_tail([toks], tail=n)   # one token at a time from the very first
        assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [pm.logits(toks)], TOL) < TOL
    toks = rng.integers(0, 70, 170).tolist()
    truth = pm.logits(toks)
    steps, expect = traces.decode_tail([toks], tail=150)
    assert traces.compare(TraceReplayer(runner).run_step, steps, expect, [truth], TOL) < TOL


def test_a_state_slot_that_is_used_again_starts_from_zero(folders):
    """Two requests one after the other in the only slot: the second one's logits are its own."""
    pm = plain.PlainLarupel.from_dir(folders["A"])
    runner = runner_for(folders["A"], 8, slots=1)
    rng = np.random.default_rng(10)
    rp = TraceReplayer(runner)
    for step in range(3):
        toks = rng.integers(0, 96, 30 + step).tolist()
        got = rp.run_step({"step": 2 * step, "entries": [{"id": f"r{step}", "tokens": toks[:20], "want": [19]}], "end": []})
        assert close(got, pm.logits(toks)[19:20])
        got = rp.run_step({"step": 2 * step + 1, "entries": [{"id": f"r{step}", "tokens": toks[20:], "want": list(range(len(toks) - 20))}],
                           "end": [f"r{step}"]})
        assert close(got, pm.logits(toks)[20:])


def test_greedy_generation_through_the_engine_and_scheduler(folders):
    """The package's entry point: prompts in portions of 16 under a budget, three requests at a time,
    few pages, state slots taken and given back; no prefix cache (the delta rules keep state)."""
    from prefixserve_amd.engine.engine import Engine, EngineConfig
    from prefixserve_amd.generation import generate

    pm = plain.PlainLarupel.from_dir(folders["B"])
    rng = np.random.default_rng(12)
    prompts = [rng.integers(0, 130, n).tolist() for n in (5, 23, 40, 9, 31)]
    eng = Engine(EngineConfig(model_path=str(folders["B"]), dtype="float32", device="cpu", max_num_seqs=3,
                              max_prefill_tokens=16, max_seq_len=128, num_blocks=14, use_graphs=False), ops=EmulatedOps())
    outs, _stats = generate(eng, prompts, 12, temperature=0.0, ignore_eos=True)
    for p, o in zip(prompts, outs):
        assert list(o.tokens) == pm.greedy(p, 12)
    assert all(o.cached_tokens == 0 for o in outs)
