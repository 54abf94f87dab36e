"""Several copies of the residual stream ("hyper-connections"), a convolution over time on what a
sub-layer reads, and a norm on the token table's output."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import (FeedForward, Mixer, Norm, Part, Runtime, StateNeed, Transform, WeightedDeltas, WeightWant, register_block,
                   register_transform)

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class _Connection:
    """One sub-layer's three tensors: read weights a [s], write weights c [s] (kept times the
    model's factor on every sub-layer's output) and the mixing matrix M [s, s] (from, to)."""

    def __init__(self, tensors: Mapping[str, torch.Tensor], names: Mapping[str, str], mult: float, rt: Runtime) -> None:
        def f32(key: str) -> torch.Tensor:
            return tensors[names[key]].to(torch.float32).contiguous().to(rt.device)

        self.read, self.mix = f32("in"), f32("mix")
        self.write = (f32("out") * mult).contiguous()


class HyperConnectionBlock:
    """A pre-norm layer over ``streams`` copies X_1 .. X_s of the residual stream. Sub-layer q
    (the mixer, then the feed-forward when the layer has one) reads u = sum_s a_s X_s, normalizes
    it, runs on it and writes every copy anew from the old ones:
        X_t <- sum_s M[s, t] X_s + mult c_t y                (M is indexed [from, to])
    With ``taps`` > 0 what the sub-layer reads, h = norm(u), is first replaced by h + conv(h): a
    causal convolution over the last ``taps`` tokens per channel (weights [hidden, taps], the last
    column meets the token itself, no bias, zeros in front of the sequence), whose last taps - 1
    inputs are part of the request's state, for both sub-layers. One copy and a = c = M = 1 is the
    plain pre-norm layer x <- x + mult y.

    The copies, the weighted sums, the norm and the convolution's sums are 32-bit; the sub-layer
    reads the result in the activation dtype. The sub-layers hand their output back
    (``ctx.residual`` is None while they run). The run's state is [saved inputs of the mixer's
    convolution | those of the feed-forward's | the mixer's own state]. ``names``: "mixer_in",
    "mixer_out", "mixer_mix", "feed_forward_in", "feed_forward_out", "feed_forward_mix" and, with
    taps, "mixer_conv", "feed_forward_conv". The norms must be RMS norms (``weight``, ``eps``)."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, feed_forward_norm: Norm | None,
                 streams: int, names: Mapping[str, str], mult: float = 1.0, taps: int = 0) -> None:
        if (feed_forward is None) != (feed_forward_norm is None):
            raise ValueError("a feed-forward comes with its norm, a layer without one has neither")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.streams, self.mult, self.taps = int(streams), float(mult), int(taps)
        if self.streams < 1 or not 0 <= self.taps <= 16:
            raise ValueError(f"{streams} streams, {taps} taps (at most 16)")
        self.names = dict(names)
        self.hidden_size = int(mixer_norm.hidden_size)
        self.tail = max(self.taps - 1, 0) * self.hidden_size
        self.sublayers = ["mixer"] + (["feed_forward"] if feed_forward is not None else [])
        self.own_state = self.tail * len(self.sublayers)
        self.mixer.state_base = self.own_state
        self.rt: Runtime | None = None

    # The block is a part itself: it owns the connections' tensors and the convolutions' taps.

    def weights(self) -> dict[str, WeightWant]:
        s, n = self.streams, self.names
        want: dict[str, WeightWant] = {}
        for q in self.sublayers:
            want[n[q + "_in"]] = WeightWant((s,), "norm")
            want[n[q + "_out"]] = WeightWant((s,), "norm")
            want[n[q + "_mix"]] = WeightWant((s, s), "bias")
            if self.taps:
                want[n[q + "_conv"]] = WeightWant((self.hidden_size, self.taps), "bias")
        return want

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.connections, self.conv_w = {}, {}
        for q in self.sublayers:
            self.connections[q] = _Connection(tensors, {k: n[f"{q}_{k}"] for k in ("in", "out", "mix")}, self.mult, rt)
            if self.taps:
                # h + conv(h) is one convolution whose last tap is one larger.
                w = tensors[n[q + "_conv"]].to(torch.float32).clone()
                w[:, -1] += 1.0
                self.conv_w[q] = w.contiguous().to(rt.device)

    def weight_bytes(self) -> int:
        return sum(w.numel() * 4 for w in self.conv_w.values())

    def parts(self) -> list[Part]:
        out: list[Any] = [self.mixer_norm, self.mixer]
        if self.feed_forward is not None:
            out += [self.feed_forward_norm, self.feed_forward]
        return out + [self]

    def state_need(self) -> StateNeed | None:
        inner = self.mixer.state_need()
        if inner is not None and inner.dtype != torch.float32:
            raise ValueError("a mixer's state beside the saved inputs must be 32-bit")
        n = self.own_state + (int(torch.Size(inner.shape).numel()) if inner is not None else 0)
        return StateNeed((n,), torch.float32) if n else None

    @property
    def state_in_graphs(self) -> bool:
        return self.mixer.state_need() is None or self.mixer.state_in_graphs

    def _sublayer(self, q: str, index: int, norm: Norm, streams: torch.Tensor, ctx: "StepContext",
                  state: torch.Tensor | None, run: Any) -> None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t = streams.shape[1]
        con = self.connections[q]
        if self.taps > 1:
            h = ws.get("hyper.h", (t, self.hidden_size), torch.float32)
            ops.hyper_read(streams, con.read, norm.weight, norm.eps, h)
            x = ws.get("block.x", (t, self.hidden_size), rt.dtype)
            ops.short_conv(h, 0, self.conv_w[q], x, state, index * self.tail, ctx, silu=False)
        else:
            x = ws.get("block.x", (t, self.hidden_size), rt.dtype)
            ops.hyper_read(streams, con.read, norm.weight, norm.eps, x,
                           factor=self.conv_w[q].view(-1) if self.taps == 1 else None)
        y = run(x)
        if isinstance(y, WeightedDeltas):
            if len(y.parts) == 2:
                (a, sa), (b, sb) = y.parts
                ops.hyper_write(streams, con.mix, con.write, a, sa, b, sb)
                return
            raise ValueError("the stream's kernel adds one output or the weighted sum of two")
        ops.hyper_write(streams, con.mix, con.write, y)

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> None:
        if pending is not None:
            raise ValueError("a block over several streams takes nothing pending from the layer in front")
        streams = residual if residual.dim() == 3 else residual.unsqueeze(0)
        if streams.shape[0] != self.streams:
            raise ValueError(f"the block is made for {self.streams} streams, the model runs {streams.shape[0]}")
        ctx.stream_copy = None
        kept, ctx.residual = ctx.residual, None      # the sub-layers hand their output back: it goes into every copy
        ctx.takes_weighted_deltas = True
        try:
            self._sublayer("mixer", 0, self.mixer_norm, streams, ctx, state,
                           lambda x: self.mixer.forward(x, ctx, cache, state, writes_cache))
            if self.feed_forward is not None:
                self._sublayer("feed_forward", 1, self.feed_forward_norm, streams, ctx, state,
                               lambda x: self.feed_forward.forward(x, ctx))
        finally:
            ctx.residual = kept
            ctx.takes_weighted_deltas = False
        return None


class NormalizeStream(Transform):
    """t <- weight * t / sqrt(mean(t^2) + eps) row by row, in 32-bit and in place: an RMS norm on the
    token table's output. ``scalar``: the stored weight is one number for all coordinates."""

    def __init__(self, hidden_size: int, vocab_size: int, eps: float, name: str, scalar: bool = False) -> None:
        self.hidden_size, self.eps, self.name, self.scalar = int(hidden_size), float(eps), name, bool(scalar)

    def weights(self) -> dict[str, WeightWant]:
        return {self.name: WeightWant(() if self.scalar else (self.hidden_size,), "norm")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        w = tensors[self.name].to(torch.float32).reshape(-1)
        self.weight = (w.expand(self.hidden_size) if self.scalar else w).contiguous().to(rt.device)

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        self.rt.ops.stream_rms_norm(t, self.weight, self.eps)


register_block("hyper", HyperConnectionBlock)
register_transform("rms_norm", NormalizeStream)
