"""How a layer's parts are arranged."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any

import torch

from .base import FeedForward, Mixer, Norm, Part, register_block

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class PreNormBlock:
    """norm -> mixer -> add, norm -> feed-forward -> add (prefixserve/model/llama.py:111-121).

    The residual stream is float32. Each sub-layer's output is not added at once: it is
    handed on as ``pending`` and summed into the residual by the next norm's fused
    add+norm, so the stream is read and written once per sub-layer. A sub-layer may also add its
    output into the stream itself and hand on None; and where a sub-layer's kernels normalize
    their tokens themselves (``takes_normed_rows``), the norm in front of it may hand over the
    rows of the stream instead of running a kernel. An arrangement that needs a sub-layer's
    output itself (to normalize it before it is added, say) sets ``ctx.residual = None`` first:
    the sub-layers then hand their output back in every step."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward, mixer_norm: Norm, feed_forward_norm: Norm) -> None:
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward]

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> torch.Tensor:
        ctx.stream_copy = None               # the stream moves on without its activation-dtype copy
        if self.mixer.takes_normed_rows:
            x = self.mixer_norm.add_norm(residual, pending, "block.x", lazy=True)
        else:
            x = self.mixer_norm.add_norm(residual, pending, "block.x")
        mixed = self.mixer.forward(x, ctx, cache, state, writes_cache)
        if self.feed_forward.takes_normed_rows:
            x = self.feed_forward_norm.add_norm(residual, mixed, "block.x", lazy=True)
        else:
            x = self.feed_forward_norm.add_norm(residual, mixed, "block.x")
        return self.feed_forward.forward(x, ctx)


class PostNormBlock:
    """The norm behind the sum: x <- norm1(alpha x + mixer(x)), then, when the layer has a
    feed-forward, x <- norm2(alpha x + feed_forward(x)). The sub-layers read the stream itself,
    which is a normalized vector from the first layer's first norm on; ``alpha`` is the factor
    on the stream in front of each sum (1: the plain arrangement). Sum, statistics and the
    stream are float32; beside the stream the norm writes its copy in the activation dtype
    for the next sub-layer's products (``ctx.stream_copy``, so that the next block of this
    kind does not convert again). ``feed_forward`` None: the second half does not exist, unless a
    second norm is given all the same, which is then applied to the stream alone, norm2(alpha x)."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm,
                 feed_forward_norm: Norm | None, alpha: float = 1.0) -> None:
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.alpha = float(alpha)

    def parts(self) -> list[Part]:
        both = [self.mixer_norm, self.mixer]
        if self.feed_forward is not None:
            return both + [self.feed_forward_norm, self.feed_forward]
        return both + ([self.feed_forward_norm] if self.feed_forward_norm is not None else [])

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> None:
        rt = self.mixer_norm.rt
        if pending is not None:
            # A sub-layer in front left its output to be added: the norm's fused sum does that
            # (its normalized output is not wanted here).
            self.mixer_norm.add_norm(residual, pending, "block.x")
            ctx.stream_copy = None
        kept, ctx.residual = ctx.residual, None   # the sub-layers hand their output back: it is normalized with the stream
        x = residual if rt.dtype == torch.float32 else getattr(ctx, "stream_copy", None)
        if x is None:
            x = rt.workspace.get("block.x", tuple(residual.shape), rt.dtype)
            rt.ops.to_activation(residual, x)
        mixed = self.mixer.forward(x, ctx, cache, state, writes_cache)
        x = self.mixer_norm.norm_of_sum(residual, mixed, self.alpha, "block.x")
        if self.feed_forward is not None:
            x = self.feed_forward_norm.norm_of_sum(residual, self.feed_forward.forward(x, ctx), self.alpha, "block.x")
        elif self.feed_forward_norm is not None:
            x = self.feed_forward_norm.norm_of_sum(residual, None, self.alpha, "block.x")
        ctx.stream_copy = x
        ctx.residual = kept
        return None


class ParallelBlock:
    """One norm, both sub-layers read it: x <- x + mixer(n(x)) + feed_forward(n(x)).

    The normalized rows are written out by the norm kernel (never left to the consumers: the
    mixer may add into the stream before the feed-forward has read it). The mixer's output goes
    into the stream at once, the feed-forward's is handed on as ``pending`` for the next layer's
    fused add+norm. ``feed_forward`` None: the layer is x <- x + mixer(n(x))."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm,
                 feed_forward_norm: Norm | None = None) -> None:
        if feed_forward_norm is not None:
            raise ValueError("a parallel block has one norm")
        self.mixer, self.feed_forward, self.mixer_norm = mixer, feed_forward, mixer_norm

    def parts(self) -> list[Part]:
        return [self.mixer_norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> torch.Tensor | None:
        ctx.stream_copy = None
        h = self.mixer_norm.add_norm(residual, pending, "block.x")
        mixed = self.mixer.forward(h, ctx, cache, state, writes_cache)
        if self.feed_forward is None:
            return mixed
        if mixed is not None:
            self.mixer_norm.rt.ops.residual_add(residual, mixed)
        return self.feed_forward.forward(h, ctx)


class SandwichBlock:
    """A norm in front of and behind each sub-layer: x <- x + post1(mixer(pre1(x))), then, when the
    layer has a feed-forward, x <- x + post2(feed_forward(pre2(x))).

    The sub-layers hand their output back (``ctx.residual`` is None while they run): it is
    normalized before it is added. The norm behind the mixer and the norm in front of the
    feed-forward are one kernel (``add_normed`` of the norms). The stream is complete when the
    block returns; nothing is left pending. ``mixer_post_norm`` / ``feed_forward_post_norm`` come
    from ``LayerSpec.extra_norms``."""

    def __init__(self, mixer: Mixer, feed_forward: FeedForward | None, mixer_norm: Norm, feed_forward_norm: Norm | None,
                 mixer_post_norm: Norm, feed_forward_post_norm: Norm | None = None) -> None:
        if (feed_forward is None) != (feed_forward_norm is None) or (feed_forward is None) != (feed_forward_post_norm is None):
            raise ValueError("a feed-forward comes with its two norms, a layer without one has neither")
        for norm in (mixer_post_norm, feed_forward_post_norm):
            if norm is not None and not hasattr(norm, "add_normed"):
                raise ValueError("the norm behind a sub-layer must offer add_normed")
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm
        self.mixer_post_norm, self.feed_forward_post_norm = mixer_post_norm, feed_forward_post_norm

    def parts(self) -> list[Part]:
        out = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        if self.feed_forward is not None:
            out += [self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm]
        return out

    def forward(self, residual: torch.Tensor, pending: torch.Tensor | None, ctx: "StepContext", cache: Any,
                state: torch.Tensor | None, writes_cache: bool) -> None:
        ctx.stream_copy = None
        h = self.mixer_norm.add_norm(residual, pending, "block.x")
        kept, ctx.residual = ctx.residual, None          # the sub-layers hand their output back: it is normalized first
        try:
            mixed = self.mixer.forward(h, ctx, cache, state, writes_cache)
            if self.feed_forward is None:
                self.mixer_post_norm.add_normed(residual, mixed)
            else:
                h = self.mixer_post_norm.add_normed(residual, mixed, then=self.feed_forward_norm, out_name="block.x")
                self.feed_forward_post_norm.add_normed(residual, self.feed_forward.forward(h, ctx))
        finally:
            ctx.residual = kept
        return None


register_block("prenorm", PreNormBlock)
register_block("sandwich", SandwichBlock)
register_block("parallel", ParallelBlock)
register_block("postnorm", PostNormBlock)
