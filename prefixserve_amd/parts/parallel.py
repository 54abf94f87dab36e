"""Two mixers side by side on the same input."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import CacheNeed, Mixer, PositionEncoding, Runtime, StateNeed, WeightedDeltas, WeightWant, make, register_mixer
from .spec import PartSpec

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class ParallelMixers(Mixer):
    """left_scale * left(x) + right_scale * right(x): both mixers read the same rows, each ends
    with its own output matrix, and the weighted sum (32-bit) is what the layer adds. ``left``
    and ``right`` are ``PartSpec``s of any registered mixers; their weight names are theirs. At
    most one of them may keep keys in pages; their fixed-size states lie side by side in the
    run's slot, the left one's first."""

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], left: PartSpec, right: PartSpec,
                 left_scale: float = 1.0, right_scale: float = 1.0) -> None:
        self.hidden_size = int(hidden_size)
        self.left = make("mixer", left.kind, hidden_size=hidden_size, positions=positions, **left.params)
        self.right = make("mixer", right.kind, hidden_size=hidden_size, positions=positions, **right.params)
        self.scales = (float(left_scale), float(right_scale))
        needs = [m.cache_need() for m in (self.left, self.right)]
        if all(n is not None for n in needs):
            raise ValueError("two mixers side by side that both keep keys in pages are not implemented")
        self.cached = self.left if needs[0] is not None else self.right if needs[1] is not None else None
        self._base = 0
        self._place()

    def _sizes(self) -> list[int]:
        out = []
        for m in (self.left, self.right):
            need = m.state_need()
            if need is not None and need.dtype != torch.float32:
                raise ValueError("states laid side by side must be 32-bit")
            out.append(0 if need is None else int(torch.Size(need.shape).numel()))
        return out

    def _place(self) -> None:
        self.left.state_base = self._base
        self.right.state_base = self._base + self._sizes()[0]

    @property
    def state_base(self) -> int:
        return self._base

    @state_base.setter
    def state_base(self, value: int) -> None:
        self._base = int(value)
        self._place()

    @property
    def state_in_graphs(self) -> bool:
        return all(m.state_in_graphs for m in (self.left, self.right) if m.state_need() is not None)

    def weights(self) -> dict[str, WeightWant]:
        return {**self.left.weights(), **self.right.weights()}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        for m in (self.left, self.right):
            m.bind({name: tensors[name] for name in m.weights()}, rt)

    def weight_bytes(self) -> int:
        return self.left.weight_bytes() + self.right.weight_bytes()

    def cache_need(self) -> CacheNeed | None:
        return None if self.cached is None else self.cached.cache_need()

    def aux_cache_needs(self) -> dict[str, CacheNeed]:
        return {} if self.cached is None else self.cached.aux_cache_needs()

    def state_need(self) -> StateNeed | None:
        n = sum(self._sizes())
        return StateNeed((n,), torch.float32) if n else None

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> "torch.Tensor | WeightedDeltas":
        rt = self.rt
        kept, ctx.residual = getattr(ctx, "residual", None), None       # both hand their output back: it is weighted first
        try:
            a = self.left.forward(x, ctx, cache if self.cached is self.left else None, state, writes_cache)
            b = self.right.forward(x, ctx, cache if self.cached is self.right else None, state, writes_cache)
        finally:
            ctx.residual = kept
        if getattr(ctx, "takes_weighted_deltas", False):
            return WeightedDeltas([(a, self.scales[0]), (b, self.scales[1])])       # the block's kernel forms the sum
        out = rt.workspace.get("parallel.delta", (1, x.shape[0], self.hidden_size), torch.float32)
        rt.ops.weighted_sum(a, self.scales[0], b, self.scales[1], out[0])
        return out


register_mixer("parallel_mixers", ParallelMixers)
