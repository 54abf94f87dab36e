"""Transforms of the residual stream: a factor behind the token table, and the re-entry into a
stretch of layers that is passed through several times."""

from __future__ import annotations

from typing import TYPE_CHECKING, Mapping

import torch

from .base import Runtime, Transform, WeightWant, register_transform

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class ScaleStream(Transform):
    """t <- factor * t, in 32-bit: the token table's rows times a constant."""

    def __init__(self, hidden_size: int, vocab_size: int, factor: float) -> None:
        self.factor = float(factor)

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        if self.factor != 1.0:
            self.rt.ops.stream_affine(t, self.factor, None)


class StreamReentry(Transform):
    """In front of every pass through a repeated stretch of layers: x <- W [x; x0] + step[pass],
    where x0 is the token table's output (behind its own transforms) and ``step`` has one row per
    pass. The product's operands are in the activation dtype; its sums and the added row are
    32-bit and become the new stream. ``names``: "in" ([hidden, 2 hidden], x's columns first)
    and "step" ([passes, hidden])."""

    needs_embedding_output = True

    def __init__(self, hidden_size: int, vocab_size: int, passes: int, names: Mapping[str, str]) -> None:
        self.hidden_size, self.passes = int(hidden_size), int(passes)
        self.names = dict(names)

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        return {n["in"]: WeightWant((h, 2 * h)), n["step"]: WeightWant((self.passes, h), "bias")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        self.w_in = rt.ops.prepare_matrix(tensors[self.names["in"]], rt)
        self.steps = tensors[self.names["step"]].to(device=rt.device, dtype=torch.float32).contiguous()

    def weight_bytes(self) -> int:
        return self.w_in.numel() * self.w_in.element_size()

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        rt, ops = self.rt, self.rt.ops
        if not 0 <= ctx.pass_index < self.passes:
            raise ValueError(f"pass {ctx.pass_index} of {self.passes}")
        both = rt.workspace.get("reentry.in", (t.shape[0], 2 * self.hidden_size), rt.dtype)
        ops.concat_to_activation(t, ctx.embedding_output, both)
        ops.linear(both, self.w_in, t)
        ops.stream_affine(t, 1.0, self.steps[ctx.pass_index])


class SinusoidalPositions(Transform):
    """t[row, 2i] += sin(p f_i), t[row, 2i + 1] += cos(p f_i) with f_i = base^(-2i / hidden) and p the
    row's position: the fixed table of sines added to the token table's rows. The frequencies are
    formed in float64 once; the kernel multiplies and reduces the angle in double before the 32-bit
    sine, so far positions keep their digits. No weights."""

    def __init__(self, hidden_size: int, vocab_size: int, base: float = 10000.0) -> None:
        self.hidden_size, self.base = int(hidden_size), float(base)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        i = torch.arange((self.hidden_size + 1) // 2, dtype=torch.float64)
        self.freq = torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / self.hidden_size).to(rt.device).contiguous()

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        if rows is not None:
            raise ValueError("the sinusoid is added to the whole stream, row by row in order")
        self.rt.ops.add_sinusoid(t, ctx.positions, self.freq)


register_transform("scale", ScaleStream)
register_transform("sinusoidal_positions", SinusoidalPositions)
register_transform("reentry", StreamReentry)
