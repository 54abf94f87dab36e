"""RMSNorm fused with the residual sum in front of it."""

from __future__ import annotations

from typing import Mapping

import torch

from .base import Norm, NormedRows, Runtime, WeightWant, register_norm


class RMSNorm(Norm):
    """weight * x * rsqrt(mean(x^2) + eps), eps inside the root; statistics, scale and the
    residual sum in 32-bit (prefixserve/model/llama.py:63-69 of the reference upcasts the
    same way). The weight is used in the dtype it is stored in. ``unit_offset``: the stored
    tensor is the weight's distance from one, the factor is 1 + w (formed in 32-bit and kept so:
    rounding 1 + w to the stored 16 bits would drop most of w). ``scalar``: the stored weight is one
    number for all coordinates (a tensor without dimensions); it is spread over the width at bind
    time, in 32-bit."""

    def __init__(self, hidden_size: int, eps: float, name: str = "weight", unit_offset: bool = False,
                 scalar: bool = False) -> None:
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.name = name
        self.unit_offset = bool(unit_offset)
        self.scalar = bool(scalar)

    def weights(self) -> dict[str, WeightWant]:
        return {self.name: WeightWant(() if self.scalar else (self.hidden_size,), "offset" if self.unit_offset else "norm")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        w = tensors[self.name]
        if self.scalar:
            w = w.to(torch.float32).reshape(1).expand(self.hidden_size)
        if w.dtype not in (torch.bfloat16, torch.float32):
            w = w.to(torch.float32)
        if self.unit_offset:
            w = 1.0 + w.to(torch.float32)
        self.weight = w.to(rt.device).contiguous()

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()

    def _lazy(self, count: int) -> bool:
        """Whether the kernels of this runtime normalize ``count`` rows of this width themselves."""
        fuses = getattr(self.rt.ops, "fuses_norm", None)
        return fuses is not None and fuses(count, self.hidden_size, self.rt.dtype)

    def add_norm(self, residual: torch.Tensor, delta: torch.Tensor | None, out_name: str,
                 lazy: bool = False) -> torch.Tensor | NormedRows:
        rt = self.rt
        if lazy and delta is None and self._lazy(residual.shape[0]):
            return NormedRows(residual, self.weight, self.eps, rt.dtype)
        out = rt.workspace.get(out_name, (residual.shape[0], self.hidden_size), rt.dtype)
        rt.ops.add_rmsnorm(residual, delta, self.weight, self.eps, out)
        return out

    def add_norm_rows(self, residual: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor,
                      out_name: str, lazy: bool = False) -> torch.Tensor | NormedRows:
        rt = self.rt
        if lazy and delta is None and self._lazy(rows.shape[0]):
            return NormedRows(residual, self.weight, self.eps, rt.dtype, rows)
        out = rt.workspace.get(out_name, (rows.shape[0], self.hidden_size), rt.dtype)
        rt.ops.add_rmsnorm_rows(residual, delta, rows, self.weight, self.eps, out)
        return out


    def norm_of_sum(self, residual: torch.Tensor, delta: torch.Tensor | None, alpha: float,
                    out_name: str) -> torch.Tensor:
        rt = self.rt
        out = None if rt.dtype == torch.float32 else rt.workspace.get(out_name, tuple(residual.shape), rt.dtype)
        rt.ops.scaled_add_rmsnorm(residual, delta, float(alpha), self.weight, self.eps, out)
        return residual if out is None else out


class LayerNorm(Norm):
    """(x - mean) / sqrt(mean((x - mean)^2) + eps) * weight + bias, eps inside the root; sums,
    statistics and the residual sum in 32-bit, weight and bias widened to 32-bit once.

    Beside the interface every norm has it offers ``add_normed``: the norm *behind* a sub-layer,
    stream += norm(delta), fused with the norm in front of the next sub-layer where there is one.
    ``name`` / ``bias_name``: the two tensors' names."""

    def __init__(self, hidden_size: int, eps: float, name: str = "weight", bias_name: str | None = None) -> None:
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.name = name
        self.bias_name = bias_name if bias_name is not None else name + ".b"

    def weights(self) -> dict[str, WeightWant]:
        return {self.name: WeightWant((self.hidden_size,), "norm"), self.bias_name: WeightWant((self.hidden_size,), "bias")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        self.weight = tensors[self.name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.bias = tensors[self.bias_name].to(device=rt.device, dtype=torch.float32).contiguous()
        self.terms = (self.weight, self.bias, self.eps)          # what the kernel takes for one norm

    def weight_bytes(self) -> int:
        return 4 * (self.weight.numel() + self.bias.numel())

    def add_norm(self, residual: torch.Tensor, delta: torch.Tensor | None, out_name: str,
                 lazy: bool = False) -> torch.Tensor:
        rt = self.rt
        if delta is not None:
            rt.ops.residual_add(residual, delta)
        out = rt.workspace.get(out_name, (residual.shape[0], self.hidden_size), rt.dtype)
        rt.ops.layernorm_step(residual, None, None, self.terms, out)
        return out

    def add_norm_rows(self, residual: torch.Tensor, delta: torch.Tensor | None, rows: torch.Tensor,
                      out_name: str, lazy: bool = False) -> torch.Tensor:
        rt = self.rt
        if delta is not None:
            rt.ops.residual_add(residual, delta)
        out = rt.workspace.get(out_name, (rows.shape[0], self.hidden_size), rt.dtype)
        rt.ops.layernorm_step(residual, None, None, self.terms, out, rows=rows)
        return out

    def add_normed(self, residual: torch.Tensor, delta: torch.Tensor, then: "LayerNorm | None" = None,
                   out_name: str = "block.x") -> torch.Tensor | None:
        """residual (float32 [T,H], in place) += self(delta), where ``delta`` is [T,H] in the
        activation dtype or [S,T,H] float32 slices that are summed first. With ``then``, another
        norm of this kind, returns then(residual) in the activation dtype from the same kernel."""
        rt = self.rt
        out = None if then is None else rt.workspace.get(out_name, (residual.shape[0], self.hidden_size), rt.dtype)
        rt.ops.layernorm_step(residual, delta, self.terms, None if then is None else then.terms, out)
        return out


register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
