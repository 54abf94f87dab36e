"""Feed-forward as a mixture of experts: a router picks a few small gated feed-forwards per token."""

from __future__ import annotations

from typing import TYPE_CHECKING, Mapping

import torch

from .base import FeedForward, Runtime, WeightWant, register_feed_forward

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class RoutedExperts(FeedForward):
    """``num_experts`` gated feed-forwards of inner size ``intermediate_size`` without biases, of
    which every token uses ``top_k``.

    Router: z = W_r x (+ a bias, ``router_bias``) in 32-bit; the ``top_k`` largest are taken (the
    lower index among equals). ``score`` "sigmoid": the weights are sigmoid(z) as they are, not
    renormalized; "softmax_of_chosen": the softmax over the chosen z alone.

    ``weight_on`` "input": the weight multiplies the expert's input, the output is the sum over
    the chosen experts of expert(w x), which is not w expert(x) when the expert clamps; "output": the
    sum of w expert(x).

    Expert: with g = min(W_gate h, limit) and u = clamp(W_up h, -limit, limit) it is
    W_down (g sigmoid(gate_alpha g) (u + up_shift)); ``limit`` None, ``gate_alpha`` 1 and
    ``up_shift`` 0 make it W_down (silu(W_gate h) * W_up h).

    ``shared`` = {"intermediate_size": F, "gated": bool}: one more SiLU-gated feed-forward that every
    token uses, its output times sigmoid(w . x), one number per token, when ``gated``.

    The chosen experts' outputs (and the shared one's) come back as float32 slices ``[top_k (+ 1), T,
    hidden]`` that the norm behind adds up in ascending order, so a token's sum does not depend on
    what else is in the step. ``names``: "router" ("router_bias"), "gate"/"up"/"down" with ``{e}``
    for the expert, "shared_gate"/"shared_up"/"shared_down" ("shared_scale": the [1, hidden] row w)."""

    def __init__(self, hidden_size: int, num_experts: int, top_k: int, intermediate_size: int,
                 names: Mapping[str, str], limit: float | None, gate_alpha: float = 1.702, up_shift: float = 1.0,
                 score: str = "sigmoid", renormalize: bool = False, weight_on: str = "input",
                 router_bias: bool = False, shared: Mapping[str, object] | None = None) -> None:
        if score not in ("sigmoid", "softmax_of_chosen") or renormalize or weight_on not in ("input", "output"):
            raise ValueError("the router kernels score with a sigmoid (scores kept as weights) or with the softmax over the "
                             f"chosen logits, on the experts' input or output; got score={score!r}, "
                             f"renormalize={renormalize}, weight_on={weight_on!r}")
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top_k {top_k} of {num_experts} experts")
        self.hidden_size, self.num_experts, self.top_k = int(hidden_size), int(num_experts), int(top_k)
        self.intermediate_size = int(intermediate_size)
        self.names = dict(names)
        self.limit = float("inf") if limit is None else float(limit)
        self.gate_alpha, self.up_shift = float(gate_alpha), float(up_shift)
        self.router_mode = 0 if score == "sigmoid" else 1
        self.weight_on_output = weight_on == "output"
        self.router_bias = bool(router_bias)
        self.shared_size = None if shared is None else int(shared["intermediate_size"])
        self.shared_gated = shared is not None and bool(shared.get("gated", False))
        # Whether every call names the newer options, or the older form of the calls serves.
        self.plain_calls = self.router_mode == 0 and not self.weight_on_output and not self.router_bias

    def weights(self) -> dict[str, WeightWant]:
        h, f, n = self.hidden_size, self.intermediate_size, self.names
        want = {n["router"]: WeightWant((self.num_experts, h))}
        if self.router_bias:
            want[n["router_bias"]] = WeightWant((self.num_experts,), "bias")
        for e in range(self.num_experts):
            want[n["gate"].format(e=e)] = WeightWant((f, h))
            want[n["up"].format(e=e)] = WeightWant((f, h))
            want[n["down"].format(e=e)] = WeightWant((h, f))
        if self.shared_size is not None:
            want[n["shared_gate"]] = WeightWant((self.shared_size, h))
            want[n["shared_up"]] = WeightWant((self.shared_size, h))
            want[n["shared_down"]] = WeightWant((h, self.shared_size))
            if self.shared_gated:
                want[n["shared_scale"]] = WeightWant((1, h))
        return want

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        n, e_n = self.names, self.num_experts
        # The router stays 32-bit whatever the activation dtype.
        self.w_router = tensors[n["router"]].to(device=rt.device, dtype=torch.float32).contiguous()
        # ... and also stands in the activation dtype for steps whose logits a product kernel computes
        # (bfloat16 x bfloat16 products are exact in float32, where they are summed).
        self.w_router_act = self.w_router if rt.dtype == torch.float32 else rt.ops.prepare_matrix(tensors[n["router"]], rt)
        self.b_router = None
        if self.router_bias:
            self.b_router = tensors[n["router_bias"]].to(device=rt.device, dtype=torch.float32).contiguous()
        # Per expert the rows of gate, then of up: [E, 2F, H]; and down [E, H, F].
        gate_up = torch.stack([torch.cat([tensors[n["gate"].format(e=e)], tensors[n["up"].format(e=e)]], dim=0)
                               for e in range(e_n)])
        self.w_gate_up = rt.ops.prepare_matrix(gate_up, rt)
        self.w_down = rt.ops.prepare_matrix(torch.stack([tensors[n["down"].format(e=e)] for e in range(e_n)]), rt)
        self.w_shared_gate_up = self.w_shared_down = self.w_shared_scale = None
        if self.shared_size is not None:
            self.w_shared_gate_up = rt.ops.prepare_matrix(torch.cat([tensors[n["shared_gate"]], tensors[n["shared_up"]]], dim=0), rt)
            self.w_shared_down = rt.ops.prepare_matrix(tensors[n["shared_down"]], rt)
            if self.shared_gated:
                self.w_shared_scale = tensors[n["shared_scale"]].to(device=rt.device, dtype=torch.float32).reshape(-1).contiguous()

    def weight_bytes(self) -> int:
        """What a decode step of one token reads: the router, ``top_k`` experts and the shared one."""
        per_expert = (self.w_gate_up.numel() + self.w_down.numel()) // self.num_experts * self.w_down.element_size()
        shared = 0
        if self.w_shared_gate_up is not None:
            shared = (self.w_shared_gate_up.numel() + self.w_shared_down.numel()) * self.w_shared_down.element_size()
        return self.w_router.numel() * 4 + self.top_k * per_expert + shared

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, k = x.shape[0], self.top_k
        chosen = ws.get("moe.chosen", (t, k), torch.int32)
        weight = ws.get("moe.weight", (t, k), torch.float32)
        act = ws.get("moe.act", (t * k, self.intermediate_size), rt.dtype)
        slices = k + (1 if self.shared_size is not None else 0)
        out = ws.get("moe.out", (slices, t, self.hidden_size), torch.float32)
        if self.plain_calls:
            ops.moe_route(x, self.w_router, chosen, weight, self.w_router_act)
            ops.moe_experts(x, chosen, weight, self.w_gate_up, self.w_down, act, out[:k], self.gate_alpha, self.limit, self.up_shift)
        else:
            ops.moe_route(x, self.w_router, chosen, weight, self.w_router_act, bias=self.b_router, mode=self.router_mode)
            ops.moe_experts(x, chosen, weight, self.w_gate_up, self.w_down, act, out[:k], self.gate_alpha, self.limit,
                            self.up_shift, weight_on_output=self.weight_on_output)
        if self.shared_size is not None:
            shared_act = ws.get("moe.shared_act", (t, self.shared_size), rt.dtype)
            ops.linear_swiglu(x, self.w_shared_gate_up, shared_act)
            ops.linear(shared_act, self.w_shared_down, out[k])
            if self.w_shared_scale is not None:
                ops.row_gate(out[k], x, self.w_shared_scale)
        return out


register_feed_forward("routed_experts", RoutedExperts)
