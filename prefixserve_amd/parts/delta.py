"""Delta-rule mixers: a matrix per head as fixed-size state per request.

Both keep, per head, S [dim, vdim] in 32-bit and change it token by token: the state is decayed,
one direction of it is partly taken out, one outer product of a key and a value is written, and
the output is the state read with a query. They share one recurrence kernel (``ops.delta_scan``:
S' = d S; S = S' + (ps p)(c^T S*) + k (xs x)^T; o = S^T r) and differ in how its operands come
about. Neither needs positions or pages."""

from __future__ import annotations

import math
from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import Mixer, PositionEncoding, Runtime, StateNeed, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext

UNIT_EPS = 1e-6          # inside the root when a key or query is made a unit vector


class GatedDeltaRule(Mixer):
    """The gated delta rule. q and k (``num_kv_heads`` x ``head_dim``; head h uses vector
    h // (heads / kv_heads)) and v (``num_heads`` x ``value_dim``) each pass a causal convolution per
    channel over ``taps`` tokens (the last tap is the token's own, zeros in front of the sequence)
    and SiLU; q and k are made unit vectors, q also times head_dim^-1/2. Per head and token a write
    strength b = sigmoid(W_b h) and a decay g = exp(-exp(A) softplus(W_a h + dt)):
        S <- g S;   S <- S + k (b (v - S^T k))^T;   o = S^T q        (read after the write)
    then o / rms(o) per head times a weight of ``value_dim`` entries shared by the heads, times
    silu(W_g h), then the output matrix.

    Strength, decay (softplus, both exponentials), unit vectors, the recurrence and its state, and
    the norm are 32-bit in every mode. The per-request state is the convolutions' last ``taps`` - 1
    inputs, then S as [heads, value_dim, head_dim], in a slot the runner clears for a request that
    starts over. ``names``: "q", "k", "v", "q_conv", "k_conv", "v_conv", "strength", "decay",
    "decay_log", "decay_bias", "gate", "norm", "o"."""

    state_in_graphs = True

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int, num_kv_heads: int,
                 head_dim: int, value_dim: int, taps: int, names: Mapping[str, str], norm_eps: float) -> None:
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads = int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim, self.taps = int(head_dim), int(value_dim), int(taps)
        if self.num_kv_heads < 1 or self.num_heads % self.num_kv_heads:
            raise ValueError(f"{num_heads} heads not divisible by {num_kv_heads} key heads")
        if not 1 <= self.head_dim <= 256 or self.value_dim < 1 or not 1 <= self.taps <= 16:
            raise ValueError(f"key size {head_dim} (at most 256), value size {value_dim}, {taps} taps (at most 16)")
        self.names = dict(names)
        self.norm_eps = float(norm_eps)
        self.key_size = self.num_kv_heads * self.head_dim
        self.value_size = self.num_heads * self.value_dim
        self.channels = 2 * self.key_size + self.value_size          # what the convolutions run over: [q | k | v]
        self.tail = (self.taps - 1) * self.channels

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        return {n["q"]: WeightWant((self.key_size, h)), n["k"]: WeightWant((self.key_size, h)),
                n["v"]: WeightWant((self.value_size, h)),
                n["q_conv"]: WeightWant((self.key_size, self.taps), "bias"),
                n["k_conv"]: WeightWant((self.key_size, self.taps), "bias"),
                n["v_conv"]: WeightWant((self.value_size, self.taps), "bias"),
                n["strength"]: WeightWant((self.num_heads, h)), n["decay"]: WeightWant((self.num_heads, h)),
                n["decay_log"]: WeightWant((self.num_heads,), "bias"), n["decay_bias"]: WeightWant((self.num_heads,), "bias"),
                n["gate"]: WeightWant((self.value_size, h)), n["norm"]: WeightWant((self.value_dim,), "norm"),
                n["o"]: WeightWant((h, self.value_size))}

    def state_need(self) -> StateNeed:
        return StateNeed((self.tail + self.num_heads * self.value_dim * self.head_dim,), torch.float32)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n, dev = self.names, rt.device

        def f32(name: str) -> torch.Tensor:
            return tensors[n[name]].to(torch.float32).contiguous().to(dev)

        # [q | k | v | gate] from one product in the activation dtype; the two numbers per head that
        # enter the recurrence from a second one with 32-bit output.
        self.w_in = rt.ops.prepare_matrix(torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]], tensors[n["gate"]]], dim=0), rt)
        self.w_coef = rt.ops.prepare_matrix(torch.cat([tensors[n["strength"]], tensors[n["decay"]]], dim=0), rt)
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        self.conv_w = torch.cat([f32("q_conv"), f32("k_conv"), f32("v_conv")], dim=0).contiguous()
        self.decay_log, self.decay_bias, self.norm_w = f32("decay_log"), f32("decay_bias"), f32("norm")

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_coef, self.w_o, self.conv_w))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, hd = x.shape[0], self.num_heads
        assert state is not None, "the delta rule keeps its state in a slot"
        rows = ws.get("delta.in", (t, self.channels + self.value_size), rt.dtype)         # [q | k | v | gate]
        ops.linear(x, self.w_in, rows)
        gates = ws.get("delta.gates", (t, 2 * hd), torch.float32)                         # [strength logits | decay inputs]
        ops.linear(x, self.w_coef, gates)
        u = ws.get("delta.u", (t, self.channels), torch.float32)
        ops.short_conv(rows, 0, self.conv_w, u, state, self.state_base, ctx, silu=True)
        coef = ws.get("delta.coef", (t, 3 * hd), torch.float32)                           # [g | -b | b]
        ops.gated_delta_prepare(u, self.num_kv_heads, self.head_dim, gates, self.decay_log, self.decay_bias, coef,
                                self.head_dim ** -0.5, UNIT_EPS)
        o = ws.get("delta.o", (t, self.value_size), torch.float32)
        k_col, v_col = self.key_size, 2 * self.key_size
        ops.delta_scan(keys=(u, k_col), directions=(u, k_col), removals=(u, k_col), queries=(u, 0),
                       key_groups=self.num_kv_heads, decay_vectors=None, decay=(coef, 0), removal_scale=(coef, hd),
                       value_scale=(coef, 2 * hd), values=(u, v_col), out=o, state=state, state_offset=self.state_base + self.tail, ctx=ctx,
                       heads=hd, dim=self.head_dim, vdim=self.value_dim, reads_decayed=True)
        out = ws.get("delta.out", (t, self.value_size), rt.dtype)
        ops.heads_norm_gate(o, hd, self.value_dim, self.norm_w, False, self.norm_eps, rows, self.channels, "silu", out)
        return ops.linear_to_residual(out, self.w_o, "delta.delta", getattr(ctx, "residual", None))


class GeneralizedDeltaRule(Mixer):
    """A delta rule with a decay and a removal rate per key channel. r, k, v = W h (``num_heads`` x
    ``head_dim`` each); w = exp(-``decay_floor`` sigmoid(W_2 tanh(W_1 h) + w0)) and a = sigmoid(W_a h
    + bias), per head and key channel; with n = k / |k|:
        S <- diag(w) S - (a * n)(n^T S) + k v^T      (both terms read the state before the token)
        o = S^T r
    then o / rms(o) per head times a weight over all heads, times sigmoid(W_g h), then the output
    matrix. With ``decay_floor`` = e^-1/2 no channel decays faster than exp(-0.607) a token.

    The decay (tanh, sigmoid, exponential), the rate, the unit key, the recurrence and its state,
    and the norm are 32-bit in every mode; the state is S as [heads, head_dim (values), head_dim
    (keys)]. ``names``: "r", "k", "v", "gate", "rate", "rate_bias", "decay_in", "decay_out",
    "decay_bias", "norm", "o"."""

    state_in_graphs = True

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int, head_dim: int,
                 decay_rank: int, names: Mapping[str, str], norm_eps: float, decay_floor: float = math.exp(-0.5)) -> None:
        self.hidden_size, self.num_heads, self.head_dim = int(hidden_size), int(num_heads), int(head_dim)
        self.decay_rank = int(decay_rank)
        if self.num_heads < 1 or not 1 <= self.head_dim <= 256 or self.decay_rank < 1:
            raise ValueError(f"{num_heads} heads of {head_dim} (at most 256), decay rank {decay_rank}")
        self.names = dict(names)
        self.norm_eps, self.decay_floor = float(norm_eps), float(decay_floor)
        self.size = self.num_heads * self.head_dim

    def weights(self) -> dict[str, WeightWant]:
        h, n, s, r = self.hidden_size, self.names, self.size, self.decay_rank
        return {n["r"]: WeightWant((s, h)), n["k"]: WeightWant((s, h)), n["v"]: WeightWant((s, h)),
                n["gate"]: WeightWant((s, h)), n["rate"]: WeightWant((s, h)), n["rate_bias"]: WeightWant((s,), "bias"),
                n["decay_in"]: WeightWant((r, h)), n["decay_out"]: WeightWant((s, r)),
                n["decay_bias"]: WeightWant((s,), "bias"), n["norm"]: WeightWant((s,), "norm"), n["o"]: WeightWant((h, s))}

    def state_need(self) -> StateNeed:
        return StateNeed((self.num_heads * self.head_dim * self.head_dim,), torch.float32)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n, dev = self.names, rt.device

        def f32(name: str) -> torch.Tensor:
            return tensors[n[name]].to(torch.float32).contiguous().to(dev)

        # [r | k | v | gate | rate logits | the decay map's inner values] from one product.
        self.w_in = rt.ops.prepare_matrix(torch.cat([tensors[n[key]] for key in ("r", "k", "v", "gate", "rate", "decay_in")], dim=0), rt)
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        self.rate_bias, self.decay_bias, self.norm_w = f32("rate_bias"), f32("decay_bias"), f32("norm")
        self.decay_out = f32("decay_out").t().contiguous()       # [rank, heads dim]: a kernel's lanes read channels side by side

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o, self.decay_out))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, s, hd = x.shape[0], self.size, self.num_heads
        assert state is not None, "the delta rule keeps its state in a slot"
        rows = ws.get("gdelta.in", (t, 5 * s + self.decay_rank), rt.dtype)
        ops.linear(x, self.w_in, rows)
        operands = ws.get("gdelta.ops", (t, 6 * s), torch.float32)                        # [r | k | v | w | p | c]
        ops.general_delta_prepare(rows, 0, s, 2 * s, 4 * s, 5 * s, self.rate_bias, self.decay_out, self.decay_bias, operands,
                                  hd, self.head_dim, self.decay_floor, UNIT_EPS)
        o = ws.get("gdelta.o", (t, s), torch.float32)
        ops.delta_scan(keys=(operands, s), directions=(operands, 5 * s), removals=(operands, 4 * s), queries=(operands, 0),
                       key_groups=hd, decay_vectors=(operands, 3 * s), decay=None, removal_scale=None, value_scale=None,
                       values=(operands, 2 * s), out=o, state=state, state_offset=self.state_base, ctx=ctx, heads=hd, dim=self.head_dim,
                       vdim=self.head_dim, reads_decayed=False)
        out = ws.get("gdelta.out", (t, s), rt.dtype)
        ops.heads_norm_gate(o, hd, self.head_dim, self.norm_w, True, self.norm_eps, rows, 3 * s, "sigmoid", out)
        return ops.linear_to_residual(out, self.w_o, "gdelta.delta", getattr(ctx, "residual", None))


register_mixer("gated_delta_rule", GatedDeltaRule)
register_mixer("generalized_delta_rule", GeneralizedDeltaRule)
