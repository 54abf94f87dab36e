"""Recurrent mixers with a matrix per head as fixed-size state: a selective state space layer with a
scalar decay per head and step, and a matrix memory with exponential gates."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import Mixer, PositionEncoding, Runtime, StateNeed, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class SelectiveStateSpace(Mixer):
    """A state space layer whose decay is one number per head and token. One input matrix gives
    [z | x | B | C | dt] with x, z of ``num_heads`` x ``value_dim`` (= inner), B, C of ``groups`` x
    ``state_dim`` (head h uses group h // (heads / groups)) and dt one number per head. [x | B | C]
    pass a causal convolution per channel over ``taps`` tokens (with a bias; the last tap is the
    token's own, zeros in front of the sequence) and SiLU. With d = softplus(dt + dt_bias), per head
        S <- exp(-exp(A) d) S + d B x^T        (S is state_dim x value_dim)
        y = S^T C + D x
    then y * silu(z), an RMS norm over each of ``norm_groups`` equal parts of the inner size, a
    weight of inner entries, and the output matrix.

    The step size (softplus), both exponentials, the recurrence and its state, and the norm are
    32-bit in every mode; dt comes from a product of its own with 32-bit output. The per-request
    state is the convolution's last ``taps`` - 1 inputs, then S as [heads, value_dim, state_dim].
    ``names``: "in", "conv", "conv_bias", "dt_bias", "decay_log", "skip", "norm", "o"."""

    state_in_graphs = True

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int, value_dim: int,
                 state_dim: int, groups: int, taps: int, norm_groups: int, names: Mapping[str, str], norm_eps: float) -> None:
        self.hidden_size = int(hidden_size)
        self.num_heads, self.value_dim, self.state_dim = int(num_heads), int(value_dim), int(state_dim)
        self.groups, self.taps, self.norm_groups = int(groups), int(taps), int(norm_groups)
        self.inner = self.num_heads * self.value_dim
        if self.groups < 1 or self.num_heads % self.groups:
            raise ValueError(f"{num_heads} heads not divisible by {groups} groups")
        if self.norm_groups < 1 or self.inner % self.norm_groups:
            raise ValueError(f"inner size {self.inner} not divisible into {norm_groups} norm groups")
        if not 1 <= self.state_dim <= 256 or self.value_dim < 1 or not 1 <= self.taps <= 16:
            raise ValueError(f"state size {state_dim} (at most 256), value size {value_dim}, {taps} taps (at most 16)")
        self.names = dict(names)
        self.norm_eps = float(norm_eps)
        self.channels = self.inner + 2 * self.groups * self.state_dim       # what the convolution runs over: [x | B | C]
        self.tail = (self.taps - 1) * self.channels

    def weights(self) -> dict[str, WeightWant]:
        h, n, hd = self.hidden_size, self.names, self.num_heads
        return {n["in"]: WeightWant((self.inner + self.channels + hd, h)),
                n["conv"]: WeightWant((self.channels, self.taps), "bias"), n["conv_bias"]: WeightWant((self.channels,), "bias"),
                n["dt_bias"]: WeightWant((hd,), "bias"), n["decay_log"]: WeightWant((hd,), "bias"),
                n["skip"]: WeightWant((hd,), "norm"), n["norm"]: WeightWant((self.inner,), "norm"),
                n["o"]: WeightWant((h, self.inner))}

    def state_need(self) -> StateNeed:
        return StateNeed((self.tail + self.inner * self.state_dim,), torch.float32)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n, dev = self.names, rt.device

        def f32(name: str) -> torch.Tensor:
            return tensors[n[name]].to(torch.float32).contiguous().to(dev)

        w_in = tensors[n["in"]]
        split = self.inner + self.channels
        self.w_in = rt.ops.prepare_matrix(w_in[:split].contiguous(), rt)       # [z | x | B | C] in the activation dtype
        self.w_dt = rt.ops.prepare_matrix(w_in[split:].contiguous(), rt)       # the step size: a product with 32-bit output
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        self.conv_w, self.conv_b = f32("conv"), f32("conv_bias")
        self.dt_bias, self.decay_log, self.skip, self.norm_w = f32("dt_bias"), f32("decay_log"), f32("skip"), f32("norm")

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_dt, self.w_o, self.conv_w))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, hd = x.shape[0], self.num_heads
        assert state is not None, "the state space layer keeps its state in a slot"
        rows = ws.get("ssm.in", (t, self.inner + self.channels), rt.dtype)
        ops.linear(x, self.w_in, rows)
        dt = ws.get("ssm.dt", (t, self.num_heads), torch.float32)
        ops.linear(x, self.w_dt, dt)
        u = ws.get("ssm.u", (t, self.channels), torch.float32)                         # [x | B | C]
        ops.short_conv(rows, self.inner, self.conv_w, u, state, self.state_base, ctx, silu=True, bias=self.conv_b)
        coef = ws.get("ssm.coef", (t, 3 * hd), torch.float32)                          # [decay | 0 | step size]
        ops.state_space_prepare(dt, self.dt_bias, self.decay_log, coef)
        # S <- decay S + B (step x)^T, y = S^T C: the delta rules' recurrence with nothing taken out.
        y = ws.get("ssm.y", (t, self.inner), torch.float32)
        b_col = self.inner
        ops.delta_scan(keys=(u, b_col), directions=(u, b_col), removals=(u, b_col), queries=(u, b_col + self.groups * self.state_dim),
                       key_groups=self.groups, decay_vectors=None, decay=(coef, 0), removal_scale=(coef, hd),
                       value_scale=(coef, 2 * hd), values=(u, 0), out=y, state=state, state_offset=self.state_base + self.tail,
                       ctx=ctx, heads=hd, dim=self.state_dim, vdim=self.value_dim, reads_decayed=True, no_removal=True)
        out = ws.get("ssm.out", (t, self.inner), rt.dtype)
        ops.gated_group_norm(y, u, 0, self.skip, hd, rows, 0, self.norm_w, self.norm_groups, self.norm_eps, out)
        return ops.linear_to_residual(out, self.w_o, "ssm.delta", getattr(ctx, "residual", None))


class MatrixMemory(Mixer):
    """A matrix memory per head with exponential gates and a running maximum. q (times
    head_dim^-1/2), k of ``num_heads`` x ``head_dim`` and v of ``num_heads`` x ``value_dim``; per
    head and token a log input gate i = cap tanh((W_i x + b_i) / cap) and a log forget gate
    f = logsigmoid(cap tanh((W_f x + b_f) / cap)). With S, n and m starting at zero:
        m' = max(f + m, i);   S <- exp(f + m - m') S + exp(i - m') k v^T;   n likewise with k alone
        o = S^T q / (max(|n . q|, exp(-m')) + 1e-6)
    then o / rms(o) per head, a weight over all heads, times sigmoid(W_g x), then the output matrix.

    The gates (tanh, logsigmoid, exponentials), the recurrence with S, n and m, the read-out and
    the norm are 32-bit in every mode; the gates' inputs come from a product of their own with
    32-bit output. n is carried as one more column of S (a value that is always 1), so the
    per-request state is S as [heads, value_dim + 1, head_dim], then m [heads]. ``names``: "q", "k", "v", "gate", "input_gate", "input_bias",
    "forget_gate", "forget_bias", "norm", "o"."""

    state_in_graphs = True
    READ_EPS = 1e-6          # added to the read-out's denominator

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int, head_dim: int,
                 value_dim: int, gate_cap: float, names: Mapping[str, str], norm_eps: float) -> None:
        self.hidden_size = int(hidden_size)
        self.num_heads, self.head_dim, self.value_dim = int(num_heads), int(head_dim), int(value_dim)
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        if self.num_heads < 1 or not 1 <= self.head_dim <= 256 or self.value_dim < 1 or not self.gate_cap > 0:
            raise ValueError(f"{num_heads} heads of {head_dim} (at most 256) and {value_dim}, gate cap {gate_cap}")
        self.names = dict(names)
        self.key_size, self.value_size = self.num_heads * self.head_dim, self.num_heads * self.value_dim

    def weights(self) -> dict[str, WeightWant]:
        h, n, hd = self.hidden_size, self.names, self.num_heads
        return {n["q"]: WeightWant((self.key_size, h)), n["k"]: WeightWant((self.key_size, h)),
                n["v"]: WeightWant((self.value_size, h)), n["gate"]: WeightWant((self.value_size, h)),
                n["input_gate"]: WeightWant((hd, h)), n["input_bias"]: WeightWant((hd,), "bias"),
                n["forget_gate"]: WeightWant((hd, h)), n["forget_bias"]: WeightWant((hd,), "bias"),
                n["norm"]: WeightWant((self.value_size,), "norm"), n["o"]: WeightWant((h, self.value_size))}

    def state_need(self) -> StateNeed:
        return StateNeed((self.num_heads * ((self.value_dim + 1) * self.head_dim + 1),), torch.float32)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n, dev = self.names, rt.device

        def f32(name: str) -> torch.Tensor:
            return tensors[n[name]].to(torch.float32).contiguous().to(dev)

        self.w_in = rt.ops.prepare_matrix(torch.cat([tensors[n[key]] for key in ("q", "k", "v", "gate")], dim=0), rt)
        self.w_gates = rt.ops.prepare_matrix(torch.cat([tensors[n["input_gate"]], tensors[n["forget_gate"]]], dim=0), rt)
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        self.gate_bias = torch.cat([f32("input_bias"), f32("forget_bias")]).contiguous()
        self.norm_w = f32("norm")

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_gates, self.w_o))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, hd = x.shape[0], self.num_heads
        assert state is not None, "the matrix memory keeps its state in a slot"
        rows = ws.get("memory.in", (t, 2 * self.key_size + 2 * self.value_size), rt.dtype)       # [q | k | v | gate]
        ops.linear(x, self.w_in, rows)
        gates = ws.get("memory.gates", (t, 2 * hd), torch.float32)                                 # [input | forget] inputs
        ops.linear(x, self.w_gates, gates)
        vd = self.value_dim + 1
        m_at = self.state_base + hd * vd * self.head_dim
        coef = ws.get("memory.coef", (t, 4 * hd), torch.float32)                                   # [keep | 0 | write | exp(-m)]
        ops.matrix_memory_gates(gates, self.gate_bias, self.gate_cap, coef, state, m_at, ctx)
        u = ws.get("memory.u", (t, 2 * self.key_size), torch.float32)                              # [q scaled | k]
        vals = ws.get("memory.v", (t, hd * vd), torch.float32)                                     # per head [v | 1]
        ops.matrix_memory_operands(rows, 0, self.key_size, 2 * self.key_size, hd, self.head_dim, self.value_dim,
                                   self.head_dim ** -0.5, u, vals)
        # S <- keep S + k (write v)^T with n as the column whose value is 1: the delta rules' recurrence
        # with nothing taken out; the read-out of that column is n . q.
        raw = ws.get("memory.raw", (t, hd * vd), torch.float32)
        k_col = self.key_size
        ops.delta_scan(keys=(u, k_col), directions=(u, k_col), removals=(u, k_col), queries=(u, 0), key_groups=hd,
                       decay_vectors=None, decay=(coef, 0), removal_scale=(coef, hd), value_scale=(coef, 2 * hd),
                       values=(vals, 0), out=raw, state=state, state_offset=self.state_base, ctx=ctx, heads=hd,
                       dim=self.head_dim, vdim=vd, reads_decayed=True, no_removal=True)
        out = ws.get("memory.out", (t, self.value_size), rt.dtype)
        ops.memory_read_norm_gate(raw, coef, 3 * hd, hd, self.value_dim, self.READ_EPS, self.norm_w, self.norm_eps, rows,
                                  2 * self.key_size + self.value_size, out)
        return ops.linear_to_residual(out, self.w_o, "memory.delta", getattr(ctx, "residual", None))


register_mixer("selective_state_space", SelectiveStateSpace)
register_mixer("matrix_memory", MatrixMemory)
