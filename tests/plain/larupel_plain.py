"""Plain, slow Larupel: the oracle the engine's Larupel tests are compared with.

Whole sequences, no cache, no paging, no batching, no state handed on; numpy float64 only; one
function per mechanism. It shares no code with the product package (its file reader is the plain
Llama oracle's, which is test code too).

The design, in this file's notation. The token table's row gets a sinusoid of the position
added (``sinusoid``). A layer has a norm in front of and behind each sub-layer,
    x <- x + B1(mix(A1(x))),    x <- x + B2(ff(A2(x)))        (the second only with a feed-forward)
where every norm is a layer norm with weight and bias (``layer_norm``). The mixer is one of
  * ``delta``: a gated delta rule. q, k (shared by groups of heads) and v each pass a short causal
    convolution and SiLU; q and k become unit vectors, q is scaled by dim^-1/2; per head and token
    a write strength b = sigmoid(.) and a decay g = exp(-exp(A) softplus(. + dt)). The state
    S [dim, vdim] goes S <- g S; S <- S + k (b (v - S^T k))^T; the output is S^T q, read after
    the write (``gated_delta``). Output: per-head RMS norm with a weight shared by the heads,
    times silu(gate), then the output matrix.
  * ``general_delta``: a delta rule with a decay per key channel and a removal rate per key
    channel: with n = k / |k|, S <- diag(w) S - (a * n) (n^T S) + k v^T where both terms read the
    old S; output S^T r (``generalized_delta``). w = exp(-e^-1/2 sigmoid(low-rank(h) + w0)),
    a = sigmoid(.). Output: per-head RMS norm, a weight over all heads, times sigmoid(gate).
  * ``attention``: causal grouped-query softmax attention without rotation; q and k get an RMS
    norm per head with a weight shared by the heads; the score is q.k * scale * temp[head]. A layer
    with ``kv_from: j`` brings no keys and values and reads layer j's (as normed there).
The feed-forward is dense, down(gelu_tanh(gate) * up), or a mixture of experts: the router's
logits (with a bias) pick the ``top`` largest, whose weights are the softmax over the picked
logits alone; experts are down(silu(gate) * up); a shared expert of the same form runs for every
token, times sigmoid(one number per token).
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from typing import Any

import numpy as np

from .llama_plain import read_safetensors, round_bf16  # noqa: F401  (test-side helpers)

DECAY_FLOOR = math.exp(-0.5)     # the generalized rule's decay is exp(-DECAY_FLOOR * sigmoid(.)): never under exp(-0.607)
UNIT_EPS = 1e-6                  # inside the root when keys and queries are made unit vectors

# ------------------------------------------------------------------- formulas


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def silu(z: np.ndarray) -> np.ndarray:
    return z * sigmoid(z)


def softplus(z: np.ndarray) -> np.ndarray:
    return np.logaddexp(0.0, z)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sinusoid(positions: np.ndarray, width: int) -> np.ndarray:
    """[n, width]: entries 2i and 2i + 1 are sin and cos of p * 10000^(-2i / width)."""
    e = np.arange(width)
    freq = 10000.0 ** (-2.0 * (e // 2) / width)
    ang = positions.astype(np.float64)[:, None] * freq[None, :]
    return np.where(e % 2 == 0, np.sin(ang), np.cos(ang))


def layer_norm(x: np.ndarray, weight: np.ndarray, bias: np.ndarray, eps: float) -> np.ndarray:
    m = x.mean(axis=-1, keepdims=True)
    d = x - m
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + eps) * weight + bias


def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def unit_length(x: np.ndarray) -> np.ndarray:
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + UNIT_EPS)


def short_conv(x: np.ndarray, taps: np.ndarray) -> np.ndarray:
    """x [n, channels], taps [channels, t]: y[p, c] = sum_j taps[c, j] x[p - (t - 1) + j, c], zeros before 0."""
    n, t = x.shape[0], taps.shape[1]
    padded = np.concatenate([np.zeros((t - 1, x.shape[1])), x], axis=0)
    y = np.zeros_like(x)
    for j in range(t):
        y += padded[j: j + n] * taps[:, j][None, :]
    return y


def gated_delta(q: np.ndarray, k: np.ndarray, v: np.ndarray, strength: np.ndarray, decay: np.ndarray) -> np.ndarray:
    """One head. q, k [n, dim], v [n, vdim], strength and decay [n]. Token by token from S = 0."""
    n, dim = k.shape
    s = np.zeros((dim, v.shape[1]))
    out = np.zeros_like(v)
    for t in range(n):
        s = decay[t] * s
        write = strength[t] * (v[t] - s.T @ k[t])
        s = s + np.outer(k[t], write)
        out[t] = s.T @ q[t]
    return out


def generalized_delta(r: np.ndarray, k: np.ndarray, v: np.ndarray, w: np.ndarray, a: np.ndarray) -> np.ndarray:
    """One head. r, k, w, a [n, dim], v [n, vdim]. Token by token from S = 0; decay and removal both read the old S."""
    n, dim = k.shape
    s = np.zeros((dim, v.shape[1]))
    out = np.zeros_like(v)
    unit = unit_length(k)
    for t in range(n):
        s = w[t][:, None] * s - np.outer(a[t] * unit[t], unit[t] @ s) + np.outer(k[t], v[t])
        out[t] = s.T @ r[t]
    return out


def causal_softmax_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float) -> np.ndarray:
    """One head; every query sees the keys at or before it. Returns (output, weights)."""
    n = q.shape[0]
    s = (q @ k.T) * scale
    s = np.where(np.arange(n)[None, :] <= np.arange(n)[:, None], s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return p @ v, p


def route(logits: np.ndarray, top: int) -> tuple[np.ndarray, np.ndarray]:
    """logits [n, experts] -> (chosen [n, top], the largest first and the lower index among equals;
    weights [n, top] = softmax over the chosen logits alone)."""
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :top]
    z = np.take_along_axis(logits, order, axis=-1)
    z = np.exp(z - z.max(axis=-1, keepdims=True))
    return order, z / z.sum(axis=-1, keepdims=True)


def gated_ff(h: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray, act, r=lambda x: x) -> np.ndarray:
    """``r`` rounds what an engine would hold in its activation type: the gated product."""
    return r(act(h @ gate.T) * (h @ up.T)) @ down.T


# ---------------------------------------------------------------------- model


class PlainLarupel:
    """``weights``: name -> float64 array (as the checkpoint names them); ``cfg``: config.json as a dict."""

    def __init__(self, cfg: dict[str, Any], weights: dict[str, np.ndarray], bf16: bool = False) -> None:
        """``bf16``: the yardstick for a 16-bit engine. The outputs of the norms, of the products with
        weight matrices and of the activations behind them, queries and keys as attention uses them, and
        every sub-layer's output are rounded to bfloat16; everything the recurrences take in behind their
        projections, scores, softmaxes, router logits and the stream are not. How far that moves the logits
        of a model is what an engine that computes in bfloat16 may be off by, whatever its order of sums."""
        self.r = (lambda x: round_bf16(np.asarray(x, dtype=np.float32)).astype(np.float64)) if bf16 else (lambda x: x)
        self.cfg = cfg
        self.w = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
        self.eps = float(cfg["norm"]["eps"])
        self.width = int(cfg["width"])

    @classmethod
    def from_dir(cls, model_dir: str | Path, bf16: bool = False) -> "PlainLarupel":
        model_dir = Path(model_dir)
        cfg = json.loads((model_dir / "config.json").read_text())
        return cls(cfg, read_safetensors(model_dir / "model.safetensors"), bf16)

    def norm(self, x: np.ndarray, name: str) -> np.ndarray:
        return layer_norm(x, self.w[name], self.w[name + ".b"], self.eps)

    def lin(self, h: np.ndarray, name: str) -> np.ndarray:
        """h W^T, as an engine's activation type holds it."""
        return self.r(h @ self.w[name].T)

    # ----- mixers

    def mix_delta(self, h: np.ndarray, p: str, m: dict[str, Any]) -> np.ndarray:
        w = self.w
        heads, groups, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        n = h.shape[0]
        q = silu(short_conv(self.lin(h, p + "q"), w[p + "q.conv"])).reshape(n, groups, dim)
        k = silu(short_conv(self.lin(h, p + "k"), w[p + "k.conv"])).reshape(n, groups, dim)
        v = silu(short_conv(self.lin(h, p + "v"), w[p + "v.conv"])).reshape(n, heads, vdim)
        q = unit_length(q) * dim ** -0.5
        k = unit_length(k)
        strength = sigmoid(h @ w[p + "b"].T)                                                    # [n, heads]
        decay = np.exp(-np.exp(w[p + "A_log"])[None, :] * softplus(h @ w[p + "a"].T + w[p + "dt_bias"][None, :]))
        out = np.zeros((n, heads, vdim))
        for hd in range(heads):
            g = hd // (heads // groups)
            out[:, hd] = gated_delta(q[:, g], k[:, g], v[:, hd], strength[:, hd], decay[:, hd])
        out = unit_rms(out, self.eps) * w[p + "norm"][None, None, :]
        out = self.r(out.reshape(n, heads * vdim) * silu(self.lin(h, p + "g")))
        return self.lin(out, p + "o")

    def mix_general_delta(self, h: np.ndarray, p: str, m: dict[str, Any]) -> np.ndarray:
        w = self.w
        heads, dim = int(m["heads"]), int(m["dim"])
        n = h.shape[0]
        r = self.lin(h, p + "r").reshape(n, heads, dim)
        k = self.lin(h, p + "k").reshape(n, heads, dim)
        v = self.lin(h, p + "v").reshape(n, heads, dim)
        low = np.tanh(self.lin(h, p + "w1")) @ w[p + "w2"].T + w[p + "w0"][None, :]
        decay = np.exp(-DECAY_FLOOR * sigmoid(low)).reshape(n, heads, dim)
        rate = sigmoid(self.lin(h, p + "a") + w[p + "a.b"][None, :]).reshape(n, heads, dim)
        out = np.zeros((n, heads, dim))
        for hd in range(heads):
            out[:, hd] = generalized_delta(r[:, hd], k[:, hd], v[:, hd], decay[:, hd], rate[:, hd])
        out = unit_rms(out, self.eps).reshape(n, heads * dim) * w[p + "norm"][None, :]
        out = self.r(out * sigmoid(self.lin(h, p + "g")))
        return self.lin(out, p + "o")

    def keys_values(self, h: np.ndarray, p: str, m: dict[str, Any]) -> tuple[np.ndarray, np.ndarray]:
        w = self.w
        groups, dim, vdim = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        n = h.shape[0]
        k = unit_rms(self.lin(h, p + "k").reshape(n, groups, dim), self.eps) * w[p + "k.norm"][None, None, :]
        v = self.lin(h, p + "v").reshape(n, groups, vdim)
        return self.r(k), v

    def mix_attention(self, h: np.ndarray, p: str, m: dict[str, Any], kv: tuple[np.ndarray, np.ndarray]) -> np.ndarray:
        w = self.w
        heads, groups, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        n = h.shape[0]
        q = self.r(unit_rms(self.lin(h, p + "q").reshape(n, heads, dim), self.eps) * w[p + "q.norm"][None, None, :])
        k, v = kv
        out = np.zeros((n, heads, vdim))
        for hd in range(heads):
            g = hd // (heads // groups)
            out[:, hd], _ = causal_softmax_attention(q[:, hd], k[:, g], v[:, g], float(m["scale"]) * w[p + "temp"][hd])
        return self.lin(self.r(out.reshape(n, heads * vdim)), p + "o")

    # ----- feed-forwards

    def feed_forward(self, h: np.ndarray, p: str, f: dict[str, Any]) -> np.ndarray:
        w = self.w
        if f["kind"] == "dense":
            return self.r(gated_ff(h, w[p + "gate"], w[p + "up"], w[p + "down"], gelu_tanh, self.r))
        top = int(f["router"]["top"])
        chosen, weight = route(h @ w[p + "router"].T + w[p + "router.b"][None, :], top)
        out = np.zeros_like(h)
        for t in range(h.shape[0]):
            for e, wt in zip(chosen[t], weight[t]):
                q = f"{p}e{e}."
                out[t] += wt * gated_ff(h[t: t + 1], w[q + "gate"], w[q + "up"], w[q + "down"], silu, self.r)[0]
        if f.get("shared") is not None:
            q = p + "shared."
            out += gated_ff(h, w[q + "gate"], w[q + "up"], w[q + "down"], silu, self.r) * sigmoid(h @ w[q + "sg"].T)
        return out

    # ----- the model

    def forward(self, tokens, return_layers: bool = False):
        """Logits [n, vocab] (and the stream behind every layer, [layers, n, width])."""
        tokens = np.asarray(tokens, dtype=np.int64)
        n = len(tokens)
        x = self.w["embed"][tokens] + sinusoid(np.arange(n), self.width)
        kept: dict[int, tuple[np.ndarray, np.ndarray]] = {}
        streams = []
        for i, layer in enumerate(self.cfg["layers"]):
            p, m = f"l{i}.", layer["mixer"]
            h = self.r(self.norm(x, p + "norm1"))
            if layer["type"] == "delta":
                y = self.mix_delta(h, p + "mix.", m)
            elif layer["type"] == "general_delta":
                y = self.mix_general_delta(h, p + "mix.", m)
            elif layer["type"] == "attention":
                if m.get("kv_from") is None:
                    kept[i] = self.keys_values(h, p + "mix.", m)
                y = self.mix_attention(h, p + "mix.", m, kept[i if m.get("kv_from") is None else int(m["kv_from"])])
            else:
                raise ValueError(layer["type"])
            x = x + self.norm(y, p + "norm1b")
            if layer.get("mlp") is not None:
                x = x + self.norm(self.feed_forward(self.r(self.norm(x, p + "norm2")), p + "mlp.", layer["mlp"]), p + "norm2b")
            streams.append(x)
        logits = self.r(self.norm(x, "final.norm")) @ self.w["head"].T
        return (logits, np.stack(streams)) if return_layers else logits

    def logits(self, tokens) -> np.ndarray:
        return self.forward(tokens)

    def greedy(self, prompt, n: int) -> list[int]:
        """The n tokens greedy decoding makes behind ``prompt`` (the whole sequence is run again for each)."""
        seq = list(prompt)
        for _ in range(n):
            seq.append(int(np.argmax(self.forward(seq)[-1])))
        return seq[len(prompt):]
