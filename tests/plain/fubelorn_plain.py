"""Plain, slow Fubelorn: the oracle the engine's Fubelorn tests are compared with.

Whole sequences, no cache, no paging, no batching, no state handed on; numpy float64 only; one
function per mechanism. It shares no code with the product package (its file reader is the plain
Llama oracle's, which is test code too).

The design, in this file's notation. The token table's row is normalized (``scalar_rms_norm``: an
RMS norm whose weight is one number) and copied into ``streams`` residual streams X_1 .. X_s.
A sub-layer (``hyper_sublayer``) reads u = sum_s a_s X_s, normalizes it, replaces it by
u + conv(u) (``causal_conv``: a convolution over the last ``taps`` tokens per channel, no bias), runs
the mixer or the feed-forward on that and writes every stream anew from the old ones:
X_t <- sum_s M[s, t] X_s + m c_t y, with m the model's ``residual_mult``. The mixer is one of
  * ``parallel``: left_scale * (attention without rotation, q and k divided by their root mean square
    per head, a sliding window that also keeps the first tokens: ``window_attention``) +
    right_scale * (gated delta rule: ``gated_delta``);
  * ``mamba2``: a selective state space layer with a scalar decay per head (``ssd``), the gate in
    front of a norm in groups;
  * ``parallel_2``: left_scale * (attention with a partly rotated head and scaled frequencies, a
    sliding window plus one mean key and value per block of tokens wholly in front of the window, and a
    gate per head on the output) + right_scale * (matrix memory with exponential gates and a running
    maximum: ``matrix_memory``).
The feed-forward is down(gelu(up x)) with the exact gelu; a layer may have none. The logits are the
output matrix on the normalized sum of the streams.
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from typing import Any

import numpy as np

from .llama_plain import read_safetensors, round_bf16  # noqa: F401  (test-side helpers)

UNIT_EPS = 1e-6        # inside the root when the delta rule's keys and queries are made unit vectors
READ_EPS = 1e-6        # added to the matrix memory's denominator

# ------------------------------------------------------------------- formulas


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def logsigmoid(z):
    return -np.logaddexp(0.0, -z)


def gelu_erf(z):
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return 0.5 * z * (1.0 + erf(z / math.sqrt(2.0)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)


def scalar_rms_norm(x, g, eps):
    return unit_rms(x, eps) * float(g)


def causal_conv(h, w, bias=None):
    """h [T, C], w [C, taps] whose last column meets the token itself; zeros in front of the sequence."""
    t_n, taps = h.shape[0], w.shape[1]
    out = np.zeros_like(h)
    for t in range(t_n):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    if bias is not None:
        out = out + bias
    return out


def rotary_frequencies(dims, base, scaling=None):
    f = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=np.float64)
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for i, fi in enumerate(f):
        wave = 2.0 * math.pi / fi
        if wave < original / high:
            continue
        if wave > original / low:
            out[i] = fi / factor
        else:
            s = (original / wave - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x, positions, dims, freqs):
    """x [T, heads, dim]: the first ``dims`` entries of a head rotate, entry i with entry i + dims/2."""
    half = dims // 2
    ang = positions[:, None].astype(np.float64) * freqs[None, :]            # [T, half]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.copy()
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def softmax_rows(scores, values):
    """One query: scores [n], values [n, v]."""
    w = np.exp(scores - scores.max())
    return (w / w.sum()) @ values


def window_attention(q, k, v, scale, size, keep_first=0, pool=0):
    """q [T, H, d], k [T, G, d], v [T, G, dv]. Query i sees key j when j <= i and (i - j < size or
    j < keep_first). With ``pool`` = P it also sees, for every block b of P tokens with
    bP + P - 1 <= i - size, the mean key and mean value of the block, in the same softmax."""
    t_n, heads, _ = q.shape
    per = heads // k.shape[1]
    out = np.zeros((t_n, heads, v.shape[2]))
    for h in range(heads):
        g = h // per
        for i in range(t_n):
            js = [j for j in range(i + 1) if i - j < size or j < keep_first]
            keys, vals = [k[j, g] for j in js], [v[j, g] for j in js]
            if pool:
                b = 0
                while b * pool + pool - 1 <= i - size:
                    keys.append(k[b * pool: (b + 1) * pool, g].mean(0))
                    vals.append(v[b * pool: (b + 1) * pool, g].mean(0))
                    b += 1
            keys, vals = np.stack(keys), np.stack(vals)
            out[i, h] = softmax_rows((keys @ q[i, h]) * scale, vals)
    return out


def gated_delta(q, k, v, beta, g):
    """q, k [T, H, d] (unit vectors, q scaled), v [T, H, dv], beta and g [T, H]. Per head
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    t_n, heads, d = q.shape
    out = np.zeros((t_n, heads, v.shape[2]))
    for h in range(heads):
        s = np.zeros((d, v.shape[2]))
        for t in range(t_n):
            s = g[t, h] * s
            u = beta[t, h] * (v[t, h] - s.T @ k[t, h])
            s = s + np.outer(k[t, h], u)
            out[t, h] = s.T @ q[t, h]
    return out


def ssd(x, b, c, dt, a_log, d_skip):
    """x [T, H, p], b and c [T, G, N], dt [T, H] (after softplus). Per head
    S <- exp(-exp(a_log) dt) S + dt b x^T;  y = S^T c + D x."""
    t_n, heads, p = x.shape
    per = heads // b.shape[1]
    out = np.zeros((t_n, heads, p))
    for h in range(heads):
        g = h // per
        s = np.zeros((b.shape[2], p))
        for t in range(t_n):
            s = math.exp(-math.exp(a_log[h]) * dt[t, h]) * s + dt[t, h] * np.outer(b[t, g], x[t, h])
            out[t, h] = s.T @ c[t, g] + d_skip[h] * x[t, h]
    return out


def matrix_memory(q, k, v, i_log, f_log):
    """q (scaled), k [T, H, d], v [T, H, dv], log gates [T, H]. With a running maximum m that starts
    at 0: m' = max(f + m, i); S <- exp(f + m - m') S + exp(i - m') k v^T; n likewise with k;
    o = S^T q / (max(|n . q|, exp(-m')) + READ_EPS)."""
    t_n, heads, d = q.shape
    out = np.zeros((t_n, heads, v.shape[2]))
    for h in range(heads):
        s, n, m = np.zeros((d, v.shape[2])), np.zeros(d), 0.0
        for t in range(t_n):
            m_new = max(f_log[t, h] + m, i_log[t, h])
            keep, write = math.exp(f_log[t, h] + m - m_new), math.exp(i_log[t, h] - m_new)
            s = keep * s + write * np.outer(k[t, h], v[t, h])
            n = keep * n + write * k[t, h]
            m = m_new
            out[t, h] = (s.T @ q[t, h]) / (max(abs(n @ q[t, h]), math.exp(-m)) + READ_EPS)
    return out


# --------------------------------------------------------------------- mixers


class _Weights:
    def __init__(self, tensors, prefix, bf16):
        self.t, self.p, self.bf16 = tensors, prefix, bf16

    def __call__(self, name):
        return np.asarray(self.t[self.p + name], dtype=np.float64)

    def sub(self, more):
        return _Weights(self.t, self.p + more, self.bf16)

    def r(self, x):
        """What an engine holds in bfloat16 is rounded here when the yardstick for that mode is asked for."""
        return round_bf16(x) if self.bf16 else x


def left_attention(h, w, m, eps, rotating, unit_qk, gated):
    t_n = h.shape[0]
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = w.r(h @ w("q").T).reshape(t_n, heads, d)
    k = w.r(h @ w("k").T).reshape(t_n, groups, d)
    v = w.r(h @ w("v").T).reshape(t_n, groups, dv)
    pos = np.arange(t_n)
    if rotating and m.get("rot"):
        rot = m["rot"]
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, pos, rot["dims"], f), rotate(k, pos, rot["dims"], f)
    if unit_qk:
        q, k = unit_rms(q, eps), unit_rms(k, eps)
    q, k = w.r(q), w.r(k)
    mask = m["mask"]
    o = window_attention(q, k, v, m["scale"], mask["size"], mask.get("keep_first", 0), mask.get("pool", 0))
    if gated:
        o = o * sigmoid(h @ w("g").T)[:, :, None]
    return w.r(w.r(o).reshape(t_n, heads * dv) @ w("o").T)


def right_gated_delta(h, w, m, eps):
    t_n = h.shape[0]
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(w.r(causal_conv(w.r(h @ w("q").T), w("q.conv")))).reshape(t_n, groups, d)
    k = silu(w.r(causal_conv(w.r(h @ w("k").T), w("k.conv")))).reshape(t_n, groups, d)
    v = silu(w.r(causal_conv(w.r(h @ w("v").T), w("v.conv")))).reshape(t_n, heads, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + UNIT_EPS) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + UNIT_EPS)
    per = heads // groups
    q, k = np.repeat(q, per, axis=1), np.repeat(k, per, axis=1)
    beta = sigmoid(h @ w("b").T)
    g = np.exp(-np.exp(w("A_log")) * softplus(h @ w("a").T + w("dt_bias")))
    o = gated_delta(q, k, v, beta, g)
    o = unit_rms(o, eps) * w("norm") * silu(w.r(h @ w("g").T)).reshape(t_n, heads, dv)
    return w.r(w.r(o).reshape(t_n, heads * dv) @ w("o").T)


def right_matrix_memory(h, w, m, eps):
    t_n = h.shape[0]
    heads, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = w.r(h @ w("q").T).reshape(t_n, heads, d) * d ** -0.5
    k = w.r(h @ w("k").T).reshape(t_n, heads, d)
    v = w.r(h @ w("v").T).reshape(t_n, heads, dv)
    i_log = cap * np.tanh((h @ w("i").T + w("i.b")) / cap)
    f_log = logsigmoid(cap * np.tanh((h @ w("f").T + w("f.b")) / cap))
    o = unit_rms(matrix_memory(q, k, v, i_log, f_log), eps).reshape(t_n, heads * dv)
    o = o * w("norm") * sigmoid(w.r(h @ w("g").T))
    return w.r(w.r(o) @ w("o").T)


def mamba2(h, w, m, eps):
    t_n = h.shape[0]
    heads, p, n, groups = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * p
    rows = h @ w("in").T
    z = w.r(rows[:, :inner])
    xbc = w.r(rows[:, inner: 2 * inner + 2 * groups * n])
    dt = softplus(rows[:, 2 * inner + 2 * groups * n:] + w("dt_bias"))
    xbc = silu(w.r(causal_conv(xbc, w("conv"), w("conv.b"))))
    x = xbc[:, :inner].reshape(t_n, heads, p)
    b = xbc[:, inner: inner + groups * n].reshape(t_n, groups, n)
    c = xbc[:, inner + groups * n:].reshape(t_n, groups, n)
    y = ssd(x, b, c, dt, w("A_log"), w("D")).reshape(t_n, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.reshape(t_n, parts, inner // parts), eps).reshape(t_n, inner) * w("norm")
    return w.r(w.r(y) @ w("o").T)


def mixer(kind, h, w, m, eps):
    if kind == "mamba2":
        return mamba2(h, w, m, eps)
    if kind == "parallel":
        left = left_attention(h, w.sub("left."), m["left"], eps, rotating=False, unit_qk=True, gated=False)
        right = right_gated_delta(h, w.sub("right."), m["right"], eps)
    elif kind == "parallel_2":
        left = left_attention(h, w.sub("left."), m["left"], eps, rotating=True, unit_qk=False, gated=True)
        right = right_matrix_memory(h, w.sub("right."), m["right"], eps)
    else:
        raise ValueError(f"unknown mixer {kind!r}")
    return m["left_scale"] * left + m["right_scale"] * right


def feed_forward(h, w, bf16=False):
    return w.r(w.r(gelu_erf(w.r(h @ w("up").T))) @ w("down").T)


def hyper_sublayer(streams, w_hc, norm_g, canon_w, eps, mult, fn, r):
    """streams [s, T, width] -> new streams. ``w_hc`` names the sub-layer's three hyper-connection
    tensors; ``fn`` is the mixer or the feed-forward."""
    u = np.tensordot(w_hc("in"), streams, axes=(0, 0))
    h = scalar_rms_norm(u, norm_g, eps)
    if canon_w is not None:
        h = h + causal_conv(h, canon_w)
    y = fn(r(h))
    mix, out = w_hc("mix"), w_hc("out")
    return np.einsum("st,sxw->txw", mix, streams) + mult * out[:, None, None] * y[None]


# ---------------------------------------------------------------------- model


def forward(cfg: dict, tensors: dict, tokens, bf16: bool = False, layers_out: list | None = None) -> np.ndarray:
    """Logits [T, vocab] of one whole sequence. ``layers_out``: a list that receives the sum of the
    streams after every layer."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg.get("residual_mult", 1.0))
    n_streams = int(cfg.get("streams", 1))
    top = _Weights(tensors, "", bf16)
    x = scalar_rms_norm(top("embed")[np.asarray(tokens)], top("embed.norm"), eps)
    streams = np.repeat(x[None], n_streams, axis=0)
    for i, layer in enumerate(cfg["layers"]):
        w = _Weights(tensors, f"l{i}.", bf16)
        canon = "canon" in cfg
        streams = hyper_sublayer(streams, w.sub("hc1."), w("norm1"), w("canon1") if canon else None, eps, mult,
                                 lambda h: mixer(layer["type"], h, w.sub("mix."), layer["mixer"], eps), w.r)
        if layer.get("mlp") is not None:
            streams = hyper_sublayer(streams, w.sub("hc2."), w("norm2"), w("canon2") if canon else None, eps, mult,
                                     lambda h: feed_forward(h, w.sub("mlp."), bf16), w.r)
        if layers_out is not None:
            layers_out.append(streams.sum(0))
    x = scalar_rms_norm(streams.sum(0), top("final.norm"), eps)
    return top.r(x) @ top("head").T


def load(model_dir: str | Path) -> tuple[dict, dict[str, Any]]:
    model_dir = Path(model_dir)
    cfg = json.loads((model_dir / "config.json").read_text())
    return cfg, read_safetensors(model_dir / "model.safetensors")
