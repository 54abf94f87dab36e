"""The Larupel architecture's configuration, typed, from its own ``config.json`` keys.

A Larupel file gives the width (``width``), the vocabulary (``vocab``), the norms' epsilon
(``norm.eps``) and its layers one by one (``layers``: each with ``type`` = which mixer, the
mixer's sizes and constants under ``mixer`` and its feed-forward under ``mlp`` or null). Every
size and constant is read from there; a key this parser does not know raises, because a rule
dropped without a word would load and then compute something else.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .llama import UnsupportedModelError
from .radivik import _only

ARCHITECTURE = "Larupel"
# No position limit is part of the design; the engine's own ``max_seq_len`` bounds the tables.
MAX_POSITION = 1 << 20


def _heads(m: Mapping[str, Any], where: str) -> tuple[int, int]:
    heads = int(m["heads"])
    kv_heads = int(m.get("kv_heads", heads))
    if heads < 1 or kv_heads < 1 or heads % kv_heads:
        raise UnsupportedModelError(f"{where}: {heads} heads cannot share {kv_heads} key heads")
    return heads, kv_heads


@dataclass(frozen=True)
class GatedDelta:
    """A delta rule with one decay and one write strength per head, behind short convolutions."""

    heads: int
    kv_heads: int            # heads of queries and keys; a group of value heads shares one
    dim: int                 # per-head size of queries and keys
    vdim: int                # per-head size of values
    conv: int                # taps of the short convolutions

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "GatedDelta":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        heads, kv_heads = _heads(m, where)
        dim, conv = int(m["dim"]), int(m["conv"])
        if dim < 1 or conv < 1:
            raise UnsupportedModelError(f"{where}: dim {dim}, {conv} taps")
        return cls(heads, kv_heads, dim, int(m.get("vdim", dim)), conv)

    def to_json(self) -> dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class GeneralDelta:
    """A delta rule with a decay and a removal rate per key channel; values have the keys' size."""

    heads: int
    dim: int
    # Inner size of the decay's low-rank map. config.json does not say: the checkpoint's l<i>.mix.w1 does
    # (``LarupelConfig.fitted_to_checkpoint``); a file written without a checkpoint to look at names it.
    decay_rank: int | None = None

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "GeneralDelta":
        _only(m, ("heads", "dim", "decay_rank"), where)
        heads, dim = int(m["heads"]), int(m["dim"])
        if heads < 1 or dim < 1:
            raise UnsupportedModelError(f"{where}: {heads} heads of {dim}")
        rank = m.get("decay_rank")
        return cls(heads, dim, None if rank is None else int(rank))

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "dim": self.dim}
        if self.decay_rank is not None:
            out["decay_rank"] = self.decay_rank
        return out


@dataclass(frozen=True)
class NormedAttention:
    """Grouped-query softmax attention without rotation, a weighted norm on q and k, a number per head on the score."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    kv_from: int | None      # the layer whose keys and values this layer reads; None: its own

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "NormedAttention":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "kv_from"), where)
        heads, kv_heads = _heads(m, where)
        dim = int(m["dim"])
        kv_from = m.get("kv_from")
        return cls(heads, kv_heads, dim, int(m.get("vdim", dim)), float(m["scale"]), None if kv_from is None else int(kv_from))

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


MIXERS = {"delta": GatedDelta, "general_delta": GeneralDelta, "attention": NormedAttention}


@dataclass(frozen=True)
class DenseFeedForward:
    ff: int

    def to_json(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertFeedForward:
    experts: int
    top: int
    ff: int                  # inner size of one expert
    shared_ff: int | None    # inner size of the expert every token uses; None: there is none

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {"kind": "moe", "router": {"experts": self.experts, "top": self.top}, "expert": {"ff": self.ff}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _feed_forward(f: Mapping[str, Any], where: str) -> "DenseFeedForward | ExpertFeedForward":
    kind = f.get("kind")
    if kind == "dense":
        _only(f, ("kind", "ff"), where)
        return DenseFeedForward(int(f["ff"]))
    if kind == "moe":
        _only(f, ("kind", "router", "expert", "shared"), where)
        _only(f["router"], ("experts", "top"), where + ".router")
        _only(f["expert"], ("ff",), where + ".expert")
        experts, top = int(f["router"]["experts"]), int(f["router"]["top"])
        if not 1 <= top <= experts:
            raise UnsupportedModelError(f"{where}: top {top} of {experts} experts")
        shared = f.get("shared")
        if shared is not None:
            _only(shared, ("ff",), where + ".shared")
        return ExpertFeedForward(experts, top, int(f["expert"]["ff"]), None if shared is None else int(shared["ff"]))
    raise UnsupportedModelError(f"{where}: feed-forward kind {kind!r}; implemented: 'dense', 'moe'")


@dataclass(frozen=True)
class LarupelLayer:
    type: str
    mixer: Any
    mlp: "DenseFeedForward | ExpertFeedForward | None"


@dataclass(frozen=True)
class LarupelConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple[LarupelLayer, ...]
    stop_token_ids: frozenset[int] = frozenset()

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "LarupelConfig":
        _only(raw, ("architecture", "architectures", "layers", "norm", "vocab", "width"), "config.json")
        _only(raw["norm"], ("eps",), "norm")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = entry.get("type")
            if kind not in MIXERS:
                raise UnsupportedModelError(f"{where}: mixer type {kind!r}; implemented: {sorted(MIXERS)}")
            m = entry["mixer"]
            j = m.get("kv_from") if kind == "attention" else None
            if isinstance(j, int) and 0 <= j < i and raw["layers"][j].get("type") == "attention":
                # A reader's key and value sizes are its source's; a file may leave them out.
                m = {**{k: v for k, v in raw["layers"][j]["mixer"].items() if k in ("kv_heads", "dim", "vdim")}, **m}
            mixer = MIXERS[kind].from_json(m, where + ".mixer")
            mlp = None if entry.get("mlp") is None else _feed_forward(entry["mlp"], where + ".mlp")
            layers.append(LarupelLayer(kind, mixer, mlp))
        for i, layer in enumerate(layers):
            j = layer.mixer.kv_from if layer.type == "attention" else None
            if j is None:
                continue
            if not 0 <= j < i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                raise UnsupportedModelError(f"layers[{i}].mixer.kv_from = {j}: must name an earlier attention layer with keys of its own")
            a, b = layer.mixer, layers[j].mixer
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise UnsupportedModelError(f"layers[{i}] reads layer {j}'s keys and values but has other sizes")
        return cls(int(raw["vocab"]), int(raw["width"]), float(raw["norm"]["eps"]), tuple(layers))

    def fitted_to_checkpoint(self, shapes: Mapping[str, tuple[int, ...]]) -> "LarupelConfig":
        """The configuration with what the checkpoint's tensor shapes decide: the inner size of
        every generalized delta layer's low-rank decay map."""
        from dataclasses import replace

        layers = []
        for i, layer in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.w1") if layer.type == "general_delta" else None
            if shape is not None:
                layer = replace(layer, mixer=replace(layer.mixer, decay_rank=int(shape[0])))
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    def to_config_json(self) -> dict[str, Any]:
        return {
            "architecture": ARCHITECTURE,
            "layers": [{"type": l.type, "mixer": l.mixer.to_json(), "mlp": None if l.mlp is None else l.mlp.to_json()}
                       for l in self.layers],
            "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.hidden_size,
        }
