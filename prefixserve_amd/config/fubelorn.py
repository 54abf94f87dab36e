"""The Fubelorn architecture's configuration, typed, from its own ``config.json`` keys.

A Fubelorn file gives the width (``width``), the vocabulary (``vocab``), the norms' epsilon
(``norm.eps``), the factor on every sub-layer's output (``residual_mult``), the number of copies of
the residual stream (``streams``), the taps of the convolution on what a sub-layer reads
(``canon.taps``) and its layers one by one (``layers``: each with ``type`` = which mixer, the
mixer's sizes and constants under ``mixer`` and its feed-forward under ``mlp`` or null). Every
size and constant is read from there; a key this parser does not know raises, because a rule
dropped without a word would load and then compute something else.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .llama import UnsupportedModelError
from .radivik import _only

ARCHITECTURE = "Fubelorn"
# No position limit is part of the design; the engine's own ``max_seq_len`` bounds the tables.
MAX_POSITION = 1 << 20


def _heads(m: Mapping[str, Any], where: str) -> tuple[int, int]:
    heads = int(m["heads"])
    kv_heads = int(m.get("kv_heads", heads))
    if heads < 1 or kv_heads < 1 or heads % kv_heads:
        raise UnsupportedModelError(f"{where}: {heads} heads cannot share {kv_heads} key heads")
    return heads, kv_heads


@dataclass(frozen=True)
class RotaryScaling:
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class Rotary:
    dims: int                # the first that many dimensions of a head rotate
    base: float
    scaling: RotaryScaling | None

    @classmethod
    def from_json(cls, r: Mapping[str, Any], where: str) -> "Rotary":
        _only(r, ("dims", "base", "scaling"), where)
        sc = r.get("scaling")
        if sc is not None:
            _only(sc, ("factor", "low", "high", "original"), where + ".scaling")
            sc = RotaryScaling(float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
        dims = int(r["dims"])
        if dims < 0 or dims % 2:
            raise UnsupportedModelError(f"{where}: {dims} rotating dimensions (an even number)")
        return cls(dims, float(r["base"]), sc)

    def to_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            s = self.scaling
            out["scaling"] = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
        return out


@dataclass(frozen=True)
class WindowAttention:
    """Grouped-query softmax attention in a sliding window that may keep the first tokens or see
    means over blocks of tokens in front of it; with or without a (partial) rotation."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int          # 0: none kept
    pool: int                # 0: no pooled blocks
    rot: Rotary | None

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "WindowAttention":
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"), where)
        heads, kv_heads = _heads(m, where)
        mask = m["mask"]
        _only(mask, ("size", "keep_first", "pool"), where + ".mask")
        size, keep, pool = int(mask["size"]), int(mask.get("keep_first", 0)), int(mask.get("pool", 0))
        if size < 1 or keep < 0 or pool < 0:
            raise UnsupportedModelError(f"{where}.mask: size {size}, keep_first {keep}, pool {pool}")
        dim = int(m["dim"])
        rot = None if m.get("rot") is None else Rotary.from_json(m["rot"], where + ".rot")
        if rot is not None and rot.dims > dim:
            raise UnsupportedModelError(f"{where}: {rot.dims} rotating dimensions in a head of {dim}")
        return cls(heads, kv_heads, dim, int(m.get("vdim", dim)), float(m["scale"]), size, keep, pool, rot)

    def to_json(self) -> dict[str, Any]:
        mask: dict[str, Any] = {"size": self.window}
        if self.keep_first:
            mask["keep_first"] = self.keep_first
        if self.pool:
            mask["pool"] = self.pool
        out: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                               "scale": self.scale, "mask": mask}
        if self.rot is not None:
            out["rot"] = self.rot.to_json()
        return out


@dataclass(frozen=True)
class GatedDelta:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

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
class MatrixMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "MatrixMemory":
        _only(m, ("heads", "dim", "vdim", "gate_cap"), where)
        heads, dim = int(m["heads"]), int(m["dim"])
        if heads < 1 or dim < 1 or not float(m["gate_cap"]) > 0:
            raise UnsupportedModelError(f"{where}: {heads} heads of {dim}, gate cap {m['gate_cap']}")
        return cls(heads, dim, int(m.get("vdim", dim)), float(m["gate_cap"]))

    def to_json(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class StateSpace:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_json(cls, m: Mapping[str, Any], where: str) -> "StateSpace":
        _only(m, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        heads, groups = int(m["heads"]), int(m.get("groups", 1))
        parts = int(m.get("norm_groups", 1))
        if heads < 1 or groups < 1 or heads % groups or parts < 1 or (heads * int(m["vdim"])) % parts or int(m["conv"]) < 1:
            raise UnsupportedModelError(f"{where}: {heads} heads in {groups} groups, {parts} norm groups, {m['conv']} taps")
        return cls(heads, int(m["vdim"]), int(m["state"]), groups, int(m["conv"]), parts)

    def to_json(self) -> dict[str, Any]:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class SideBySide:
    """Two mixers on the same input, their outputs weighted."""

    left: WindowAttention
    right: Any               # GatedDelta in a "parallel" layer, MatrixMemory in a "parallel_2" layer
    left_scale: float
    right_scale: float

    def to_json(self) -> dict[str, Any]:
        return {"left": self.left.to_json(), "right": self.right.to_json(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


RIGHT = {"parallel": GatedDelta, "parallel_2": MatrixMemory}
MIXER_TYPES = ("mamba2", "parallel", "parallel_2")


def _mixer(kind: str, m: Mapping[str, Any], where: str) -> Any:
    if kind == "mamba2":
        return StateSpace.from_json(m, where)
    _only(m, ("left", "right", "left_scale", "right_scale"), where)
    left = WindowAttention.from_json(m["left"], where + ".left")
    return SideBySide(left, RIGHT[kind].from_json(m["right"], where + ".right"), float(m.get("left_scale", 1.0)),
                      float(m.get("right_scale", 1.0)))


@dataclass(frozen=True)
class DenseFeedForward:
    ff: int

    def to_json(self) -> dict[str, Any]:
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class FubelornLayer:
    type: str
    mixer: Any
    mlp: DenseFeedForward | None


@dataclass(frozen=True)
class FubelornConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    streams: int
    canon_taps: int          # 0: what a sub-layer reads passes no convolution
    layers: tuple[FubelornLayer, ...]
    stop_token_ids: frozenset[int] = frozenset()

    @classmethod
    def from_dicts(cls, raw: Mapping[str, Any], gen: Mapping[str, Any] | None = None) -> "FubelornConfig":
        _only(raw, ("architecture", "architectures", "canon", "layers", "norm", "residual_mult", "streams", "vocab", "width"),
              "config.json")
        _only(raw["norm"], ("eps",), "norm")
        taps = 0
        if raw.get("canon") is not None:
            _only(raw["canon"], ("taps",), "canon")
            taps = int(raw["canon"]["taps"])
            if not 1 <= taps <= 16:
                raise UnsupportedModelError(f"canon.taps = {taps}: 1 to 16 are implemented")
        streams = int(raw.get("streams", 1))
        if streams < 1:
            raise UnsupportedModelError(f"streams = {streams}")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _only(entry, ("type", "mixer", "mlp"), where)
            kind = entry.get("type")
            if kind not in MIXER_TYPES:
                raise UnsupportedModelError(f"{where}: mixer type {kind!r}; implemented: {list(MIXER_TYPES)}")
            mlp = None
            if entry.get("mlp") is not None:
                f = entry["mlp"]
                if f.get("kind") != "dense":
                    raise UnsupportedModelError(f"{where}.mlp: feed-forward kind {f.get('kind')!r}; implemented: 'dense'")
                _only(f, ("kind", "ff"), where + ".mlp")
                mlp = DenseFeedForward(int(f["ff"]))
            layers.append(FubelornLayer(kind, _mixer(kind, entry["mixer"], where + ".mixer"), mlp))
        return cls(int(raw["vocab"]), int(raw["width"]), float(raw["norm"]["eps"]), float(raw.get("residual_mult", 1.0)),
                   streams, taps, tuple(layers))

    def to_config_json(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architecture": ARCHITECTURE,
            "layers": [{"type": l.type, "mixer": l.mixer.to_json(), "mlp": None if l.mlp is None else l.mlp.to_json()}
                       for l in self.layers],
            "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "streams": self.streams,
            "vocab": self.vocab_size, "width": self.hidden_size,
        }
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        return out
