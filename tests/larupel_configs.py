"""Tiny Larupel configurations for the tests. They differ from each other in what the design lets
differ: width, vocabulary, the norms' eps, the order and kinds of layers, head counts and groups
(also one head, and as many key heads as heads), key and value sizes (larger, smaller, equal; no
multiples of 16), the taps of the short convolutions (1 to 5), the inner size of the decay's
low-rank map, the score scale, which attention layers read another layer's keys (and how many read
the same one), dense and expert feed-forwards (1 to all experts per token, with and without the
shared expert) and layers without one."""

from __future__ import annotations

import copy
import json
from pathlib import Path


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def general_delta(heads, dim, rank):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim, "decay_rank": rank}}


def attention(heads, kv_heads, dim, vdim, scale, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    out = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared is not None:
        out["shared"] = {"ff": shared}
    return out


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


def model(vocab, width, eps, layers):
    return {"architecture": "Larupel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


_A1 = dict(heads=6, kv_heads=2, dim=8, vdim=12, scale=0.5)
_C1 = dict(heads=1, kv_heads=1, dim=40, vdim=16, scale=0.2)
_C2 = dict(heads=4, kv_heads=4, dim=16, vdim=8, scale=0.4)

LARUPEL = {
    # every mixer, a reader without a feed-forward, all experts used by every token in one layer
    "A": model(96, 64, 1e-5, [
        layer(general_delta(2, 16, 5), moe(5, 2, 24, shared=40)),
        layer(attention(**_A1), dense(80)),
        layer(delta(4, 2, 8, 12, 3), moe(4, 4, 16)),
        layer(attention(**_A1, kv_from=1), None),
    ]),
    # as many key heads as heads and one tap, one head, one kv head for three, one expert per token
    "B": model(130, 72, 1e-6, [
        layer(delta(3, 3, 24, 8, 1), None),
        layer(general_delta(1, 40, 12), dense(48)),
        layer(attention(3, 1, 24, 24, 0.25), moe(3, 1, 32, shared=16)),
    ]),
    # attention first, two layer groups, two readers of the same layer, five taps, a value head larger than the key
    "C": model(70, 48, 1e-5, [
        layer(attention(**_C1), dense(24)),
        layer(attention(**_C1, kv_from=0), moe(7, 3, 8, shared=8)),
        layer(delta(2, 1, 12, 20, 5), moe(7, 3, 8, shared=8)),
        layer(general_delta(3, 8, 3), None),
        layer(attention(**_C2), dense(40)),
        layer(attention(**_C2, kv_from=4), None),
        layer(attention(**_C1, kv_from=0), dense(24)),
    ]),
}

STD = 0.15      # projections of unit-size rows come out near 1: the softmax, the gates and the router all bite


def write_larupel(folder, name_or_config, seed: int = 3, std: float = STD, keep_rank: bool = False, edit=None) -> Path:
    """A model folder with random weights. config.json does not say how large the decay's low-rank
    map is inside (unless ``keep_rank``): the loader takes that from the checkpoint, as for a file
    that never had the key. ``edit(tensors)`` may change the tensors before they are written."""
    from safetensors.torch import save_file

    import prefixserve_amd.models  # noqa: F401
    from prefixserve_amd.config.registry import architecture_of
    from prefixserve_amd.parts.model import DecoderModel
    from prefixserve_amd.weights import random_tensors

    config = copy.deepcopy(LARUPEL[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    arch = architecture_of(config)
    want = DecoderModel(arch.build_spec(arch.config_cls.from_dicts(config, {}))).weights()
    tensors = random_tensors(want, seed=seed, std=std)
    if edit is not None:
        edit(tensors)
    if not keep_rank:
        for entry in config["layers"]:
            entry["mixer"].pop("decay_rank", None)
    (folder / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
