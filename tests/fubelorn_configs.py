"""Tiny Fubelorn configurations for the tests. They differ from each other in what the design lets
differ: width, vocabulary, eps, the factor on a sub-layer's output, the number of residual streams
(also one), the taps of the convolution in front of a sub-layer (none, 1, 3), the order and kinds of
layers, head counts and groups, key and value sizes (no multiples of 16), windows, kept first tokens
(none, fewer and more than a page), pooled blocks (none, smaller than a page, a page), the rotating part of a head
(none, a part, the whole head; with and without scaled frequencies), the state space layer's groups,
norm groups and taps, the gate cap, and layers without a feed-forward."""

from __future__ import annotations

import copy
import json
from pathlib import Path


def attention(heads, kv_heads, dim, vdim, scale, size, keep_first=None, pool=None, rot=None):
    mask = {"size": size}
    if keep_first is not None:
        mask["keep_first"] = keep_first
    if pool is not None:
        mask["pool"] = pool
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": mask}
    if rot is not None:
        m["rot"] = rot
    return m


def side_by_side(kind, left, right, left_scale, right_scale):
    return {"type": kind, "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def memory(heads, dim, vdim, cap):
    return {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def mamba2(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def layer(mixer, ff):
    return {**mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(vocab, width, eps, layers, streams=None, taps=None, mult=None):
    out = {"architecture": "Fubelorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams is not None:
        out["streams"] = streams
    if taps is not None:
        out["canon"] = {"taps": taps}
    if mult is not None:
        out["residual_mult"] = mult
    return out


_SCALED = {"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}}

FUBELORN = {
    # every mixer; three streams and three taps; grouped heads everywhere; a part of the head rotates with scaled frequencies
    "A": model(90, 48, 1e-5, [
        layer(side_by_side("parallel_2", attention(4, 2, 12, 20, 0.3, 9, pool=4, rot=_SCALED), memory(2, 12, 8, 10.0), 0.8, 0.6), 64),
        layer(mamba2(4, 8, 12, 2, 4, 2), None),
        layer(side_by_side("parallel", attention(3, 3, 8, 12, 0.35, 6, keep_first=3), delta(4, 2, 8, 6, 2), 1.1, 0.5), 40),
    ], streams=3, taps=3, mult=0.4),
    # one stream, no convolution in front of the sub-layers, no factor; nothing kept, nothing pooled, no rotation; one tap
    "B": model(70, 40, 1e-6, [
        layer(mamba2(2, 10, 5, 1, 1, 1), 24),
        layer(side_by_side("parallel", attention(2, 1, 24, 24, 0.2, 11), delta(3, 3, 12, 8, 1), 1.0, 1.0), None),
        layer(side_by_side("parallel_2", attention(2, 2, 8, 8, 0.4, 5), memory(3, 6, 10, 4.0), 0.7, 1.3), 32),
    ]),
    # windows longer than a round of keys in the kernels, more kept tokens than a page holds, a block of a page's size,
    # the whole head rotating without scaling, one tap in front of the sub-layers, two streams
    "C": model(64, 32, 1e-5, [
        layer(side_by_side("parallel", attention(2, 1, 16, 8, 0.3, 40, keep_first=20), delta(1, 1, 20, 20, 3), 0.9, 0.7), 48),
        layer(side_by_side("parallel_2", attention(2, 2, 12, 12, 0.3, 70, pool=16, rot={"dims": 12, "base": 500.0}),
                           memory(1, 20, 12, 15.0), 1.0, 0.5), None),
    ], streams=2, taps=1, mult=0.7),
}

STD = 0.15      # projections of unit-size rows come out near 1: the softmax and the gates bite


def write_fubelorn(folder, name_or_config, seed: int = 3, std: float = STD, edit=None) -> Path:
    """A model folder with random weights. The matrices that mix the residual streams are drawn near
    the identity, so that a few layers neither blow the streams up nor make them equal.
    ``edit(tensors)`` may change the tensors before they are written."""
    import torch
    from safetensors.torch import save_file

    import prefixserve_amd.models  # noqa: F401
    from prefixserve_amd.config.registry import architecture_of
    from prefixserve_amd.parts.model import DecoderModel
    from prefixserve_amd.weights import random_tensors

    config = copy.deepcopy(FUBELORN[name_or_config] if isinstance(name_or_config, str) else name_or_config)
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    arch = architecture_of(config)
    want = DecoderModel(arch.build_spec(arch.config_cls.from_dicts(config, {}))).weights()
    tensors = random_tensors(want, seed=seed, std=std)
    gen = torch.Generator().manual_seed(seed + 1000)
    for name, t in tensors.items():
        if name.endswith(".mix") and t.dim() == 2 and "hc" in name:
            tensors[name] = (torch.eye(t.shape[0]) + 0.3 * torch.randn(t.shape, generator=gen)).to(t.dtype)
    if edit is not None:
        edit(tensors)
    (folder / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
