"""The Fubelorn decoder as a ``ModelSpec``.

The token table's rows pass an RMS norm whose weight is one number and become ``streams`` copies of
the residual stream; every layer is a block over all copies (block "hyper"): a sub-layer reads a
weighted sum of them through a norm (one number again) and a causal convolution over a few tokens,
and writes every copy from a mix of the old ones plus ``residual_mult`` times its output. The
mixer is, layer by layer,
  * ``mamba2``: a selective state space layer (``selective_state_space``);
  * ``parallel``: attention without rotation whose queries and keys are divided by their root mean
    square per head, in a sliding window that keeps the sequence's first tokens, beside a gated
    delta rule, both weighted (``parallel_mixers`` of ``paged_attention`` and ``gated_delta_rule``);
  * ``parallel_2``: attention with a partly rotated head, scaled frequencies, a sliding window with
    means over blocks of tokens in front of it and a gate per head, beside a matrix memory with
    exponential gates (``parallel_mixers`` of ``paged_attention`` and ``matrix_memory``).
The feed-forward, where a layer has one, is down(gelu(up x)) with the exact GELU. The final norm
reads the sum of the copies. Weight names are the checkpoint's own (``l<i>.mix.left.q`` ...).
"""

from __future__ import annotations

from prefixserve_amd.config.fubelorn import MAX_POSITION, FubelornConfig, GatedDelta, WindowAttention
from prefixserve_amd.config.registry import register_architecture
from prefixserve_amd.parts.attention import slot_size
from prefixserve_amd.parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

STATE_SPACE_NAMES = {"in": "mix.in", "conv": "mix.conv", "conv_bias": "mix.conv.b", "dt_bias": "mix.dt_bias",
                     "decay_log": "mix.A_log", "skip": "mix.D", "norm": "mix.norm", "o": "mix.o"}
ATTENTION_NAMES = {"q": "mix.left.q", "k": "mix.left.k", "v": "mix.left.v", "o": "mix.left.o", "head_gate": "mix.left.g"}
GATED_DELTA_NAMES = {"q": "mix.right.q", "k": "mix.right.k", "v": "mix.right.v", "q_conv": "mix.right.q.conv",
                     "k_conv": "mix.right.k.conv", "v_conv": "mix.right.v.conv", "strength": "mix.right.b",
                     "decay": "mix.right.a", "decay_log": "mix.right.A_log", "decay_bias": "mix.right.dt_bias",
                     "gate": "mix.right.g", "norm": "mix.right.norm", "o": "mix.right.o"}
MEMORY_NAMES = {"q": "mix.right.q", "k": "mix.right.k", "v": "mix.right.v", "gate": "mix.right.g",
                "input_gate": "mix.right.i", "input_bias": "mix.right.i.b", "forget_gate": "mix.right.f",
                "forget_bias": "mix.right.f.b", "norm": "mix.right.norm", "o": "mix.right.o"}
FEED_FORWARD_NAMES = {"up": "mlp.up", "down": "mlp.down"}
BLOCK_NAMES = {"mixer_in": "hc1.in", "mixer_out": "hc1.out", "mixer_mix": "hc1.mix", "mixer_conv": "canon1",
               "feed_forward_in": "hc2.in", "feed_forward_out": "hc2.out", "feed_forward_mix": "hc2.mix",
               "feed_forward_conv": "canon2"}


def _norm(eps: float, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"eps": eps, "name": name, "scalar": True})


def _attention(i: int, a: WindowAttention, eps: float, kind: str, positions: dict[str, PartSpec]) -> PartSpec:
    params = {"num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim, "value_dim": a.vdim,
              "names": ATTENTION_NAMES, "scale": a.scale, "window": a.window, "exact_weights": True,
              "keep_first": a.keep_first, "pooled_block": a.pool}
    if kind == "parallel":
        params["qk_norm_eps"] = eps                  # the design's first kind divides q and k by their root mean square
    else:
        params["head_gate"] = True                   # its second kind gates every head's output
    if a.rot is not None and a.rot.dims:
        sc = a.rot.scaling
        scaling = None if sc is None else {"factor": sc.factor, "low_freq_factor": sc.low, "high_freq_factor": sc.high,
                                           "original_max_position_embeddings": sc.original}
        positions[f"rope{i}"] = PartSpec("rope", {"head_dim": slot_size(a.dim, a.vdim), "theta": a.rot.base,
                                                  "scaling": scaling, "rotary_dim": a.rot.dims})
        params["position"] = f"rope{i}"
    return PartSpec("paged_attention", params)


def build_fubelorn_spec(cfg: FubelornConfig) -> ModelSpec:
    layers, order = [], []
    positions: dict[str, PartSpec] = {}
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "mamba2":
            mixer = PartSpec("selective_state_space", {
                "num_heads": m.heads, "value_dim": m.vdim, "state_dim": m.state, "groups": m.groups, "taps": m.conv,
                "norm_groups": m.norm_groups, "names": STATE_SPACE_NAMES, "norm_eps": cfg.norm_eps})
        else:
            r = m.right
            if isinstance(r, GatedDelta):
                right = PartSpec("gated_delta_rule", {
                    "num_heads": r.heads, "num_kv_heads": r.kv_heads, "head_dim": r.dim, "value_dim": r.vdim, "taps": r.conv,
                    "names": GATED_DELTA_NAMES, "norm_eps": cfg.norm_eps})
            else:
                right = PartSpec("matrix_memory", {
                    "num_heads": r.heads, "head_dim": r.dim, "value_dim": r.vdim, "gate_cap": r.gate_cap,
                    "names": MEMORY_NAMES, "norm_eps": cfg.norm_eps})
            mixer = PartSpec("parallel_mixers", {
                "left": _attention(i, m.left, cfg.norm_eps, layer.type, positions), "right": right,
                "left_scale": m.left_scale, "right_scale": m.right_scale})
        ff = ff_norm = None
        if layer.mlp is not None:
            ff = PartSpec("dense_mlp", {"intermediate_size": layer.mlp.ff, "names": FEED_FORWARD_NAMES, "activation": "gelu"})
            ff_norm = _norm(cfg.norm_eps, "norm2")
        layers.append(LayerSpec(
            prefix=f"l{i}.", mixer=mixer, feed_forward=ff, mixer_norm=_norm(cfg.norm_eps, "norm1"), feed_forward_norm=ff_norm,
            block="hyper", block_params={"streams": cfg.streams, "names": BLOCK_NAMES, "mult": cfg.residual_mult,
                                         "taps": cfg.canon_taps}))
        order.append(LayerRun(i, i, True))
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embedding="embed", layers=tuple(layers),
        order=tuple(order), final_norm=_norm(cfg.norm_eps, "final.norm"), final_norm_prefix="", head="head",
        positions=positions, max_position=MAX_POSITION, stop_token_ids=cfg.stop_token_ids, streams=cfg.streams,
        embedding_transforms=(PartSpec("rms_norm", {"eps": cfg.norm_eps, "name": "embed.norm", "scalar": True}),),
        # A layer without a feed-forward still carries the tensors of its second sub-layer's place.
        ignored_weights=(".norm2", ".hc2.in", ".hc2.out", ".hc2.mix", ".canon2"),
    )


register_architecture("Fubelorn", FubelornConfig, build_fubelorn_spec)
