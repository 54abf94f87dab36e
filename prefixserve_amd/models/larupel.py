"""The Larupel decoder as a ``ModelSpec``.

The token table's rows get a sinusoid of the position added. Every layer has a layer norm (weight
and bias) in front of and behind each sub-layer (block "sandwich"). The mixer is, layer by layer,
a gated delta rule behind short convolutions, a generalized delta rule with a decay and a removal
rate per key channel, or paged grouped-query attention without rotation whose queries and keys get
a weighted norm per head and whose scores are multiplied by a learned number per head; an
attention layer that names another under ``kv_from`` has no key and value projections and reads
the cache entry that layer's run writes. The feed-forward, where a layer has one, is a dense gated
one (GELU on the gate) or a mixture of SiLU-gated experts chosen by the router's largest logits,
weighted by the softmax over the chosen logits, beside a shared expert with a gate per token.
Layers may differ in all of this; weight names are the checkpoint's own (``l<i>.mix.q`` ...).
"""

from __future__ import annotations

import math

from prefixserve_amd.config.larupel import MAX_POSITION, DenseFeedForward, LarupelConfig
from prefixserve_amd.config.llama import UnsupportedModelError
from prefixserve_amd.config.registry import register_architecture
from prefixserve_amd.parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec

ATTENTION_NAMES = {"q": "mix.q", "k": "mix.k", "v": "mix.v", "o": "mix.o", "q_norm": "mix.q.norm", "k_norm": "mix.k.norm",
                   "head_scale": "mix.temp"}
GATED_DELTA_NAMES = {"q": "mix.q", "k": "mix.k", "v": "mix.v", "q_conv": "mix.q.conv", "k_conv": "mix.k.conv",
                     "v_conv": "mix.v.conv", "strength": "mix.b", "decay": "mix.a", "decay_log": "mix.A_log",
                     "decay_bias": "mix.dt_bias", "gate": "mix.g", "norm": "mix.norm", "o": "mix.o"}
GENERAL_DELTA_NAMES = {"r": "mix.r", "k": "mix.k", "v": "mix.v", "gate": "mix.g", "rate": "mix.a", "rate_bias": "mix.a.b",
                       "decay_in": "mix.w1", "decay_out": "mix.w2", "decay_bias": "mix.w0", "norm": "mix.norm", "o": "mix.o"}
DENSE_NAMES = {"gate": "mlp.gate", "up": "mlp.up", "down": "mlp.down"}
EXPERT_NAMES = {"router": "mlp.router", "router_bias": "mlp.router.b", "gate": "mlp.e{e}.gate", "up": "mlp.e{e}.up",
                "down": "mlp.e{e}.down", "shared_gate": "mlp.shared.gate", "shared_up": "mlp.shared.up",
                "shared_down": "mlp.shared.down", "shared_scale": "mlp.shared.sg"}
# Fixed by the design, not by a file.
SINUSOID_BASE = 10000.0
DECAY_FLOOR = math.exp(-0.5)         # the generalized rule's decay is exp(-DECAY_FLOOR sigmoid(.))


def _norm(eps: float, name: str) -> PartSpec:
    return PartSpec("layernorm", {"eps": eps, "name": name, "bias_name": name + ".b"})


def build_larupel_spec(cfg: LarupelConfig) -> ModelSpec:
    layers, order = [], []
    for i, layer in enumerate(cfg.layers):
        m = layer.mixer
        run = LayerRun(i, i, True)
        if layer.type == "delta":
            mixer = PartSpec("gated_delta_rule", {
                "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim, "taps": m.conv,
                "names": GATED_DELTA_NAMES, "norm_eps": cfg.norm_eps,
            })
        elif layer.type == "general_delta":
            if m.decay_rank is None:
                raise UnsupportedModelError(f"layers[{i}]: the inner size of the decay's low-rank map is not known "
                                            "(neither a checkpoint's l<i>.mix.w1 nor a 'decay_rank' key says)")
            mixer = PartSpec("generalized_delta_rule", {
                "num_heads": m.heads, "head_dim": m.dim, "decay_rank": m.decay_rank, "names": GENERAL_DELTA_NAMES,
                "norm_eps": cfg.norm_eps, "decay_floor": DECAY_FLOOR,
            })
        else:
            mixer = PartSpec("paged_attention", {
                "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
                "names": ATTENTION_NAMES, "scale": m.scale, "qk_norm_eps": cfg.norm_eps, "qk_norm_weights": True,
                "head_scale": True, "own_kv": m.kv_from is None, "exact_weights": True,
            })
            if m.kv_from is not None:
                run = LayerRun(i, m.kv_from, False)
        ff = ff_norm = None
        extra = {"mixer_post_norm": _norm(cfg.norm_eps, "norm1b")}
        if layer.mlp is not None:
            f = layer.mlp
            if isinstance(f, DenseFeedForward):
                ff = PartSpec("swiglu", {"intermediate_size": f.ff, "names": DENSE_NAMES, "activation": "gelu_tanh"})
            else:
                ff = PartSpec("routed_experts", {
                    "num_experts": f.experts, "top_k": f.top, "intermediate_size": f.ff, "names": EXPERT_NAMES,
                    "limit": None, "gate_alpha": 1.0, "up_shift": 0.0, "score": "softmax_of_chosen", "weight_on": "output",
                    "router_bias": True,
                    "shared": None if f.shared_ff is None else {"intermediate_size": f.shared_ff, "gated": True},
                })
            ff_norm = _norm(cfg.norm_eps, "norm2")
            extra["feed_forward_post_norm"] = _norm(cfg.norm_eps, "norm2b")
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=mixer, feed_forward=ff, mixer_norm=_norm(cfg.norm_eps, "norm1"),
                                feed_forward_norm=ff_norm, block="sandwich", extra_norms=extra))
        order.append(run)
    return ModelSpec(
        vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, embedding="embed", layers=tuple(layers),
        order=tuple(order), final_norm=_norm(cfg.norm_eps, "final.norm"), final_norm_prefix="", head="head",
        positions={}, max_position=MAX_POSITION, stop_token_ids=cfg.stop_token_ids,
        embedding_transforms=(PartSpec("sinusoidal_positions", {"base": SINUSOID_BASE}),),
    )


register_architecture("Larupel", LarupelConfig, build_larupel_spec)
