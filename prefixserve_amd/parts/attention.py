"""Grouped-query causal attention over the paged cache."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import CacheNeed, Mixer, PositionEncoding, RotaryTable, Runtime, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


@dataclass
class LayerCache:
    """One cache entry as a run sees it: the pages of its layer group.

    ``kv`` is ``[num_blocks, 2, kv_heads, 16 * head_dim]``. Half 0 of a page holds the keys
    of its 16 positions as ``[16, head_dim]`` (after rotation); half 1 holds the values
    transposed, ``[head_dim, 16]``, which is the operand order the matrix cores want for
    probabilities x values. ``group`` selects the block tables of the step batch."""

    kv: torch.Tensor
    group: int
    window: int | None
    # Further entries of the same run by the mixer's own names (``Mixer.aux_cache_needs``).
    aux: "dict[str, LayerCache] | None" = None


def slot_size(head_dim: int, value_dim: int, largest: int = 256) -> int:
    """The head size the pages and kernels run with: the larger of the two sizes, rounded up to
    one the matrix-core attention takes (multiples of 16 up to 128, then 160, 192, 256). A mixer
    whose other kernels take more may allow up to 512 (``largest``): sizes above 256 are multiples
    of 64 and run the attention kernel of the 32-bit path in either dtype."""
    need = max(int(head_dim), int(value_dim))
    for size in (*range(16, 129, 16), 160, 192, 256, 320, 384, 448, 512):
        if need <= size <= largest:
            return size
    raise ValueError(f"head sizes up to {largest} are implemented, got {need}")


def head_slots(head_dim: int, rotary_dim: int, slots: int) -> list[int]:
    """Slot of each of a head's ``head_dim`` dimensions in a head of ``slots`` slots whose pair
    (i, i + slots/2) rotates together. The model's partners (i, i + rotary_dim/2), i < rotary_dim/2,
    go to (i, i + slots/2); the dimensions that do not rotate fill the first half's remaining
    slots and then the second half's (their table entries are the identity)."""
    half, r2 = slots // 2, rotary_dim // 2
    out = [i if i < r2 else half + (i - r2) for i in range(rotary_dim)]
    free = list(range(r2, half)) + list(range(half + r2, slots))
    out += free[: head_dim - rotary_dim]
    assert len(out) == head_dim and len(set(out)) == head_dim
    return out


def distance_bucket(n: int, buckets: int, far: float) -> int:
    """The row of a learned bias table for a key ``n`` tokens back: the first half of the rows is one
    row per distance; the other half covers the distances from there to ``far`` in steps that grow
    geometrically; every distance from ``far`` on shares the last row."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half))))


def distance_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """[buckets, heads] -> float32 [heads, n]: the bias for every distance 0 .. n - 1, where the last
    entry stands for every larger distance too (n - 1 >= far, so it reads the last row)."""
    buckets = rel.shape[0]
    n = max(int(math.ceil(far)), buckets // 2) + 1
    rows = torch.tensor([distance_bucket(d, buckets, far) for d in range(n)], dtype=torch.long)
    assert int(rows[-1]) == buckets - 1
    return rel.to(torch.float32)[rows].t().contiguous()


class PagedAttention(Mixer):
    """q/k/v projection (one fused product), position encoding on q and k, keys and values
    written to their pages, causal attention of every new token over the request's cache,
    output projection. Query head h reads kv head h // (heads / kv_heads); scores are
    q.k / sqrt(head_dim) unless ``scale`` is given; softmax in 32-bit
    (prefixserve/model/llama.py:113-117, prefixserve/model/attention.py:103-120).

    Further parameters, all off by default:

    * ``value_dim``: a value size other than the query/key size. Pages and kernels then run
      with one head size that holds both (``slot_size``); the projections' rows are laid into
      it at bind time with zeros in the unused slots, which change neither q.k nor the output.
    * a position encoding whose ``rotary_dim`` is smaller than the head: the rotating partners
      are laid ``slots / 2`` apart (``head_slots``), the rest of the head meets identity entries
      of the table.
    * ``qk_norm_eps``: after the rotation, every query and key head is divided by its root mean
      square over ``head_dim`` (no weight, eps inside the root), in 32-bit, before the key goes
      to its page.
    * ``own_kv`` False: the layer has no key and value projections; its run reads the cache
      entry another run writes (``LayerRun.writes_cache`` False) with queries of its own.
    * ``exact_weights``: the softmax weights enter the product with the values as they were computed
      in 32-bit instead of rounded to the activation dtype.
    * ``qk_bias``: the q and k projections have biases (names "q_bias", "k_bias"), added in 32-bit.
    * ``qk_norm_weights`` (with ``qk_norm_eps``): the normalized q and k heads are multiplied by
      a weight of ``head_dim`` entries each, shared by the heads (names "q_norm", "k_norm").
    * ``values_are_keys``: there is no value projection; a token's value is its key as
      projected (with its bias, before rotation and norm).
    * ``sink``: a learned number per head (name "sink") whose exponential joins the softmax's
      denominator; it has no key and no value.
    * ``distance_bias`` = {"buckets": B, "far": D}: a learned table [B, heads] (name "rel") whose
      row bucket(i - j) is added to the scaled score of query i and key j (``distance_bucket``).
    * ``head_scale``: a learned number per query head (name "head_scale") that multiplies the head's
      scores beside ``scale``. It is folded, in 32-bit, into the factor each query head is multiplied
      with behind its norm (a weight per head instead of one shared by the heads).
    * ``keep_first`` (with ``window``): a query also sees the sequence's first that many positions,
      at their true places, however far back they lie; their pages are never given back.
    * ``pooled_block`` = P (with ``window``): beside the window's tokens a query at position i sees one
      key and one value for every block of P tokens that lies wholly in front of its window
      (block b = positions bP .. bP + P - 1, seen once bP + P - 1 <= i - window): the means of the
      block's keys and values as the pages hold them, in the same softmax. The means live in a
      cache entry of their own with one place per P tokens (``aux_cache_needs``: "pool"), written
      when the block's last token runs; tokens that have left the window and whose block is not
      complete in front of it are not seen.
    * ``head_gate``: a number per query head and token, sigmoid(W x)_h (name "head_gate",
      [heads, hidden]), multiplies the head's output before the output matrix; 32-bit."""

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int,
                 num_kv_heads: int, head_dim: int, names: Mapping[str, str], position: str | None = None,
                 window: int | None = None, scale: float | None = None, value_dim: int | None = None,
                 qk_norm_eps: float | None = None, own_kv: bool = True, exact_weights: bool = False,
                 qk_bias: bool = False, qk_norm_weights: bool = False, values_are_keys: bool = False,
                 sink: bool = False, distance_bias: Mapping[str, Any] | None = None, head_scale: bool = False,
                 keep_first: int = 0, pooled_block: int = 0, head_gate: bool = False) -> None:
        if num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads not divisible by {num_kv_heads} kv heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.own_kv = bool(own_kv)
        self.exact_weights = bool(exact_weights)
        self.qk_bias, self.qk_norm_weights = bool(qk_bias), bool(qk_norm_weights)
        self.values_are_keys, self.has_sink = bool(values_are_keys), bool(sink)
        self.head_scale = bool(head_scale)
        self.keep_first, self.pooled_block, self.head_gate = int(keep_first), int(pooled_block), bool(head_gate)
        if (self.keep_first or self.pooled_block) and window is None:
            raise ValueError("kept first positions and pooled blocks belong to a sliding window")
        if self.keep_first < 0 or self.pooled_block < 0 or (self.pooled_block and not own_kv):
            raise ValueError("bad kept positions or pooled block (pooled blocks need keys of the layer's own)")
        self.distance_bias = None if distance_bias is None else (int(distance_bias["buckets"]), float(distance_bias["far"]))
        if self.qk_norm_weights and self.qk_norm_eps is None:
            raise ValueError("weights on the q/k norm need qk_norm_eps")
        if self.values_are_keys and (self.value_dim != self.head_dim or not self.own_kv):
            raise ValueError("values that are the keys have the keys' size and belong to a layer with keys of its own")
        if self.qk_bias and not self.own_kv:
            raise ValueError("biases on q and k are implemented for layers with keys of their own")
        if self.distance_bias is not None and not 2 <= self.distance_bias[0] < 2 * self.distance_bias[1]:
            raise ValueError(f"a distance bias needs at least 2 buckets and a reach beyond half of them, got {self.distance_bias}")
        extras = (self.qk_bias or self.qk_norm_weights or self.values_are_keys or self.has_sink
                  or self.distance_bias is not None or self.head_scale or self.keep_first or self.pooled_block
                  or self.head_gate)
        self.masked = bool(self.keep_first or self.pooled_block or self.head_gate)
        if self.masked and (self.has_sink or self.distance_bias is not None):
            raise ValueError("kept positions, pooled blocks and a gate per head are not combined with a sink or a distance bias")
        self.bias = self.q_norm_weight = self.k_norm_weight = self.sink = self.distance_table = None
        self.names = dict(names)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.pos = positions[position] if position is not None else None
        if self.pos is not None and not isinstance(self.pos, RotaryTable):
            raise ValueError("PagedAttention applies rotation tables; other encodings belong to their own mixer")
        rotary = self.head_dim if self.pos is None or self.pos.rotary_dim is None else int(self.pos.rotary_dim)
        self.plain = (self.value_dim == self.head_dim and rotary == self.head_dim and self.qk_norm_eps is None
                      and self.own_kv and not extras)
        if self.plain:
            if head_dim % 16 or not 16 <= head_dim <= 256:
                raise ValueError(f"head_dim must be a multiple of 16 in [16, 256], got {head_dim}")
            self.slots = self.head_dim
            self.index = None
        else:
            if self.head_dim < 1 or self.value_dim < 1 or rotary > self.head_dim:
                raise ValueError(f"bad head sizes: {self.head_dim}, {self.value_dim}, rotating {rotary}")
            self.slots = slot_size(self.head_dim, self.value_dim)
            self.index = head_slots(self.head_dim, rotary, self.slots)
        if isinstance(self.pos, RotaryTable) and self.pos.head_dim != self.slots:
            raise ValueError(f"the rotation table is made for heads of {self.pos.head_dim}, attention runs with {self.slots}")
        # The norm kernels in front may be skipped only by the form whose first kernel normalizes.
        self.takes_normed_rows = self.plain
        self.q_size = self.num_heads * self.slots
        self.kv_size = self.num_kv_heads * self.slots if self.own_kv else 0
        self.row_width = self.q_size + (1 if self.values_are_keys else 2) * self.kv_size

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        want = {n["q"]: WeightWant((self.num_heads * self.head_dim, h)),
                n["o"]: WeightWant((h, self.num_heads * self.value_dim))}
        if self.own_kv:
            want[n["k"]] = WeightWant((self.num_kv_heads * self.head_dim, h))
            if not self.values_are_keys:
                want[n["v"]] = WeightWant((self.num_kv_heads * self.value_dim, h))
        if self.qk_bias:
            want[n["q_bias"]] = WeightWant((self.num_heads * self.head_dim,), "bias")
            want[n["k_bias"]] = WeightWant((self.num_kv_heads * self.head_dim,), "bias")
        if self.qk_norm_weights:
            want[n["q_norm"]] = WeightWant((self.head_dim,), "norm")
            if self.own_kv:                  # a layer that reads another layer's keys reads them as normed there
                want[n["k_norm"]] = WeightWant((self.head_dim,), "norm")
        if self.head_scale:
            want[n["head_scale"]] = WeightWant((self.num_heads,), "norm")
        if self.has_sink:
            want[n["sink"]] = WeightWant((self.num_heads,), "bias")
        if self.distance_bias is not None:
            want[n["rel"]] = WeightWant((self.distance_bias[0], self.num_heads), "bias")
        if self.head_gate:
            want[n["head_gate"]] = WeightWant((self.num_heads, h))
        return want

    def cache_need(self) -> CacheNeed:
        if self.pooled_block:
            # A block's tokens must still be in their pages when its last one runs.
            return CacheNeed(self.num_kv_heads, self.slots, max(self.window, self.pooled_block), self.keep_first)
        return CacheNeed(self.num_kv_heads, self.slots, self.window, self.keep_first)

    def aux_cache_needs(self) -> dict[str, CacheNeed]:
        if not self.pooled_block:
            return {}
        return {"pool": CacheNeed(self.num_kv_heads, self.slots, None, 0, self.pooled_block)}

    def _spread(self, w: torch.Tensor, heads: int, size: int, index: "list[int] | None") -> torch.Tensor:
        """Rows [heads * size, K] laid into [heads * slots, K]; ``index``: slot of each row of a head."""
        out = torch.zeros((heads, self.slots, w.shape[1]), dtype=w.dtype)
        out[:, list(range(size)) if index is None else index, :] = w.view(heads, size, w.shape[1])
        return out.view(heads * self.slots, w.shape[1])

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n = self.names
        if self.plain:
            # Rows of q, then k, then v: one product per layer instead of three
            # (prefixserve/model/weights.py:115-119). No permutation: checkpoints are laid
            # out for the rotate-half pairing already.
            self.w_qkv = rt.ops.prepare_matrix(torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]], dim=0), rt)
            self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
            return
        rows = [self._spread(tensors[n["q"]], self.num_heads, self.head_dim, self.index)]
        if self.own_kv:
            rows.append(self._spread(tensors[n["k"]], self.num_kv_heads, self.head_dim, self.index))
            if not self.values_are_keys:
                rows.append(self._spread(tensors[n["v"]], self.num_kv_heads, self.value_dim, None))
        self.w_qkv = rt.ops.prepare_matrix(torch.cat(rows, dim=0), rt)
        o = tensors[n["o"]]
        wide = torch.zeros((o.shape[0], self.num_heads, self.slots), dtype=o.dtype)
        # A value that is the key lies in the key's slots.
        cols = self.index if self.values_are_keys else list(range(self.value_dim))
        wide[:, :, cols] = o.view(o.shape[0], self.num_heads, self.value_dim)
        self.w_o = rt.ops.prepare_matrix(wide.view(o.shape[0], self.num_heads * self.slots), rt)

        def on_device(t: torch.Tensor) -> torch.Tensor:
            return t.to(device=rt.device, dtype=torch.float32).contiguous()

        self.bias = self.q_norm_weight = self.k_norm_weight = self.sink = self.distance_table = None
        if self.qk_bias:
            both = [self._spread(tensors[n[key]].to(torch.float32)[:, None], heads, self.head_dim, self.index)
                    for key, heads in (("q_bias", self.num_heads), ("k_bias", self.num_kv_heads))]
            self.bias = on_device(torch.cat(both, dim=0).view(-1))
        self.q_weight_per_head = False
        if self.qk_norm_weights:
            self.q_norm_weight = on_device(self._spread(tensors[n["q_norm"]].to(torch.float32)[:, None], 1, self.head_dim, self.index).view(-1))
            if self.own_kv:
                self.k_norm_weight = on_device(self._spread(tensors[n["k_norm"]].to(torch.float32)[:, None], 1, self.head_dim, self.index).view(-1))
        if self.head_scale:
            # score = scale * number[h] * q.k: the number goes into the query head's factor, [heads, slots].
            per_head = tensors[n["head_scale"]].to(torch.float32).view(-1, 1)
            shared = self.q_norm_weight.cpu() if self.q_norm_weight is not None else \
                self._spread(torch.ones((self.head_dim, 1)), 1, self.head_dim, self.index).view(-1)
            self.q_norm_weight = on_device((per_head * shared[None, :]).reshape(-1))
            self.q_weight_per_head = True
        if self.head_gate:
            self.w_gate = rt.ops.prepare_matrix(tensors[n["head_gate"]], rt)
        if self.has_sink:
            self.sink = on_device(tensors[n["sink"]])
        if self.distance_bias is not None:
            self.distance_table = on_device(distance_table(tensors[n["rel"]].to(torch.float32), self.distance_bias[1]))

    def weight_bytes(self) -> int:
        gate = self.w_gate.numel() * self.w_gate.element_size() if self.head_gate else 0
        return sum(w.numel() * w.element_size() for w in (self.w_qkv, self.w_o)) + gate

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t = x.shape[0]
        table = self.pos.table if self.pos is not None else None
        if writes_cache and not self.own_kv:
            raise ValueError("a layer without keys and values of its own cannot write a cache entry")
        if self.plain:
            qkv = ws.get("attn.qkv", (t, self.q_size + 2 * self.kv_size), rt.dtype)
            ops.qkv_rope_append(x, self.w_qkv, qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx.positions, table,
                                cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot)
        else:
            # Product, then one kernel that rotates, divides by the root mean square and writes
            # the pages (the statistic needs a whole head, which the fused product spreads over
            # workgroups).
            own = self.num_kv_heads if self.own_kv else 0
            qkv = ws.get("attn.qkv" if own else "attn.q", (t, self.row_width), rt.dtype)
            ops.linear(x, self.w_qkv, qkv)
            norm_dim, eps = (self.head_dim, self.qk_norm_eps) if self.qk_norm_eps is not None else (0, 0.0)
            if self.head_scale:
                ops.rope_norm_kv_append(qkv, self.num_heads, own, self.slots, ctx.positions, table,
                                        cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot,
                                        norm_dim, eps, bias=self.bias, q_weight=self.q_norm_weight,
                                        k_weight=self.k_norm_weight, values_from_keys=self.values_are_keys,
                                        q_weight_per_head=self.q_weight_per_head)
            elif self.qk_bias or self.qk_norm_weights or self.values_are_keys:
                ops.rope_norm_kv_append(qkv, self.num_heads, own, self.slots, ctx.positions, table,
                                        cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot,
                                        norm_dim, eps, bias=self.bias, q_weight=self.q_norm_weight,
                                        k_weight=self.k_norm_weight, values_from_keys=self.values_are_keys)
            else:
                ops.rope_norm_kv_append(qkv, self.num_heads, own, self.slots, ctx.positions, table,
                                        cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot,
                                        norm_dim, eps)
        out = ws.get("attn.out", (t, self.q_size), rt.dtype)
        if self.masked:
            gate = pooled = None
            if self.head_gate:
                gate = ws.get("attn.gate", (t, self.num_heads), torch.float32)
                ops.linear(x, self.w_gate, gate)
            if self.pooled_block:
                pool = cache.aux["pool"]
                if writes_cache:
                    ops.pool_kv_append(cache.kv, pool.kv, ctx, cache.group, pool.group, self.num_kv_heads, self.slots,
                                       self.pooled_block)
                pooled = (pool.kv, pool.group, self.pooled_block)
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, self.window, exact_weights=self.exact_weights,
                                keep_first=self.keep_first, pooled=pooled, head_gate=gate)
        elif self.sink is not None or self.distance_table is not None:
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, cache.window, exact_weights=self.exact_weights,
                                sink=self.sink, dist_bias=self.distance_table)
        elif self.exact_weights:
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, cache.window, exact_weights=True)
        else:
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, cache.window)
        return ops.linear_to_residual(out, self.w_o, "attn.delta", getattr(ctx, "residual", None))


register_mixer("paged_attention", PagedAttention)
