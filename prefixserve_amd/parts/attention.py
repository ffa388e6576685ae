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


def slot_size(head_dim: int, value_dim: int) -> int:
    """The head size the pages and kernels run with: the larger of the two sizes, rounded up to
    one the matrix-core attention takes (multiples of 16 up to 128, then 160, 192, 256)."""
    need = max(int(head_dim), int(value_dim))
    for size in (*range(16, 129, 16), 160, 192, 256):
        if need <= size:
            return size
    raise ValueError(f"head sizes up to 256 are implemented, got {need}")


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
      in 32-bit instead of rounded to the activation dtype."""

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int,
                 num_kv_heads: int, head_dim: int, names: Mapping[str, str], position: str | None = None,
                 window: int | None = None, scale: float | None = None, value_dim: int | None = None,
                 qk_norm_eps: float | None = None, own_kv: bool = True, exact_weights: bool = False) -> None:
        if num_kv_heads < 1 or num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads not divisible by {num_kv_heads} kv heads")
        self.hidden_size = int(hidden_size)
        self.num_heads, self.num_kv_heads, self.head_dim = int(num_heads), int(num_kv_heads), int(head_dim)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.own_kv = bool(own_kv)
        self.exact_weights = bool(exact_weights)
        self.names = dict(names)
        self.window = None if window is None else int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.pos = positions[position] if position is not None else None
        if self.pos is not None and not isinstance(self.pos, RotaryTable):
            raise ValueError("PagedAttention applies rotation tables; other encodings belong to their own mixer")
        rotary = self.head_dim if self.pos is None or self.pos.rotary_dim is None else int(self.pos.rotary_dim)
        self.plain = (self.value_dim == self.head_dim and rotary == self.head_dim and self.qk_norm_eps is None
                      and self.own_kv)
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

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        want = {n["q"]: WeightWant((self.num_heads * self.head_dim, h)),
                n["o"]: WeightWant((h, self.num_heads * self.value_dim))}
        if self.own_kv:
            want[n["k"]] = WeightWant((self.num_kv_heads * self.head_dim, h))
            want[n["v"]] = WeightWant((self.num_kv_heads * self.value_dim, h))
        return want

    def cache_need(self) -> CacheNeed:
        return CacheNeed(self.num_kv_heads, self.slots, self.window)

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
            rows.append(self._spread(tensors[n["v"]], self.num_kv_heads, self.value_dim, None))
        self.w_qkv = rt.ops.prepare_matrix(torch.cat(rows, dim=0), rt)
        o = tensors[n["o"]]
        wide = torch.zeros((o.shape[0], self.num_heads, self.slots), dtype=o.dtype)
        wide[:, :, : self.value_dim] = o.view(o.shape[0], self.num_heads, self.value_dim)
        self.w_o = rt.ops.prepare_matrix(wide.view(o.shape[0], self.num_heads * self.slots), rt)

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_qkv, self.w_o))

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
            qkv = ws.get("attn.qkv" if own else "attn.q", (t, self.q_size + 2 * self.kv_size), rt.dtype)
            ops.linear(x, self.w_qkv, qkv)
            ops.rope_norm_kv_append(qkv, self.num_heads, own, self.slots, ctx.positions, table,
                                    cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot,
                                    self.head_dim if self.qk_norm_eps is not None else 0, self.qk_norm_eps or 0.0)
        out = ws.get("attn.out", (t, self.q_size), rt.dtype)
        if self.exact_weights:
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, cache.window, exact_weights=True)
        else:
            ops.paged_attention(qkv, out, cache.kv, ctx, cache.group, self.num_heads, self.num_kv_heads,
                                self.slots, self.scale, cache.window)
        return ops.linear_to_residual(out, self.w_o, "attn.delta", getattr(ctx, "residual", None))


register_mixer("paged_attention", PagedAttention)
