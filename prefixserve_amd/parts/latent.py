"""Latent attention: keys and values made from one compressed vector per token."""

from __future__ import annotations

import math
from typing import TYPE_CHECKING, Any, Mapping

import torch

from .attention import slot_size
from .base import CacheNeed, Mixer, PositionEncoding, RotaryTable, Runtime, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class LatentAttention(Mixer):
    """Every token is projected down to ``rank`` numbers c (divided by their root mean square and
    weighted) and ``rot_dim`` more, a rotated key part that all heads share. Head h's key is
    [U_h c | shared part], its value V_h c, its query [``head_dim`` un-rotated | ``rot_dim``
    rotated] dimensions of one projection; the score is their product times ``scale``.

    Only c and the shared part are cached, and attention runs in the compressed space: the
    query's un-rotated part is folded through U_h first (q . U_h c = (U_h^T q) . c), all heads
    then read the one cached "head" [c | shared part], and the weighted sum of c is unfolded
    through V_h afterwards. The cache entry has one kv head of ``rank + rot_dim`` dimensions
    (rounded up to a size the attention kernels take), its value is c.

    The rotation pairs neighbouring dimensions (2i, 2i + 1) and takes its angles from a rotation
    table of ``rot_dim`` dimensions. Optional: a sliding ``window`` and a learned ``sink`` per
    head. ``names``: "q", "down", "down_norm", "up_k", "up_v", "o" and "sink"."""

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], num_heads: int, head_dim: int,
                 rot_dim: int, value_dim: int, rank: int, names: Mapping[str, str], norm_eps: float,
                 position: str | None = None, scale: float | None = None, window: int | None = None,
                 sink: bool = False) -> None:
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.rot_dim, self.value_dim, self.rank = int(head_dim), int(rot_dim), int(value_dim), int(rank)
        if self.rot_dim % 2 or min(self.num_heads, self.rank, self.value_dim) < 1 or self.head_dim < 0:
            raise ValueError(f"bad sizes: heads {num_heads}, dim {head_dim}, rotated {rot_dim}, values {value_dim}, rank {rank}")
        self.names = dict(names)
        self.norm_eps = float(norm_eps)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim + self.rot_dim)
        self.window = None if window is None else int(window)
        self.has_sink = bool(sink)
        self.pos = positions[position] if position is not None else None
        if self.rot_dim:
            if not isinstance(self.pos, RotaryTable) or self.pos.head_dim != self.rot_dim \
                    or (self.pos.rotary_dim or self.rot_dim) != self.rot_dim:
                raise ValueError(f"the rotated part needs a rotation table of {self.rot_dim} dimensions")
        self.slots = slot_size(self.rank + self.rot_dim, self.rank, largest=512)
        self.q_width = self.num_heads * (self.head_dim + self.rot_dim)

    def weights(self) -> dict[str, WeightWant]:
        h, n, heads = self.hidden_size, self.names, self.num_heads
        want = {n["q"]: WeightWant((self.q_width, h)),
                n["down"]: WeightWant((self.rank + self.rot_dim, h)),
                n["down_norm"]: WeightWant((self.rank,), "norm"),
                n["up_k"]: WeightWant((heads * self.head_dim, self.rank)),
                n["up_v"]: WeightWant((heads * self.value_dim, self.rank)),
                n["o"]: WeightWant((h, heads * self.value_dim))}
        if self.has_sink:
            want[n["sink"]] = WeightWant((heads,), "bias")
        return want

    def cache_need(self) -> CacheNeed:
        return CacheNeed(1, self.slots, self.window)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n, heads = self.names, self.num_heads
        # Queries and the projection down are one product.
        self.w_in = rt.ops.prepare_matrix(torch.cat([tensors[n["q"]], tensors[n["down"]]], dim=0), rt)
        up_k = tensors[n["up_k"]].view(heads, self.head_dim, self.rank)
        self.w_fold = rt.ops.prepare_matrix(up_k.transpose(1, 2).contiguous(), rt)          # [H, rank, dim]: q -> U^T q
        self.w_unfold = rt.ops.prepare_matrix(tensors[n["up_v"]].view(heads, self.value_dim, self.rank), rt)
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        self.norm_weight = tensors[n["down_norm"]].to(device=rt.device, dtype=torch.float32).contiguous()
        self.sink = tensors[n["sink"]].to(device=rt.device, dtype=torch.float32).contiguous() if self.has_sink else None

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_fold, self.w_unfold, self.w_o))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, heads = x.shape[0], self.num_heads
        rows = ws.get("latent.in", (t, self.w_in.shape[0]), rt.dtype)
        ops.linear(x, self.w_in, rows)
        q_lat = ws.get("latent.q", (t, heads * self.slots), rt.dtype)
        ops.latent_kv_append(rows, q_lat, heads, self.head_dim, self.rot_dim, self.rank, self.slots, ctx.positions,
                             self.pos.table if self.rot_dim else None, self.norm_weight, self.norm_eps,
                             cache.kv if writes_cache else None, ctx.groups[cache.group].write_slot)
        if self.head_dim:
            ops.heads_linear(rows, 0, self.head_dim + self.rot_dim, self.w_fold, q_lat, 0, self.slots)
        else:
            q_lat.view(t, heads, self.slots)[:, :, : self.rank].zero_()
        mixed = ws.get("latent.mixed", (t, heads * self.slots), rt.dtype)
        ops.paged_attention(q_lat, mixed, cache.kv, ctx, cache.group, heads, 1, self.slots, self.scale, cache.window,
                            exact_weights=True, sink=self.sink)
        out = ws.get("latent.out", (t, heads * self.value_dim), rt.dtype)
        ops.heads_linear(mixed, 0, self.slots, self.w_unfold, out, 0, self.value_dim)
        return ops.linear_to_residual(out, self.w_o, "attn.delta", getattr(ctx, "residual", None))


register_mixer("latent_attention", LatentAttention)
