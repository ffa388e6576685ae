"""Feed-forward as a mixture of experts: a router picks a few small gated feed-forwards per token."""

from __future__ import annotations

from typing import TYPE_CHECKING, Mapping

import torch

from .base import FeedForward, Runtime, WeightWant, register_feed_forward

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class RoutedExperts(FeedForward):
    """``num_experts`` gated feed-forwards of inner size ``intermediate_size`` without biases, of
    which every token uses ``top_k``.

    Router: z = W_r x in 32-bit, score = sigmoid(z); the ``top_k`` largest scores are taken
    (the lower index among equals) and are the weights as they are, not renormalized. The
    weight multiplies the expert's *input*: the output is the sum over the chosen experts of
    expert(w x), which is not w expert(x) because the expert clamps.

    Expert: with g = min(W_gate h, limit) and u = clamp(W_up h, -limit, limit) it is
    W_down (g sigmoid(gate_alpha g) (u + up_shift)).

    The chosen experts' outputs come back as ``top_k`` float32 slices ``[top_k, T, hidden]`` that
    the norm behind adds up in ascending order, so a token's sum does not depend on what else
    is in the step. ``names``: "router", and "gate"/"up"/"down" with ``{e}`` for the expert."""

    def __init__(self, hidden_size: int, num_experts: int, top_k: int, intermediate_size: int,
                 names: Mapping[str, str], limit: float, gate_alpha: float = 1.702, up_shift: float = 1.0,
                 score: str = "sigmoid", renormalize: bool = False, weight_on: str = "input") -> None:
        if score != "sigmoid" or renormalize or weight_on != "input":
            raise ValueError("the router kernel scores with a sigmoid, keeps the scores as weights and applies them "
                             f"to the experts' input; got score={score!r}, renormalize={renormalize}, weight_on={weight_on!r}")
        if not 1 <= top_k <= num_experts:
            raise ValueError(f"top_k {top_k} of {num_experts} experts")
        self.hidden_size, self.num_experts, self.top_k = int(hidden_size), int(num_experts), int(top_k)
        self.intermediate_size = int(intermediate_size)
        self.names = dict(names)
        self.limit, self.gate_alpha, self.up_shift = float(limit), float(gate_alpha), float(up_shift)

    def weights(self) -> dict[str, WeightWant]:
        h, f, n = self.hidden_size, self.intermediate_size, self.names
        want = {n["router"]: WeightWant((self.num_experts, h))}
        for e in range(self.num_experts):
            want[n["gate"].format(e=e)] = WeightWant((f, h))
            want[n["up"].format(e=e)] = WeightWant((f, h))
            want[n["down"].format(e=e)] = WeightWant((h, f))
        return want

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        n, e_n = self.names, self.num_experts
        # The router stays 32-bit whatever the activation dtype.
        self.w_router = tensors[n["router"]].to(device=rt.device, dtype=torch.float32).contiguous()
        # ... and also stands in the activation dtype for steps whose logits a product kernel computes
        # (bfloat16 x bfloat16 products are exact in float32, where they are summed).
        self.w_router_act = self.w_router if rt.dtype == torch.float32 else rt.ops.prepare_matrix(tensors[n["router"]], rt)
        # Per expert the rows of gate, then of up: [E, 2F, H]; and down [E, H, F].
        gate_up = torch.stack([torch.cat([tensors[n["gate"].format(e=e)], tensors[n["up"].format(e=e)]], dim=0)
                               for e in range(e_n)])
        self.w_gate_up = rt.ops.prepare_matrix(gate_up, rt)
        self.w_down = rt.ops.prepare_matrix(torch.stack([tensors[n["down"].format(e=e)] for e in range(e_n)]), rt)

    def weight_bytes(self) -> int:
        """What a decode step of one token reads: the router and ``top_k`` experts."""
        per_expert = (self.w_gate_up.numel() + self.w_down.numel()) // self.num_experts * self.w_down.element_size()
        return self.w_router.numel() * 4 + self.top_k * per_expert

    def forward(self, x: torch.Tensor, ctx: "StepContext") -> torch.Tensor:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, k = x.shape[0], self.top_k
        chosen = ws.get("moe.chosen", (t, k), torch.int32)
        weight = ws.get("moe.weight", (t, k), torch.float32)
        ops.moe_route(x, self.w_router, chosen, weight, self.w_router_act)
        act = ws.get("moe.act", (t * k, self.intermediate_size), rt.dtype)
        out = ws.get("moe.out", (k, t, self.hidden_size), torch.float32)
        ops.moe_experts(x, chosen, weight, self.w_gate_up, self.w_down, act, out, self.gate_alpha, self.limit, self.up_shift)
        return out


register_feed_forward("routed_experts", RoutedExperts)
