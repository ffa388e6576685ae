"""A gated linear recurrence behind a short convolution: a mixer with fixed-size state per request."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, Mapping

import torch

from .base import Mixer, PositionEncoding, Runtime, StateNeed, WeightWant, register_mixer

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class GatedLinearRecurrence(Mixer):
    """Two branches of ``width`` channels from the input: y = gelu_tanh(W_y h + b_y), and
    u = conv(W_x h + b_x), a causal convolution per channel over ``taps`` tokens (the last tap is
    the token's own; zeros in front of the sequence). u is cut into ``blocks`` parts; in each,
    r = sigmoid(A_r u + .) and i = sigmoid(A_i u + .) with square matrices per part. With
    log a = -``decay_scale`` r softplus(lam): S <- a S + sqrt(1 - a^2) (i u), from S = 0; the
    output is W_o (S y).

    The gates, the decay and its exponential, the step size and S are 32-bit in every mode; the
    per-request state is S and the convolution's last ``taps`` - 1 inputs, in a slot the runner
    clears for a request that starts over. It needs no positions and no pages.
    ``names``: "y", "y_bias", "x", "x_bias", "conv", "conv_bias", "gate_r", "gate_r_bias", "gate_i",
    "gate_i_bias", "lam", "o"."""

    state_in_graphs = True

    def __init__(self, hidden_size: int, positions: Mapping[str, PositionEncoding], width: int, blocks: int, taps: int,
                 names: Mapping[str, str], decay_scale: float = 8.0) -> None:
        self.hidden_size, self.width, self.blocks, self.taps = int(hidden_size), int(width), int(blocks), int(taps)
        if self.blocks < 1 or self.width % self.blocks or not 1 <= self.taps <= 16:
            raise ValueError(f"width {width} in {blocks} blocks, {taps} taps (at most 16)")
        self.names = dict(names)
        self.decay_scale = float(decay_scale)

    def weights(self) -> dict[str, WeightWant]:
        h, w, n, b = self.hidden_size, self.width, self.names, self.blocks
        bw = w // b
        return {n["y"]: WeightWant((w, h)), n["y_bias"]: WeightWant((w,), "bias"),
                n["x"]: WeightWant((w, h)), n["x_bias"]: WeightWant((w,), "bias"),
                n["conv"]: WeightWant((w, self.taps), "bias"), n["conv_bias"]: WeightWant((w,), "bias"),
                n["gate_r"]: WeightWant((b, bw, bw)), n["gate_r_bias"]: WeightWant((b, bw), "bias"),
                n["gate_i"]: WeightWant((b, bw, bw)), n["gate_i_bias"]: WeightWant((b, bw), "bias"),
                n["lam"]: WeightWant((w,), "bias"), n["o"]: WeightWant((h, w))}

    def state_need(self) -> StateNeed:
        # taps - 1 saved inputs of the convolution (oldest first), then the recurrence's S.
        return StateNeed((self.taps * self.width,), torch.float32)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        Mixer.bind(self, tensors, rt)
        n = self.names

        def f32(name: str) -> torch.Tensor:
            return tensors[n[name]].to(torch.float32)

        self.w_in = rt.ops.prepare_matrix(torch.cat([tensors[n["y"]], tensors[n["x"]]], dim=0), rt)     # [y | x] in one product
        self.w_o = rt.ops.prepare_matrix(tensors[n["o"]], rt)
        dev = rt.device
        self.y_bias, self.x_bias = f32("y_bias").contiguous().to(dev), f32("x_bias").contiguous().to(dev)
        self.conv_w, self.conv_b = f32("conv").contiguous().to(dev), f32("conv_bias").contiguous().to(dev)
        # Both gates of a block from one product: rows of r, then rows of i.
        self.w_gates = torch.cat([f32("gate_r"), f32("gate_i")], dim=1).contiguous().to(dev)             # [B, 2 bw, bw]
        self.gate_bias = torch.cat([f32("gate_r_bias"), f32("gate_i_bias")], dim=1).contiguous().to(dev)
        lam = tensors[n["lam"]].to(torch.float64)
        self.decay = (-self.decay_scale * torch.nn.functional.softplus(lam)).to(torch.float32).contiguous().to(dev)

    def weight_bytes(self) -> int:
        return sum(w.numel() * w.element_size() for w in (self.w_in, self.w_o, self.w_gates))

    def forward(self, x: torch.Tensor, ctx: "StepContext", cache: Any, state: torch.Tensor | None,
                writes_cache: bool) -> torch.Tensor | None:
        rt, ops, ws = self.rt, self.rt.ops, self.rt.workspace
        t, w = x.shape[0], self.width
        assert state is not None, "the recurrence keeps its state in a slot"
        rows = ws.get("recurrent.in", (t, 2 * w), rt.dtype)                  # [y | x]
        ops.linear(x, self.w_in, rows)
        u = ws.get("recurrent.u", (t, w), torch.float32)
        ops.causal_conv(rows, w, self.x_bias, self.conv_w, self.conv_b, u, state, ctx)
        gates = ws.get("recurrent.gates", (t, 2 * w), torch.float32)         # per block: r's sums, then i's
        bw = w // self.blocks
        ops.heads_linear(u, 0, bw, self.w_gates, gates, 0, 2 * bw)
        out = ws.get("recurrent.out", (t, w), rt.dtype)
        ops.gated_scan(gates, self.gate_bias, u, self.decay, rows, 0, w, self.y_bias, self.x_bias, out, state, ctx,
                       self.blocks, self.taps)
        return ops.linear_to_residual(out, self.w_o, "recurrent.delta", getattr(ctx, "residual", None))


register_mixer("gated_linear_recurrence", GatedLinearRecurrence)
