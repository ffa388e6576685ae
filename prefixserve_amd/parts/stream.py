"""Transforms of the residual stream: a factor behind the token table, and the re-entry into a
stretch of layers that is passed through several times."""

from __future__ import annotations

from typing import TYPE_CHECKING, Mapping

import torch

from .base import Runtime, Transform, WeightWant, register_transform

if TYPE_CHECKING:
    from prefixserve_amd.engine.batch import StepContext


class ScaleStream(Transform):
    """t <- factor * t, in 32-bit: the token table's rows times a constant."""

    def __init__(self, hidden_size: int, vocab_size: int, factor: float) -> None:
        self.factor = float(factor)

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        if self.factor != 1.0:
            self.rt.ops.stream_affine(t, self.factor, None)


class StreamReentry(Transform):
    """In front of every pass through a repeated stretch of layers: x <- W [x; x0] + step[pass],
    where x0 is the token table's output (behind its own transforms) and ``step`` has one row per
    pass. The product's operands are in the activation dtype; its sums and the added row are
    32-bit and become the new stream. ``names``: "in" ([hidden, 2 hidden], x's columns first)
    and "step" ([passes, hidden])."""

    needs_embedding_output = True

    def __init__(self, hidden_size: int, vocab_size: int, passes: int, names: Mapping[str, str]) -> None:
        self.hidden_size, self.passes = int(hidden_size), int(passes)
        self.names = dict(names)

    def weights(self) -> dict[str, WeightWant]:
        h, n = self.hidden_size, self.names
        return {n["in"]: WeightWant((h, 2 * h)), n["step"]: WeightWant((self.passes, h), "bias")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        self.w_in = rt.ops.prepare_matrix(tensors[self.names["in"]], rt)
        self.steps = tensors[self.names["step"]].to(device=rt.device, dtype=torch.float32).contiguous()

    def weight_bytes(self) -> int:
        return self.w_in.numel() * self.w_in.element_size()

    def apply(self, t: torch.Tensor, ctx: "StepContext", rows: torch.Tensor | None) -> None:
        rt, ops = self.rt, self.rt.ops
        if not 0 <= ctx.pass_index < self.passes:
            raise ValueError(f"pass {ctx.pass_index} of {self.passes}")
        both = rt.workspace.get("reentry.in", (t.shape[0], 2 * self.hidden_size), rt.dtype)
        ops.concat_to_activation(t, ctx.embedding_output, both)
        ops.linear(both, self.w_in, t)
        ops.stream_affine(t, 1.0, self.steps[ctx.pass_index])


register_transform("scale", ScaleStream)
register_transform("reentry", StreamReentry)
