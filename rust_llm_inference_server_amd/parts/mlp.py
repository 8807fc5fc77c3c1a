"""SwiGLU feed-forward: ``down(silu(gate(x)) * up(x))`` with three bias-free projections
(crates/model/src/layers.rs:156-187).  Gate and up run as one product over the row-concatenated
weights; ``silu`` and the product are 32-bit with one rounding."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .. import ops
from .base import BuildContext, FeedForward, TensorSpec, join, project, register


@register("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    """Parameters: ``hidden_size``, ``intermediate_size``."""

    graph_safe = True

    takes_normed_input = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        return [TensorSpec(join(prefix, "gate_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "up_proj.weight"), (I, H)),
                TensorSpec(join(prefix, "down_proj.weight"), (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        gate = ctx.weights.pop(join(prefix, "gate_proj.weight"))
        up = ctx.weights.pop(join(prefix, "up_proj.weight"))
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        del gate, up
        self.w_down = ctx.take(join(prefix, "down_proj.weight"))
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        hidden = project(x, self.w_gate_up, self.act_dtype, gated=True)
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)


@register("feed_forward", "clamped_glu")
class ClampedGLU(FeedForward):
    """A gated unit whose branches are bounded before they meet:
    ``down(g * sigmoid(alpha * g) * (u + 1))`` with ``g = min(gate(x), limit)`` and
    ``u = clamp(up(x), -limit, limit)``; three bias-free projections, gate and up as one
    product over the row-concatenated weights.

    Parameters: ``hidden_size``, ``intermediate_size``, ``limit``, ``alpha`` (1.702 by
    default), ``names`` (the tensors of gate, up and down under the prefix; default
    ``gate_proj.weight`` and so on)."""

    graph_safe = True
    takes_normed_input = True        # the norm in front goes into the gate/up product where it can

    _DEFAULT_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight",
                      "down": "down_proj.weight"}

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str) -> Dict[str, str]:
        names = {**cls._DEFAULT_NAMES, **(params.get("names") or {})}
        return {k: join(prefix, v) for k, v in names.items()}

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, I = params["hidden_size"], params["intermediate_size"]
        n = cls._names(params, prefix)
        return [TensorSpec(n["gate"], (I, H)), TensorSpec(n["up"], (I, H)),
                TensorSpec(n["down"], (H, I))]

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        n = self._names(params, prefix)
        gate, up = ctx.weights.pop(n["gate"]), ctx.weights.pop(n["up"])
        if gate.dtype != up.dtype:
            gate, up = gate.to(torch.float32), up.to(torch.float32)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        del gate, up
        self.w_down = ctx.take(n["down"])
        self.limit = float(params["limit"])
        self.alpha = float(params.get("alpha", 1.702))
        if not self.limit > 0:
            raise ValueError(f"feed-forward 'clamped_glu': limit {self.limit} must be positive")
        self.act_dtype = ctx.act_dtype

    def forward(self, x: Any, step: Any) -> torch.Tensor:
        gu = project(x, self.w_gate_up, self.act_dtype)
        hidden = ops.clamped_glu(gu, self.limit, self.alpha)
        return ops.pending_linear(hidden, self.w_down, self.act_dtype)
