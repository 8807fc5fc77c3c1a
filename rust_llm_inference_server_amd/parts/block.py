"""Decoder blocks.  The pre-norm block: ``x += mixer(norm(x)); x += feed_forward(norm(x))``
(crates/model/src/llama.rs:264-271).  Which mixer, feed-forward and norms it holds, and under
which weight names, is given by its parameters, layer by layer.  The parallel block:
``x += mixer(h) + feed_forward(h)`` with ``h = norm(x)``, one norm that both sublayers read."""
from __future__ import annotations

from typing import Any, Dict, List

import torch

from .base import (Block, BuildContext, CacheBinding, ResidualStream, TensorSpec,
                   create, join, normed, register, tensor_specs)
from .. import ops


@register("block", "prenorm")
class PreNormBlock(Block):
    """Parameters: ``mixer``, ``feed_forward``, ``mixer_norm``, ``ffn_norm`` (PartSpecs) and
    ``names``: the weight-name suffix of each of the four under the block's prefix.  A block
    whose ``feed_forward`` is None has the mixer's sublayer only.  Optional
    ``residual_scale`` m: each sublayer's output joins the stream as ``x += m * f(norm(x))``,
    the product formed in float32 where the sum is."""

    _SLOTS = (("mixer_norm", "norm"), ("mixer", "mixer"), ("ffn_norm", "norm"),
              ("feed_forward", "feed_forward"))

    @classmethod
    def _slots(cls, params: Dict[str, Any]):
        if params.get("feed_forward") is None:
            return cls._SLOTS[:2]
        return cls._SLOTS

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for slot, category in cls._slots(params):
            out += tensor_specs(category, params[slot], join(prefix, params["names"][slot]))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        built = {slot: create(category, params[slot], join(prefix, params["names"][slot]), ctx)
                 for slot, category in self._slots(params)}
        self.mixer_norm, self.mixer = built["mixer_norm"], built["mixer"]
        self.ffn_norm, self.feed_forward = built.get("ffn_norm"), built.get("feed_forward")
        self.residual_scale = float(params.get("residual_scale", 1.0))

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.mixer_norm, self.mixer, self.ffn_norm,
                                          self.feed_forward) if p is not None)

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        m = self.residual_scale
        stream.add(self.mixer.forward(normed(self.mixer_norm, stream, self.mixer), step, binding),
                   m)
        if self.feed_forward is not None:
            stream.add(self.feed_forward.forward(
                normed(self.ffn_norm, stream, self.feed_forward), step), m)


@register("block", "parallel")
class ParallelBlock(Block):
    """Parameters: ``mixer``, ``feed_forward`` (None: the mixer alone), ``norm`` (PartSpecs) and
    ``names``: the weight-name suffix of each under the block's prefix.  The two sublayers'
    outputs are added in float32 and join the stream as one delta.  A feed-forward that sets
    ``wants_residual`` also gets the float32 residual rows that the norm normalised and the
    norm itself (``forward(h, step, resid=..., norm=...)``), for decisions that it wants to make
    on the unrounded input."""

    _SLOTS = (("norm", "norm"), ("mixer", "mixer"), ("feed_forward", "feed_forward"))

    @classmethod
    def _slots(cls, params: Dict[str, Any]):
        return cls._SLOTS[:2] if params.get("feed_forward") is None else cls._SLOTS

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        out: List[TensorSpec] = []
        for slot, category in cls._slots(params):
            out += tensor_specs(category, params[slot], join(prefix, params["names"][slot]))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        built = {slot: create(category, params[slot], join(prefix, params["names"][slot]), ctx)
                 for slot, category in self._slots(params)}
        self.norm, self.mixer = built["norm"], built["mixer"]
        self.feed_forward = built.get("feed_forward")

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in (self.norm, self.mixer, self.feed_forward)
                   if p is not None)

    def forward(self, stream: ResidualStream, step: Any, binding: CacheBinding) -> None:
        h = self.norm.forward(stream)
        mixed = self.mixer.forward(h, step, binding)
        if self.feed_forward is None:
            stream.add(mixed)
            return
        if getattr(self.feed_forward, "wants_residual", False):
            # (the norm has folded the pending delta in: stream.x is what it normalised)
            fed = self.feed_forward.forward(h, step, resid=stream.x, norm=self.norm)
        else:
            fed = self.feed_forward.forward(h, step)
        mixed, fed = (d if isinstance(d, torch.Tensor) else d.run() for d in (mixed, fed))
        stream.add(ops.weighted_sum(mixed, 1.0, fed, 1.0, round_parts=stream.round_parts))
