"""Grouped-query attention over the paged cache.

As the reference's ``Attention::forward`` (crates/model/src/attention.rs:61-103): three
bias-free projections (here fused into one product over the row-concatenated weights), heads
split column-wise (column ``h * d + j`` is head ``h``, dim ``j``), rotation of q and k by
absolute position, K and V of the new tokens written to the cache before attention reads them
(crates/model/src/paged.rs:324-337), query head ``h`` using KV head ``h / group``
(attention.rs:166-171), scores scaled by ``scale``, float32 softmax, heads merged head-major,
output projection."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import (BuildContext, CacheBinding, CacheRequest, Mixer, PartSpec, TensorSpec, join,
                   project, register)
from .rope import shared_position


@register("mixer", "attention")
class PagedAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``num_kv_heads``, ``head_dim``, ``scale``,
    ``window`` (None: all earlier positions), ``position`` (a PartSpec); optional ``value_dim``
    (size of a value head when it differs from ``head_dim``, the size of a query and key head)
    and ``names`` (the tensors of q, k, v and o under the prefix; default ``q_proj.weight`` and
    so on).

    With ``value_dim != head_dim`` the kernels run at one head size ``D``, the larger of the two
    rounded up to a multiple of 16: the rows of the narrower projection's weight are padded
    with zero rows per head at build time (and the output projection's columns with zero
    columns), so the extra query and key dims add exact zeros to every score and the extra
    value dims come out as exact zeros that meet zero columns.  The kernels stay specialised on
    one head size; the price is that the narrower of keys and values is cached at ``D``.

    What the position part may carry: ``rot_dim``, ``cos``, ``sin`` (float32 tables, a rotation
    of the first ``rot_dim`` dims of every q and k head; rot_dim 0: none), ``interleaved``
    (the rotation pairs dim 2j with 2j + 1 instead of j with j + rot/2), ``bias_slopes``
    (float32, one per query head: slope * (key position - query position) is added to the
    scores).  The reference's Llama uses the first three (crates/model/src/rope.rs:61-117)."""

    graph_safe = True
    takes_normed_input = True

    @classmethod
    def _names(cls, params: Dict[str, Any], prefix: str) -> Dict[str, str]:
        names = {**{n: f"{n}_proj.weight" for n in "qkvo"}, **(params.get("names") or {})}
        return {k: join(prefix, v) for k, v in names.items()}

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        H, nh, nkv, d = (params[k] for k in ("hidden_size", "num_heads", "num_kv_heads",
                                             "head_dim"))
        dv = params.get("value_dim") or d
        n = cls._names(params, prefix)
        return [TensorSpec(n["q"], (nh * d, H)), TensorSpec(n["k"], (nkv * d, H)),
                TensorSpec(n["v"], (nkv * dv, H)), TensorSpec(n["o"], (H, nh * dv))]

    @staticmethod
    def _pad_heads(w: torch.Tensor, heads: int, size: int, to: int, rows: bool) -> torch.Tensor:
        """A projection whose heads of ``size`` lie along its rows (or columns) with every head
        padded to ``to`` by zeros."""
        if size == to:
            return w
        if rows:
            out = w.new_zeros((heads, to, w.shape[1]))
            out[:, :size] = w.reshape(heads, size, w.shape[1])
            return out.reshape(heads * to, w.shape[1])
        out = w.new_zeros((w.shape[0], heads, to))
        out[:, :, :size] = w.reshape(w.shape[0], heads, size)
        return out.reshape(w.shape[0], heads * to)

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        qk_dim = int(params["head_dim"])
        v_dim = int(params.get("value_dim") or qk_dim)
        # the one head size the kernels run at
        self.head_dim = qk_dim if v_dim == qk_dim else -(-max(qk_dim, v_dim) // 16) * 16
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"attention: {self.num_heads} heads are not a multiple of "
                             f"{self.num_kv_heads} KV heads")
        names = self._names(params, prefix)
        q, k, v = (ctx.weights.pop(names[n]) for n in "qkv")
        if not (q.dtype == k.dtype == v.dtype):
            q, k, v = (t.to(torch.float32) for t in (q, k, v))
        q = self._pad_heads(q, self.num_heads, qk_dim, self.head_dim, rows=True)
        k = self._pad_heads(k, self.num_kv_heads, qk_dim, self.head_dim, rows=True)
        v = self._pad_heads(v, self.num_kv_heads, v_dim, self.head_dim, rows=True)
        # One product for q, k and v: the rows of the three weights, concatenated.
        self.w_qkv = torch.cat([q, k, v], dim=0).contiguous()
        del q, k, v
        self.w_o = self._pad_heads(ctx.take(names["o"]), self.num_heads, v_dim, self.head_dim,
                                   rows=False).contiguous()
        self.act_dtype = ctx.act_dtype
        self.position = shared_position(params.get("position") or PartSpec("none"), ctx)
        if self.position.rot_dim > qk_dim:
            raise ValueError("attention: the rotated width exceeds the head size")

        self.planner = ops.attention_planner(
            self.num_heads, self.num_kv_heads, self.head_dim, self.act_dtype,
            biased=getattr(self.position, "bias_slopes", None) is not None)

    def cache_request(self) -> CacheRequest:
        return CacheRequest.kv(self.num_kv_heads, self.head_dim, self.window)

    def step_planner(self):
        return self.planner

    def forward(self, x: Any, step: Any, binding: CacheBinding) -> torch.Tensor:
        group = step.groups[binding.group]
        qkv = project(x, self.w_qkv, self.act_dtype)
        if step.max_context > self.position.max_positions:
            raise ValueError(f"sequence of {step.max_context} positions exceeds max_seq_len "
                             f"{self.position.max_positions}")
        out = ops.rope_attention(qkv, self.num_heads, self.num_kv_heads, self.head_dim,
                                 self.position.cos, self.position.sin, step.positions,
                                 group.slots, binding.k_pages, binding.v_pages, group.page_size,
                                 group.block_tables, step, self.scale, self.window,
                                 write_kv=binding.writes, plan=step.plans.get(self.planner.key()),
                                 interleaved=bool(getattr(self.position, "interleaved", False)),
                                 bias_slopes=getattr(self.position, "bias_slopes", None),
                                 counters=binding.counters)
        return ops.pending_linear(out, self.w_o, self.act_dtype)
