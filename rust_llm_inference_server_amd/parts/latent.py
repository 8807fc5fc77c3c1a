"""Attention whose keys and values are linear maps of one cached latent per position.

Per token the mixer makes queries ``q = Wq h`` (per head ``dim`` numbers that meet the key
made from the latent, then ``rot_dim`` numbers that meet a rotated key part), and
``Wdkv h``: ``kv_rank`` numbers that an RMS norm turns into the latent ``c``, then ``rot_dim``
numbers that are rotated by position and serve every head as the second part of its key.
Head ``h`` has ``k_h = Uk_h c`` and ``v_h = Uv_h c``; its score for a cached position is
``(q_h . k_h + q_rot_h . k_rot) * scale``.  Only ``[c | k_rot]`` is cached, one row per
position, and both maps are taken to the query side (``Uk_h^T q_h`` meets ``c``; the weighted
sum of cached latents goes through ``Uv_h`` afterwards), so the cache is read as it lies.  (In
bfloat16 the latent is kept a second time with the positions of a page innermost, which is how
the matrix-core kernel loads it as values.)

Options, each a parameter: a rotated part (``rot_dim`` 0: none), a sliding window, a learned
sink per head in the softmax's denominator, a sigmoid gate on the heads' outputs (its own
projection of the mixer's input), and reading the latents that an earlier run has cached
instead of making one's own (the run's binding then does not write, and the mixer has no
down projection).  Scores, softmax, the latent's norm and the rotation are float32."""
from __future__ import annotations

from typing import Any, Dict, List, Optional

import torch

from .. import ops
from .base import (PAGE, BuildContext, CacheBinding, CacheRequest, Mixer, PageArray, PartSpec,
                   TensorSpec, join, register)
from .rope import shared_position


@register("mixer", "latent_attention")
class LatentAttention(Mixer):
    """Parameters: ``hidden_size``, ``num_heads``, ``head_dim`` (unrotated query/key size),
    ``rot_dim`` (0: none), ``value_dim``, ``kv_rank``, ``scale``, ``eps`` (of the latent's
    norm), ``window`` (None: every earlier position), ``cache_window`` (what the cache keeps:
    the widest window among the runs that read it; None: everything), ``sink`` (bool),
    ``gate`` (bool), ``own_latent`` (False: reads another run's cache), ``position`` (a
    PartSpec, needed with ``rot_dim``).

    Tensors under the prefix: ``q`` (heads * (dim + rot_dim), W); ``dkv`` (kv_rank + rot_dim,
    W) and ``dkv.norm`` (kv_rank) with ``own_latent``; ``uk`` (heads * dim, kv_rank), ``uv``
    (heads * vdim, kv_rank); ``sink`` (heads); ``g`` (heads * vdim, W); ``o`` (W, heads *
    vdim)."""

    graph_safe = True

    @classmethod
    def tensor_specs(cls, params: Dict[str, Any], prefix: str) -> List[TensorSpec]:
        W, H, d, r = (params[k] for k in ("hidden_size", "num_heads", "head_dim", "rot_dim"))
        dv, R = params["value_dim"], params["kv_rank"]
        out = [TensorSpec(join(prefix, "q"), (H * (d + r), W))]
        if params.get("own_latent", True):
            out += [TensorSpec(join(prefix, "dkv"), (R + r, W)),
                    TensorSpec(join(prefix, "dkv.norm"), (R,), init="ones_normal")]
        out += [TensorSpec(join(prefix, "uk"), (H * d, R)), TensorSpec(join(prefix, "uv"), (H * dv, R))]
        if params.get("sink"):
            out.append(TensorSpec(join(prefix, "sink"), (H,), std=1.0))
        if params.get("gate"):
            out.append(TensorSpec(join(prefix, "g"), (H * dv, W)))
        out.append(TensorSpec(join(prefix, "o"), (W, H * dv)))
        return out

    def __init__(self, params: Dict[str, Any], prefix: str, ctx: BuildContext):
        super().__init__(params, prefix, ctx)
        self.heads, self.dim = int(params["num_heads"]), int(params["head_dim"])
        self.rot_width, self.vdim = int(params["rot_dim"]), int(params["value_dim"])
        self.rank = int(params["kv_rank"])
        self.scale, self.eps = float(params["scale"]), float(params["eps"])
        self.window: Optional[int] = params.get("window")
        self.cache_window: Optional[int] = params.get("cache_window", self.window)
        if self.window is not None and (self.cache_window is not None
                                        and self.cache_window < self.window):
            raise ValueError("latent_attention: the cache keeps fewer positions than the window")
        self.own_latent = bool(params.get("own_latent", True))
        if not self.own_latent and self.rot_width:
            raise ValueError("latent_attention: a mixer that reads another's latents has no "
                             "rotated key part of its own")
        self.act_dtype = ctx.act_dtype
        take = lambda n: ctx.take(join(prefix, n))
        H, d, dv, R = self.heads, self.dim, self.vdim, self.rank
        self.w_q = take("q")
        if self.own_latent:
            self.w_dkv = take("dkv")
            self.norm = take("dkv.norm").to(torch.float32).contiguous()
        # per head, as (out, in): Uk^T (rank x dim) in front of the attention, Uv (vdim x rank)
        # behind it
        self.w_uk_t = take("uk").to(ctx.act_dtype).reshape(H, d, R).transpose(1, 2).contiguous()
        self.w_uv = take("uv").to(ctx.act_dtype).reshape(H, dv, R).contiguous()
        self.sink = take("sink").to(torch.float32).contiguous() if params.get("sink") else None
        self.w_g = take("g") if params.get("gate") else None
        self.w_o = take("o")
        # the matrix-core kernel reads the latents as values from a second copy that lies with
        # the positions of a page innermost; the mixer keeps it where that kernel applies
        self.keeps_transposed = ctx.device.type == "cuda" and ops.latent_mfma_ok(
            ctx.act_dtype, R, R + self.rot_width)
        self.position = None
        self.rot_dims = 0
        if self.rot_width:
            self.position = shared_position(params.get("position") or PartSpec("none"), ctx)
            self.rot_dims = int(self.position.rot_dim)
            if self.rot_dims > self.rot_width:
                raise ValueError("latent_attention: more rotated dims than the rotated part has")

    def cache_request(self) -> CacheRequest:
        arrays = (PageArray("latent", (PAGE, self.rank + self.rot_width)),)
        if self.keeps_transposed:
            arrays += (PageArray("latent_t", (self.rank, PAGE)),)
        return CacheRequest(arrays, self.cache_window)

    def forward(self, x: torch.Tensor, step: Any, binding: CacheBinding) -> Any:
        group = step.groups[binding.group]
        pages, pages_t = binding.pages["latent"], binding.pages.get("latent_t")
        H, d, r, R = self.heads, self.dim, self.rot_width, self.rank
        T = x.shape[0]
        if self.position is not None and step.max_context > self.position.max_positions:
            raise ValueError(f"sequence of {step.max_context} positions exceeds max_seq_len "
                             f"{self.position.max_positions}")
        q = ops.linear(x, self.w_q, self.act_dtype)                    # (T, H * (d + r))
        q_lat = torch.empty((T, H * (R + r)), dtype=self.act_dtype, device=x.device)
        ops.head_linear(q, self.w_uk_t, d + r, out=q_lat, out_head=R + r)
        writes = binding.writes and self.own_latent
        if writes or r:
            down = ops.linear_f32(x, self.w_dkv) if writes else None
            cos = self.position.cos if self.rot_dims else None
            sin = self.position.sin if self.rot_dims else None
            ops.latent_write(down, self.norm if writes else None, self.eps, R, r, self.rot_dims,
                             cos, sin, step.positions, group.slots if writes else None, pages,
                             q if r else None, d + r, q_lat if r else None, H, pages_t)
        mixed = ops.latent_attention(q_lat, pages, group.block_tables, step.seq_of_token,
                                     step.positions, H, R, self.scale, self.window, self.sink,
                                     pages_t, step.cu_seqlens, step.num_seqs)
        out = ops.head_linear(mixed, self.w_uv, R)                     # (T, H * vdim)
        if self.w_g is not None:
            ops.sigmoid_gate_(out, ops.linear(x, self.w_g, self.act_dtype))
        return ops.pending_linear(out, self.w_o, self.act_dtype)
