"""The kernels of attention over a cached latent (``csrc/kernels/latent.hip``) as Python
functions: one product per head, the norm / rotation / cache write of a step's tokens, the
attention itself over cached rows ``[latent | rotated key part]``, and a sigmoid gate.

Keys and values of such a mixer are linear maps of the cached latent, and both maps are taken
to the query side (``head_linear`` in front of and behind the attention), so the cache is read
as it lies, once for all heads.  Every function checks on the host what its kernel assumes."""
from __future__ import annotations

from typing import Optional

import torch

from . import lib
from .lib import KernelError

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _rows2(t: torch.Tensor, what: str) -> int:
    if not t.is_cuda or t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1) \
            or t.dtype not in _DT:
        raise KernelError(f"{what}: a float32 or bfloat16 2-D tensor on the GPU with contiguous "
                          "rows is needed")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, n: int, what: str) -> int:
    if not t.is_cuda or t.dtype != torch.int32 or not t.is_contiguous() or t.numel() < n:
        raise KernelError(f"{what}: needs {n} contiguous int32 entries on the GPU")
    return t.data_ptr()


def head_linear(x: torch.Tensor, w: torch.Tensor, x_head: int, out: Optional[torch.Tensor] = None,
                out_head: Optional[int] = None, out_dtype: Optional[torch.dtype] = None
                ) -> torch.Tensor:
    """``y[t, h] = w[h] @ x[t, h]`` for ``w (H, N, K)`` and rows of ``x`` that hold head ``h``'s
    ``K`` numbers from column ``h * x_head`` on.  The result goes to ``out`` (rows with head
    ``h`` at column ``h * out_head``) or to a new ``(T, H * N)`` tensor."""
    ldx = _rows2(x, "head_linear x")
    if not w.is_cuda or w.dim() != 3 or not w.is_contiguous() or w.dtype != x.dtype:
        raise KernelError("head_linear: the weight must be a contiguous (H, N, K) tensor of x's dtype")
    H, N, K = w.shape
    T = x.shape[0]
    if x.shape[1] < (H - 1) * x_head + K or x_head < K:
        raise KernelError(f"head_linear: rows of {x.shape[1]} do not hold {H} heads {x_head} apart")
    if out is None:
        out_head = N
        out = torch.empty((T, H * N), dtype=out_dtype or x.dtype, device=x.device)
    ldy = _rows2(out, "head_linear out")
    if out.shape[0] != T or out_head is None or out_head < N \
            or out.shape[1] < (H - 1) * out_head + N:
        raise KernelError("head_linear: the result's rows do not hold the heads")
    lib.call("rlis_head_linear", x.data_ptr(), _DT[x.dtype], ldx, int(x_head), w.data_ptr(),
             out.data_ptr(), _DT[out.dtype], ldy, int(out_head), T, H, N, K, lib.stream_ptr())
    return out


def latent_write(x: Optional[torch.Tensor], weight: Optional[torch.Tensor], eps: float, rank: int,
                 rot_width: int, rot_dims: int, cos: Optional[torch.Tensor],
                 sin: Optional[torch.Tensor], positions: torch.Tensor,
                 slots: Optional[torch.Tensor], pages: Optional[torch.Tensor],
                 q: Optional[torch.Tensor], q_head: int, q_out: Optional[torch.Tensor],
                 heads: int, pages_t: Optional[torch.Tensor] = None) -> None:
    """For every token of the step: the first ``rank`` columns of ``x`` (float32), divided by
    their root mean square (``eps`` inside the root) and multiplied by ``weight``, go to the
    token's row of ``pages (pages, page size, rank + rot_width)`` at ``slots``; the
    ``rot_width`` columns behind them follow, the first ``rot_dims`` of them rotated by the
    token's position (entry i with entry i + rot_dims / 2, angles from the float32 tables
    ``cos``/``sin (positions, rot_dims / 2)``).  The last ``rot_width`` numbers of every head
    of ``q`` (heads ``q_head`` apart) are rotated the same way into ``q_out`` behind each
    head's first ``rank`` columns (heads ``rank + rot_width`` apart).  ``x`` None: nothing is
    written to the cache (a mixer that reads another's).  ``pages_t (pages, rank, page size)``:
    the latent is stored there once more, with the positions of a page innermost (what the
    matrix-core attention kernel reads as values)."""
    T = positions.numel() if q is None else q.shape[0]
    write = x is not None
    D = rank + rot_width
    ldx = 0
    if write:
        ldx = _rows2(x, "latent_write x")
        if x.dtype != torch.float32 or x.shape[1] < D:
            raise KernelError(f"latent_write: x must be float32 with at least {D} columns")
        if pages is None or pages.dim() != 3 or pages.shape[2] != D or not pages.is_contiguous():
            raise KernelError(f"latent_write: pages must be contiguous (pages, page size, {D})")
        if weight is None or weight.dtype != torch.float32 or weight.numel() != rank \
                or not weight.is_contiguous():
            raise KernelError(f"latent_write: the norm's weight must be {rank} float32 values")
        _i32(slots, T, "latent_write slots")
        T = x.shape[0]
        if pages_t is not None and (tuple(pages_t.shape) != (pages.shape[0], rank, pages.shape[1])
                                    or pages_t.dtype != pages.dtype
                                    or not pages_t.is_contiguous()):
            raise KernelError("latent_write: the transposed pages must be contiguous "
                              "(pages, rank, page size) of the pages' dtype")
    ldq = ldo = 0
    dtype = pages.dtype if pages is not None else (q.dtype if q is not None else torch.float32)
    if rot_width:
        ldq, ldo = _rows2(q, "latent_write q"), _rows2(q_out, "latent_write q_out")
        if q.dtype != dtype or q_out.dtype != dtype or q_head < rot_width \
                or q.shape[1] < heads * q_head or q_out.shape[1] < heads * D:
            raise KernelError("latent_write: the queries' rows do not match the heads")
        if rot_dims:
            for t in (cos, sin):
                if t is None or t.dtype != torch.float32 or not t.is_contiguous() \
                        or t.shape[1] != rot_dims // 2:
                    raise KernelError("latent_write: the rotation needs float32 tables "
                                      "(positions, rot_dims / 2)")
    lib.call("rlis_latent_write", None if not write else x.data_ptr(), ldx,
             None if not write else weight.data_ptr(), float(eps), int(rank), int(rot_width),
             int(rot_dims), None if cos is None else cos.data_ptr(),
             None if sin is None else sin.data_ptr(), _i32(positions, T, "positions"),
             None if not write else slots.data_ptr(),
             None if pages is None else pages.data_ptr(),
             None if pages_t is None or not write else pages_t.data_ptr(),
             0 if pages is None else pages.shape[1], _DT[dtype], int(write),
             None if q is None else q.data_ptr(), ldq, int(q_head), int(q_head - rot_width),
             None if q_out is None else q_out.data_ptr(), ldo, D, int(heads), T, lib.stream_ptr())


# "matrix": bfloat16 attention over cached latents runs on the matrix cores where it applies;
# "vector": always the vector-unit kernel (tests hold the two against each other).
LATENT_ATTENTION = "matrix"
# Steps that make at most this many blocks of 16 (token, head) columns (upper bound: tokens and
# heads alone) let the four waves of a workgroup share a block and split its keys; larger steps
# give every wave a block of its own.  The two differ in the order of the last additions.
LATENT_SPLIT_MAX_BLOCKS = 1024
# Larger steps stage a chunk's keys and values once per workgroup of four column blocks
# (False: every wave loads its own).
LATENT_STAGED = True


def latent_mfma_ok(dtype: torch.dtype, rank: int, row: int, page_size: int = 16) -> bool:
    """Whether the matrix-core kernel takes latents of ``rank`` numbers in cached rows of
    ``row`` (it reads a second, transposed copy of the latents, which the mixer then keeps)."""
    return dtype == torch.bfloat16 and bool(
        lib.load().rlis_latent_attention_mfma_ok(int(rank), int(row), int(page_size)))


def latent_attention(q: torch.Tensor, pages: torch.Tensor, block_tables: torch.Tensor,
                     seq_of_token: torch.Tensor, positions: torch.Tensor, heads: int, rank: int,
                     scale: float, window: Optional[int] = None,
                     sink: Optional[torch.Tensor] = None,
                     pages_t: Optional[torch.Tensor] = None, cu: Optional[torch.Tensor] = None,
                     num_seqs: int = 0) -> torch.Tensor:
    """Softmax attention of ``q (T, heads * D)`` over cached rows ``pages (pages, page size,
    D)``: the score of a row is ``scale * (q_h . row)``, the output per head the weighted sum
    of the rows' first ``rank`` numbers, ``(T, heads * rank)``.  A query at position p sees rows
    at positions <= p and, under ``window`` w, > p - w.  ``sink (heads)`` float32: the
    softmax's denominator also holds ``exp(sink[h])``.  With ``pages_t`` (the latents once more
    as ``(pages, rank, page size)``), ``cu`` (cumulative token counts of the step's
    ``num_seqs`` sequences) and bfloat16 operands of sizes it takes, the matrix-core kernel
    runs; otherwise the vector-unit kernel (any sizes, both dtypes)."""
    ldq = _rows2(q, "latent_attention q")
    T = q.shape[0]
    if pages.dim() != 3 or not pages.is_contiguous() or pages.dtype != q.dtype:
        raise KernelError("latent_attention: pages must be contiguous (pages, page size, D) of "
                          "q's dtype")
    page_size, D = pages.shape[1], pages.shape[2]
    if q.shape[1] != heads * D or rank > D:
        raise KernelError(f"latent_attention: q has {q.shape[1]} columns, {heads} heads of {D}")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 \
            or not block_tables.is_contiguous():
        raise KernelError("latent_attention: block tables must be contiguous int32 (S, pages)")
    if sink is not None and (sink.dtype != torch.float32 or sink.numel() != heads
                             or not sink.is_contiguous()):
        raise KernelError(f"latent_attention: the sink must be {heads} float32 values")
    out = torch.empty((T, heads * rank), dtype=q.dtype, device=q.device)
    if pages_t is not None and cu is not None and num_seqs > 0 and LATENT_ATTENTION == "matrix" \
            and ldq % 8 == 0 and latent_mfma_ok(q.dtype, rank, D, page_size):
        if tuple(pages_t.shape) != (pages.shape[0], rank, page_size) \
                or pages_t.dtype != q.dtype or not pages_t.is_contiguous():
            raise KernelError("latent_attention: the transposed pages must be contiguous "
                              "(pages, rank, page size)")
        lib.call("rlis_latent_attention_mfma", q.data_ptr(), ldq, out.data_ptr(), heads * rank,
                 pages.data_ptr(), pages_t.data_ptr(), block_tables.data_ptr(),
                 block_tables.shape[1], _i32(cu, num_seqs + 1, "cu"),
                 _i32(positions, T, "positions"), T, int(num_seqs), heads, rank, D, page_size,
                 float(scale), int(window or 0), None if sink is None else sink.data_ptr(),
                 int(LATENT_SPLIT_MAX_BLOCKS), int(LATENT_STAGED), lib.stream_ptr())
        return out
    lib.call("rlis_latent_attention", q.data_ptr(), _DT[q.dtype], ldq, out.data_ptr(),
             heads * rank, pages.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
             _i32(seq_of_token, T, "seq_of_token"), _i32(positions, T, "positions"), T, heads,
             rank, D, page_size, float(scale), int(window or 0),
             None if sink is None else sink.data_ptr(), lib.stream_ptr())
    return out


def sigmoid_gate_(o: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """``o *= sigmoid(g)`` in place, element by element; both ``(T, N)`` with contiguous rows."""
    ldo, ldg = _rows2(o, "sigmoid_gate o"), _rows2(g, "sigmoid_gate g")
    if o.shape != g.shape or o.dtype != g.dtype:
        raise KernelError("sigmoid_gate: the gate must have the shape and dtype of o")
    lib.call("rlis_sigmoid_gate", o.data_ptr(), ldo, g.data_ptr(), ldg, _DT[o.dtype], o.shape[0],
             o.shape[1], lib.stream_ptr())
    return o
