"""A projection y = a W^T through the hand-written matrix kernels, for any meeting of
precisions: bf16 weights take bf16 activations (matrix cores, float accumulation); a
weight stored in 32-bit stays so and is multiplied in 32-bit, with the activations
widened for it.  reference: op_linear_proj, kernels/megakernel_ops.hip:166-276 (bf16
weight, f32 activation, f32 accumulate, no bias)."""
from __future__ import annotations

import os

import torch

from .. import kernels as K
from .base import NormedInput, ProductRuns, ResidualSink


def linear(a, w: torch.Tensor, out, ws, accumulate: bool = False) -> None:
    """out (+)= a @ w^T.  `accumulate` needs a float32 `out`.  `w` is [N, K] or what
    `stream_layout` made of it.

    `a` may be a `NormedInput` (the product is then taken of the normed rows, from what the
    product before prepared where it did) and `out` a `ResidualSink` (the product is added
    to its rows and, where the next norm can, prepares that norm in the same kernel)."""
    if isinstance(a, NormedInput):
        if a.prepared is not None and not accumulate and not isinstance(out, ResidualSink) \
                and a.norm.product_of_prepared(a.prepared, w, out):
            return
        a = a.tensor()
    if isinstance(out, ResidualSink):
        sink, out = out, out.x
        if accumulate and sink.next_norm is not None:
            sink.prepared = sink.next_norm.prepare_in_product(a, w, out, ws)
            if sink.prepared is not None:
                return
    if a.dtype == w.dtype:
        if a.dtype == torch.float32 or out.dtype == torch.float32 or not accumulate:
            if a.dtype == torch.float32 and out.dtype != torch.float32:
                tmp = ws.get("linear_out32", out.shape, torch.float32)
                K.gemm(a, w, tmp)
                K.convert(tmp, out)
                return
            scratch = None
            if a.dtype == torch.bfloat16 and 16 < a.shape[0] <= 1024:     # products that may be split along k
                scratch = ws.get("gemm_scratch", (K.GEMM_SCRATCH_FLOATS,), torch.float32)
            K.gemm(a, w, out, accumulate, scratch=scratch)
            return
    if w.dtype == torch.float32 and a.dtype == torch.bfloat16:
        a32 = ws.get("linear_in32", a.shape, torch.float32)
        if a.is_contiguous():
            K.convert(a, a32)
        else:
            a32.copy_(a)
        linear(a32, w, out, ws, accumulate)
        return
    if w.dtype == torch.bfloat16 and a.dtype == torch.float32:
        a16 = ws.get("linear_in16", a.shape, torch.bfloat16)
        K.convert(a.contiguous(), a16)
        linear(a16, w, out, ws, accumulate)
        return
    raise TypeError(f"linear: activations {a.dtype}, weight {w.dtype}")


def linear_runs(a, w: torch.Tensor, n_out: int, ws):
    """a @ w^T (bfloat16, `n_out` columns) left as the float sums of its runs along k
    (`ProductRuns`) where the product of these sizes is cut into runs anyway (17 to 64 rows over
    few weight rows), for a caller whose next kernel adds the runs itself; None with nothing
    done otherwise, and `linear` is then the way."""
    if isinstance(a, NormedInput):
        if a.prepared is not None:
            return a.norm.runs_of_prepared(a.prepared, w, n_out, ws)
        if not 16 < a.x.shape[0] <= 64 or w.dtype != torch.bfloat16 or a.dtype != torch.bfloat16:
            return None
        a = a.tensor()
    if not (a.dtype == w.dtype == torch.bfloat16 and 16 < a.shape[0] <= 64):
        return None
    scratch = ws.get("gemm_scratch", (K.GEMM_SCRATCH_FLOATS,), torch.float32)
    runs = K.gemm_wide_partial(a, w, n_out, scratch)
    return ProductRuns(scratch, runs, a.shape[0], n_out) if runs else None


BLOCK_FROM_ROWS = 8192


def blocks_at_load(rows: int, k: int, dtype: torch.dtype, rt) -> bool:
    """Whether `stream_layout` turns a [rows, k] matrix of this dtype into blocks."""
    want = os.environ.get("BRAIDINFER_WEIGHT_LAYOUT", "")
    return (rt.is_bf16 and dtype == torch.bfloat16 and rt.device.type == "cuda" and k % 128 == 0 and k >= 1024
            and want != "rows" and (rows >= BLOCK_FROM_ROWS or want == "blocks"))


def stream_layout(w: torch.Tensor, rt) -> torch.Tensor:
    """The weight as the part keeps it and as the bf16 products read it fastest.  Parts call
    it once at load on every matrix that only `linear` and the fused products read.  Wide
    matrices (from 8,192 rows: gate/up, the head) become blocks of 16 rows x 128 k
    (`kernels.block_weight`) where the runtime allows it: measured on a 28,672 x 4,096 matrix,
    products of 17 to 128 rows gain 10 to 15 %, others nothing, while matrices of 4,096 to 6,144
    rows lose up to 4 % in blocks and keep their rows.  BRAIDINFER_WEIGHT_LAYOUT=rows or =blocks
    in the environment forces one (measurements and tests).  The result lies in the
    runtime's arena when it has one."""
    if w.dim() == 2 and blocks_at_load(w.shape[0], w.shape[1], w.dtype, rt) and K.weight_blockable(w):
        return K.block_weight(w, rt.empty)
    return rt.own(w)


def fused_layout(mats, rt, interleave: bool = False) -> torch.Tensor:
    """`stream_layout` of the matrices stacked along the output dimension (`fuse_rows`), or
    of gate and up rows interleaved for the SwiGLU epilogue (`kernels.interleave_gate_up`):
    what is kept is written once, into the runtime's memory; a stack that becomes blocks is
    put together in a transient tensor first."""
    rows = sum(m.shape[0] for m in mats)
    dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
    transient = blocks_at_load(rows, mats[0].shape[1], dt, rt)
    alloc = None if transient else rt.empty
    w = K.interleave_gate_up(mats[0], mats[1], alloc) if interleave else fuse_rows(mats, None if transient else rt)
    return stream_layout(w, rt)


def fuse_rows(mats, rt=None):
    """Stack weight matrices along the output dimension so that one product serves all
    (the reference keeps q/k/v and gate/up separate: three and two launches,
    megakernel/compile_attention.rs:82-85).  Mixed precisions widen to float32.  With a
    runtime the result is memory of its own (`rt.empty`), else a new tensor."""
    dt = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
    rows = sum(m.shape[0] for m in mats)
    shape = (rows,) + tuple(mats[0].shape[1:])
    out = rt.empty(shape, dt) if rt is not None else torch.empty(shape, dtype=dt, device=mats[0].device)
    r = 0
    for m in mats:
        out[r:r + m.shape[0]].copy_(m)
        r += m.shape[0]
    return out
