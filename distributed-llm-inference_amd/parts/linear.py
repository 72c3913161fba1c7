"""``y = x W^T + b`` for both paths.

On the 32-bit path the product is the engine's own IEEE single-precision kernel. On the bfloat16
path it is the vendor library's matrix product (the reference's engine uses a library product
there as well: ``F.linear``, src/dli/model/llama.py:72-74,95,190,305), bfloat16 operands with
32-bit accumulation and the bias added inside; the library is called directly, with its choice of
kernel cached per shape, because a framework's dispatch costs more host time than the product
takes on the GPU when a step has a few hundred tokens.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import DecodeStream, Norm, Runtime


def linear(rt: Runtime, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [n, k] @ weight[m, k].T (+ bias [m]) -> [n, m]`` in the runtime's activation type."""
    n, m = x.shape[0], weight.shape[0]
    if out is None:
        out = rt.empty(n, m)
    if n == 0:
        return out
    if rt.dtype == torch.float32:
        ops.gemm_f32(x, weight, out, bias=bias)
        return out
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or x.shape[1] != weight.shape[1]:
        raise ops.KernelArgumentError("linear: operands must be bfloat16 [n, k] and [m, k]")
    if not ops.gemm_bf16(x, weight, out, bias):
        # a shape for which the direct call finds no kernel: the same library through torch
        torch.mm(x, weight.t(), out=out)
        if bias is not None:
            ops.add(out, None, out, bias=bias)
    return out


def decode_copy(rt: Runtime, weight: Optional[torch.Tensor], epilogue: int) -> Optional[torch.Tensor]:
    """The matrix once more in the tile order of the decode product (``ops.tile_weights``), or
    ``None`` where that would not be used: another type, sizes that do not tile, a product that
    neither the few-row tile kernel nor the kernel for 17 to 64 rows reads in that order, or a
    runtime that does not want it."""
    if (weight is None or not rt.is_bf16 or not rt.decode_weight_copy or weight.dtype != torch.bfloat16
            or weight.dim() != 2 or not weight.is_cuda):
        return None
    if not (ops.tiled_weights_help(weight.shape[0], weight.shape[1], epilogue, weight.device)
            or ops.mid_tiles_help(weight.shape[0], weight.shape[1], epilogue)):
        return None
    # (rows that are no whole blocks of 128: zero-filled to whole blocks, for the 17-to-64-row kernel alone)
    return ops.tile_weights(weight, whole_blocks=False)


# From this many rows on, the kernel that makes the residual sum also applies the norm that follows
# (one workgroup per row), so that the 256 workgroups of the next product need not each normalise
# every row again: 2% of a decode step at 48 rows and 1% at 64 at the 1B sizes; with 17 to 32 rows
# normalising inside the product is cheaper than a finishing kernel of so few workgroups (steps
# 0.5 to 1% slower), so below it the sums of squares are handed on as they are.
NORM_WITH_THE_SUM_FROM_ROWS = 33


def finish_residual(rt: Runtime, stream: DecodeStream, partial: torch.Tensor, bias: Optional[torch.Tensor],
                    following: Optional[Norm]) -> None:
    """The residual sum of a product that left partial sums, and with it the norm that follows
    where that is known, the rows are many enough for it to pay and narrow enough for one
    workgroup each."""
    fused = following.fused_params() if following is not None and hasattr(following, "fused_params") else None
    rows, width = stream.x.shape
    if (fused is not None and rows >= NORM_WITH_THE_SUM_FROM_ROWS and width <= ops.MID_NORMED_WIDTH
            and fused[0].shape[0] == width):
        normed = rt.empty(rows, width)
        ssq = ops.mid_finish_residual(partial, stream.x, bias, norm_w=fused[0], eps=fused[1], normed_out=normed)
        stream.wrote(ssq, normed, following)
    else:
        stream.wrote(ops.mid_finish_residual(partial, stream.x, bias))


class RoundedStream:
    """The rounded copy of a 32-bit residual stream that the kernel which last wrote the stream
    left beside it (the embedding, a norm that adds into the stream): whoever reads the stream as
    a product's operand next takes it instead of rounding the stream once more. It is kept on the
    step's context under the stream's address and dropped by whoever changes the stream."""

    KEY = "rounded stream"

    @staticmethod
    def offer(ctx, x: torch.Tensor, rounded: Optional[torch.Tensor]) -> None:
        if ctx is not None and hasattr(ctx, "_memo"):
            if rounded is None:
                ctx._memo.pop(RoundedStream.KEY, None)
            else:
                ctx._memo[RoundedStream.KEY] = (x.data_ptr(), tuple(x.shape), rounded)

    @staticmethod
    def take(ctx, x: torch.Tensor) -> Optional[torch.Tensor]:
        hit = getattr(ctx, "_memo", {}).get(RoundedStream.KEY) if ctx is not None else None
        return hit[2] if hit is not None and hit[:2] == (x.data_ptr(), tuple(x.shape)) else None


def as_operand(rt: Runtime, x: torch.Tensor, ctx=None) -> torch.Tensor:
    """``x`` in the type that the runtime's products read: a 32-bit residual stream is rounded to
    bfloat16 when serving (or its rounded copy is taken from ``ctx`` where its last writer left
    one) and used as it is on the 32-bit path."""
    if x.dtype == rt.dtype:
        return x
    if x.dtype != torch.float32:
        raise ops.KernelArgumentError(f"an operand of type {x.dtype} in a runtime of {rt.dtype}")
    ready = RoundedStream.take(ctx, x)
    if ready is not None:
        return ready
    out = rt.empty(*x.shape)
    ops.cast_from_f32(x, out)
    return out


F32_FEW_ROWS = 16  # up to here the few-row product streams the weights faster than the library does


def linear_f32(rt: Runtime, x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [n, k] @ weight[m, k].T -> float32 [n, m]``: the 32-bit sums of the product as they are,
    for what is computed in 32-bit after a projection (recurrences, norms, gates). ``out`` may be a
    view of some columns of a wider float32 matrix."""
    n, m = x.shape[0], weight.shape[0]
    if out is None:
        out = torch.empty(n, m, device=rt.device, dtype=torch.float32)
    if n == 0:
        return out
    if rt.dtype == torch.float32:
        ops.gemm_f32(x, weight, out)
        return out
    k = x.shape[1]
    if (n <= F32_FEW_ROWS and ops.skinny_gemm_supports(n, k, x.dtype) and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and out.data_ptr() % 16 == 0 and weight.is_contiguous()):
        ops.skinny_gemm(x, weight, epilogue=ops.SKINNY_F32, out=out)
        return out
    if not ops.gemm_bf16(x, weight, out):
        # a shape for which the direct call finds no kernel: the same library through torch
        # (bfloat16 result, widened)
        tmp = torch.mm(x, weight.t())
        wide = torch.empty(n, m, device=rt.device, dtype=torch.float32)
        ops.to_float(tmp, wide)
        out.copy_(wide)
    return out


def stack_rows(matrices, multiple: int = 16) -> torch.Tensor:
    """The matrices one below the other, filled up with zero rows to a multiple of ``multiple`` rows
    (a product kernel's tiles then need no edge case)."""
    stacked = torch.cat(list(matrices), dim=0)
    pad = -stacked.shape[0] % multiple
    if pad:
        stacked = torch.cat([stacked, stacked.new_zeros(pad, stacked.shape[1])], dim=0)
    return stacked.contiguous()
