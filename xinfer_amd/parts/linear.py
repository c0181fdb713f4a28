"""y = x @ W^T, the matrix product shared by the parts.

The reference routes every dense projection through candle's matmul, i.e. the vendor
BLAS (/root/reference/src/models/layers/linear.rs:76-124).  Here:
  float32  : the hand-written fixed-order kernel (`kernels.gemm_tn`) - true 32-bit, and
             an output element does not depend on the batch it was computed in;
  bfloat16 : the hand-written kernels for few rows (decode), the vendor library
             (hipBLASLt through torch) for many rows, as the reference uses a library;
             narrow outputs at 129 to 1,024 rows in the hand-written many-row tiled kernel over
             slices of K where the caller takes partial sums (`kernels.tile_split_plan`).
A weight that the checkpoint stores in 32 bits stays in 32 bits; activations are then
widened for this product.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import kernels
from .base import Folded, NormSink


class Linear:
    def __init__(self, weight: torch.Tensor):
        if weight.dim() != 2:
            raise ValueError("a linear weight must be [out, in]")
        self.weight = weight.contiguous()
        self.out_features, self.in_features = weight.shape

    def __call__(self, x, out_dtype: Optional[torch.dtype] = None, skinny_rows: Optional[int] = None,
                 allow_split: bool = False, sink: Optional[NormSink] = None, gated: bool = False):
        """`x`: rows, or a `Folded` (the norm before this product is half done: this product
        finishes it).  `sink`: the norm after this product may be folded: if the sizes allow
        (bfloat16, up to `kernels.FOLD_ROWS` rows) the result is added into the stream here and a
        `Folded` comes back instead of rows.  `gated`: the weight is [gate; up] and the result
        silu(gate) * up, where the fused kernel takes the sizes (else None: the caller does it
        in two steps).
        `allow_split`: the caller hands the result to a norm, which also takes a stack
        [P, T, out] of float32 partial sums; few rows and a narrow output then come back so.
        A workgroup of the split product takes more rows of the weight per read of x, which
        on an MI355X pays from about 16 rows on (o and down projections at Qwen3 sizes)."""
        if skinny_rows is None:
            skinny_rows = kernels.SKINNY_ROWS
        w = self.weight
        if isinstance(x, Folded):
            if w.dtype == torch.bfloat16 and x.xg.shape[1] % 8 == 0 and (not gated or out_dtype in (None, torch.bfloat16)):
                if gated and kernels.gated_uses_mid(x.xg.shape[0], w):
                    return kernels.linear_mid_gated(x.xg, w, x.ss, x.norm.eps)
                if not gated and kernels.thin_ahead(x.xg.shape[0], w):
                    return kernels.linear_thin_fold_in(x.xg, x.ss, x.norm.eps, w, out_dtype or torch.bfloat16)
                return kernels.linear_fold_in(x.xg, x.ss, x.norm.eps, w, out_dtype or torch.bfloat16, gated=gated)
            x = x.rows(torch.bfloat16 if w.dtype == torch.bfloat16 else torch.float32)
        if gated:
            if x.dtype == torch.bfloat16 and x.dim() == 2 and kernels.gated_uses_mid(x.shape[0], w):
                return kernels.linear_mid_gated(x, w)                 # gate, up and silu*mul in one pass
            if (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
                    and 0 < x.shape[0] <= kernels.SKINNY_GATED_ROWS and x.shape[1] % 8 == 0):
                return kernels.linear_skinny(x, w, gated=True)        # the same with the streaming kernel
            return None
        if (sink is not None and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
                and 0 < x.shape[0] <= kernels.FOLD_ROWS and x.shape[1] % 8 == 0 and w.shape[0] % 8 == 0
                and sink.norm.foldable and sink.norm.weight.shape[0] == w.shape[0]
                and sink.resid.dtype == torch.float32 and sink.resid.is_contiguous()
                and kernels.linear_fold_parts(x.shape[0], w.shape[0], w.shape[1]) <= kernels.FOLD_PARTS):
            fold_out = kernels.linear_thin_fold_out if kernels.thin_ahead(x.shape[0], w) else kernels.linear_fold_out
            xg, ss = fold_out(x, w, sink.resid, sink.norm.weight)
            return Folded(xg, ss, sink.norm)
        out_dtype = out_dtype or x.dtype
        if w.dtype == torch.float32:
            xf = x if x.dtype == torch.float32 else x.float()
            y = kernels.gemm_tn(xf, w, out_dtype=torch.float32)
            return y if out_dtype == torch.float32 else y.to(out_dtype)
        if x.dtype != w.dtype:
            raise kernels.KernelError(f"linear: activations are {x.dtype} but the weight is {w.dtype}")
        return kernels.linear_bf16(x, w, out_dtype, skinny_rows, allow_split)
