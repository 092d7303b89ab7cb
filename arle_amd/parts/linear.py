"""y = x . W^T for a weight stored [out, in], the one projection every part uses.

Which kernel runs depends only on the types of the operands:

* float32 x, float32 W  -> the fixed-order float32 kernel (the true 32-bit path);
* bfloat16 x, bfloat16 W -> the hand-written MFMA kernel for few rows (decode), the
  vendor library (hipBLASLt through torch) for many rows, as the reference uses
  cuBLAS for its projections (infer/src/ops/linear.rs:921-959);
* bfloat16 x, float32 W (a tensor that the checkpoint stores in 32 bits stays so):
  x is widened and the float32 kernel runs.

The few-rows kernel may split K over workgroups and leave a stack of float32 partial products
[S, T, out] behind.  A caller whose consumer can add such a stack in order (the residual add fused
into RMSNorm, the q/k/v preparation) says `partials_ok=True` and passes it on; otherwise the stack
is added here.

With `tiles=True` a bfloat16 weight is held a second time as operand tiles (ops.pack_weight_tiles): the
few-rows kernels then read one contiguous kilobyte a wave and k step instead of sixteen pieces a row apart,
which is worth a fifth of their time on MI355X.  The library needs the rows, so both copies stay.
"""
from __future__ import annotations

import torch

from ..kernels import ops


class Linear:
    def __init__(self, weight: torch.Tensor, tiles: bool = False, packed: torch.Tensor | None = None):
        """packed: operand tiles that exist already (of a matrix this weight is the first rows of)."""
        if weight.dim() != 2 or not weight.is_contiguous():
            raise ValueError("a projection weight must be a contiguous [out, in] matrix")
        self.weight = weight
        self.out_features, self.in_features = weight.shape
        self.tiles = packed
        if packed is None and tiles and weight.dtype == torch.bfloat16 and weight.is_cuda and self.in_features % 8 == 0:
            self.tiles = ops.pack_weight_tiles(weight)

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype | None = None, partials_ok: bool = False) -> torch.Tensor:
        """x [T, in] -> [T, out] in `out_dtype` (default: the type of x); with `partials_ok` possibly a
        float32 stack [S, T, out] whose sum over S, in order, is the product."""
        out_dtype = out_dtype or x.dtype
        w = self.weight
        if x.shape[0] == 0:
            return torch.empty((0, self.out_features), dtype=out_dtype, device=x.device)
        if w.dtype == torch.float32:
            y = ops.gemm_f32(x if x.dtype == torch.float32 else x.float(), w)
            return y if out_dtype == torch.float32 else y.to(out_dtype)
        if x.dtype != torch.bfloat16:
            raise ops.ShapeError(f"a bfloat16 weight needs bfloat16 activations, got {x.dtype}")
        return ops.gemm_bf16(x, w, out_dtype, partials_ok=partials_ok, tiles=self.tiles)
