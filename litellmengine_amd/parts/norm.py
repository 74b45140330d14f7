"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w; the weight multiplies directly,
no bias, no mean subtraction (src/layers/rms_norm.cu:81-93).  The residual add
that precedes a norm in the block is folded into the same kernel."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..weights.spec import INIT_NORM, INIT_NORMAL, TensorSpec
from .base import BuildContext, Norm, NormFold, ScaledSum


class RMSNorm(Norm):
    def __init__(self, name: str, size: int, eps: float, scalar: bool = False, one_plus: bool = False):
        """`scalar`: the checkpoint holds ONE gain for all coordinates (a tensor without
        dimensions); the kernels see it repeated `size` times.  `one_plus`: the stored weight
        lies around zero and the gain is 1 + weight (added in 32-bit, kept in 32-bit)."""
        self.one_plus = bool(one_plus)
        self.name = name
        self.size = size
        self.eps = float(eps)
        self.scalar = bool(scalar)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec(() if self.scalar else (self.size,), INIT_NORMAL if self.one_plus else INIT_NORM)}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        w = weights[self.name]  # bfloat16 or float32, as stored
        if self.one_plus:
            w = 1.0 + w.float()
        self.weight = (w.reshape(1).expand(self.size) if self.scalar else w).contiguous()

    def add_normed(self, hidden, y, extra=None, then=None) -> torch.Tensor:
        ops = self.ctx.ops
        if then is None:
            return ops.rmsnorm_add(hidden, y, self.weight, self.eps, self.ctx.dtype, extra)
        if isinstance(then, RMSNorm) and then.size == self.size:  # both norms in one launch
            return ops.rmsnorm_add_rmsnorm(hidden, y, self.weight, self.eps, then.weight, then.eps, self.ctx.dtype, extra)
        ops.rmsnorm_add(hidden, y, self.weight, self.eps, self.ctx.dtype, extra)
        return then.forward(hidden, None)

    def forward(self, hidden, delta, rows=None) -> torch.Tensor:
        if isinstance(delta, ScaledSum):  # the add, times its constant, and the norm in one launch
            return self.ctx.ops.scaled_add_rmsnorm(hidden, delta.a, delta.b, delta.mult, self.weight, self.eps,
                                                   self.ctx.dtype, rows)
        return self.ctx.ops.add_rmsnorm(hidden, delta, self.weight, self.eps, self.ctx.dtype, rows)

    def of_embedding(self, ids, table, step=None):
        if table.dtype != self.ctx.dtype or table.shape[1] != self.size:
            return None
        if step is not None and step.token_feedback is not None:
            return self.ctx.ops.embedding_rmsnorm(ids, table, self.weight, self.eps, step.token_feedback,
                                                  step.token_seq, step.seq_slots)
        return self.ctx.ops.embedding_rmsnorm(ids, table, self.weight, self.eps)

    def fold(self, hidden) -> Optional[NormFold]:
        if self.one_plus:
            return None
        if not self.ctx.ops.can_fold_norm(hidden.shape[0], self.size, self.ctx.dtype):
            return None
        return NormFold(hidden, self.weight, self.eps)
