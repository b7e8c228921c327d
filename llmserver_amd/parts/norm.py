"""RMSNorm fused with the residual sum.

``y = s * rsqrt(mean(s^2) + eps) * w`` with ``s = resid + delta`` and everything in 32-bit inside
(utils/layers.py:131-138; fused form utils/fused_ops.py:23-26,
65-78).  ``s`` is rounded to the activation dtype once, when it is stored back as the new
residual stream (utils/fused_ops.py:73).
"""
from __future__ import annotations

from .base import VECTOR, Norm, ParamSpec


class RMSNorm(Norm):
    def __init__(self, width: int, eps: float):
        self.width = width
        self.eps = float(eps)
        self.weight = None  # float32 [width]

    def param_specs(self):
        return {"weight": ParamSpec((self.width,), VECTOR, "norm")}

    def assign(self, name, tensor):
        assert name == "weight"
        self.weight = tensor

    def add_norm(self, resid, delta, ctx, rows=None):
        n = resid.shape[0] if rows is None else rows.shape[0]
        out = ctx.empty((n, self.width))
        ctx.ops.add_rmsnorm(resid, delta, self.weight, self.eps, out, rows)
        return out

    def row_scale_form(self):
        return self.weight, self.eps
