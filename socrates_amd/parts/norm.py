"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w  (model/qwen/qwen_kv_cont.py:45-53).

eps sits inside the square root and the gain is the plain weight, as in the
reference. Statistics are taken in float32 whatever the compute dtype.
"""

from __future__ import annotations

from ..config.specs import RMSNormSpec
from .registry import TensorDecl, register_part


class RMSNorm:
    @staticmethod
    def tensors(spec: RMSNormSpec):
        return {"weight": TensorDecl((spec.dim,), "vector")}

    def __init__(self, spec: RMSNormSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.weight = tensors["weight"]

    free_layout = True      # add_norm takes ``by_tile``

    def add_norm(self, residual, delta, rows=None, by_tile=False):
        """residual (fp32, [N, dim]) += delta; return norm(residual) in the compute dtype.

        With ``rows`` (int32 indices) only those rows are summed and normed, into a
        new [len(rows), dim] tensor, and ``residual`` is left unchanged. ``by_tile``: the
        result goes to one product of the kernel set and nowhere else, so the kernel set may
        lay it out as that product reads it best.
        """
        if by_tile and getattr(self.ops, "rows_by_tile", None):
            return self.ops.add_rmsnorm(residual, delta, self.weight, self.spec.eps, rows, by_tile=True)
        return self.ops.add_rmsnorm(residual, delta, self.weight, self.spec.eps, rows)

    def fusable(self):
        """(gain, eps): all a kernel set needs to compute this norm inside the products
        around it (``HipKernels.linear_add_norm``)."""
        return self.weight, self.spec.eps

    def __call__(self, x):
        """Plain norm over the last dimension of ``x`` (any leading shape)."""
        return self.ops.rmsnorm(x, self.weight, self.spec.eps)


register_part(RMSNormSpec, RMSNorm)
