"""Rotate-half rotary position encoding (model/qwen/qwen_kv_cont.py:56-77).

inv_freq[j] = 1 / theta ** (2j / rotary_dim) in float32, angle = position *
inv_freq[j], and y[j] = x[j] cos - x[j+h] sin, y[j+h] = x[j+h] cos + x[j] sin with
h = rotary_dim / 2. Angles, sines and cosines are float32; the product is rounded
once to the compute dtype.
"""

from __future__ import annotations

import torch

from ..config.specs import RopeSpec
from .registry import register_part


class Rope:
    @staticmethod
    def tensors(spec: RopeSpec):
        return {}

    def __init__(self, spec: RopeSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        r = spec.rotary_dim
        # The reference's own expression (qwen_kv_cont.py:60), evaluated in float32.
        inv_freq = 1.0 / (spec.theta ** (torch.arange(0, r, 2).float() / r))
        self.inv_freq = inv_freq.to(ops.device)
        self._table = None

    def rotary(self):
        """Constants for the fused QK-norm + rotation + cache-write kernel."""
        return self.inv_freq, self.spec.rotary_dim

    def table(self, n_positions):
        """Cosines and sines of positions 0 .. n_positions - 1, float32 [>= n_positions, 2,
        rotary_dim / 2], for kernels that look them up instead of computing them; None if
        the kernel set has no such table or the rotation covers part of the head only. Kept,
        and grown by doubling when a step reaches further."""
        if not hasattr(self.ops, "rope_table") or self.spec.rotary_dim != self.spec.head_dim:
            return None
        have = 0 if self._table is None else self._table.shape[0]
        if have < n_positions:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("the rotation's table has to grow inside a graph capture: run the step "
                                   "eagerly once before capturing it")
            rows = max(n_positions, 2 * have, 1024)
            grown = torch.empty((rows, 2, self.inv_freq.numel()), dtype=torch.float32, device=self.ops.device)
            if have:
                grown[:have] = self._table
            self.ops.rope_table(self.inv_freq, have, rows - have, grown[have:])
            self._table = grown
        return self._table

    def apply(self, q, k, positions):
        """Rotate q [N, Hq, D] and k [N, Hkv, D] in place at ``positions`` [N]."""
        self.ops.rope(q, positions, self.inv_freq, self.spec.rotary_dim)
        self.ops.rope(k, positions, self.inv_freq, self.spec.rotary_dim)


register_part(RopeSpec, Rope)
