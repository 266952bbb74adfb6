"""Rotate-half rotary position encoding (model/qwen/qwen_kv_cont.py:56-77).

inv_freq[j] = 1 / theta ** (2j / rotary_dim) in float32, angle = position *
inv_freq[j], and y[j] = x[j] cos - x[j+h] sin, y[j+h] = x[j+h] cos + x[j] sin with
h = rotary_dim / 2. Angles, sines and cosines are float32; the product is rounded
once to the compute dtype.

The constants of a rotation (inv_freq, and the table of cosines and sines by position
that the fused decode kernel looks up) belong to (kernel set, theta, rotary_dim), not to
a layer: all layers with the same rotation (theta, rotary size, stretch factor) share one
``PositionTable``. The reference
keeps what its captured steps read in module buffers at fixed addresses
(model/qwen/qwen_kv_cont.py:97-127); here the table is sized once, for the cache's
longest row, before any step runs (``reserve``), and a kernel set is told when it
moves after all (``invalidate_graphs``), so that no captured step reads a freed table.
"""

from __future__ import annotations

import weakref

import torch

from ..config.specs import RopeSpec
from .registry import register_part

_SHARED = weakref.WeakKeyDictionary()        # kernel set -> {(theta, rotary_dim): PositionTable}


class PositionTable:
    """inv_freq [rotary_dim / 2] and, once reserved, cosines and sines of positions
    0 .. n - 1, float32 [n, 2, rotary_dim / 2], made by the kernel set's own arithmetic."""

    def __init__(self, theta, rotary_dim, ops, factor=1.0):
        self.ops = ops
        # The reference's own expression (qwen_kv_cont.py:60), evaluated in float32.
        inv_freq = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2).float() / rotary_dim))
        if factor != 1.0:
            inv_freq = inv_freq / factor
        self.inv_freq = inv_freq.to(ops.device)
        self.rows = None

    def reserve(self, n_positions):
        """Make the table hold at least ``n_positions`` positions. A table that has to be
        made anew (it is never grown in place: a captured step holds its address) tells the
        kernel set, which drops what was captured with the old one."""
        have = 0 if self.rows is None else self.rows.shape[0]
        if have >= n_positions:
            return self.rows
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(f"the rotation's table holds {have} positions and a step that is being captured "
                               f"reaches {n_positions}: reserve the positions before capturing")
        rows = torch.empty((n_positions, 2, self.inv_freq.numel()), dtype=torch.float32, device=self.ops.device)
        self.ops.rope_table(self.inv_freq, 0, n_positions, rows)
        if have and hasattr(self.ops, "invalidate_graphs"):
            self.ops.invalidate_graphs()
        self.rows = rows
        return rows


def shared_table(ops, theta, rotary_dim, factor=1.0) -> PositionTable:
    per_ops = _SHARED.setdefault(ops, {})
    key = (float(theta), int(rotary_dim), float(factor))
    if key not in per_ops:
        per_ops[key] = PositionTable(theta, rotary_dim, ops, factor)
    return per_ops[key]


class Rope:
    @staticmethod
    def tensors(spec: RopeSpec):
        return {}

    def __init__(self, spec: RopeSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        self.shared = shared_table(ops, spec.theta, spec.rotary_dim, spec.factor)
        self.inv_freq = self.shared.inv_freq
        # kernels look cosines and sines up only for a rotation over the whole head
        self._tabled = hasattr(ops, "rope_table") and spec.rotary_dim == spec.head_dim

    def rotary(self):
        """Constants for the fused QK-norm + rotation + cache-write kernel."""
        return self.inv_freq, self.spec.rotary_dim

    def reserve(self, n_positions):
        """Called once with the cache's longest row before the first step: the table is
        then at its final address."""
        if self._tabled:
            self.shared.reserve(n_positions)

    def table(self, n_positions):
        """Cosines and sines of positions 0 .. n_positions - 1, float32 [>= n_positions, 2,
        rotary_dim / 2], for kernels that look them up instead of computing them; None if
        the kernel set has no such table or the rotation covers part of the head only."""
        if not self._tabled:
            return None
        return self.shared.reserve(n_positions)

    def apply(self, q, k, positions):
        """Rotate q [N, Hq, D] and k [N, Hkv, D] in place at ``positions`` [N]."""
        self.ops.rope(q, positions, self.inv_freq, self.spec.rotary_dim)
        self.ops.rope(k, positions, self.inv_freq, self.spec.rotary_dim)


register_part(RopeSpec, Rope)
