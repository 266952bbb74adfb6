"""SwiGLU feed-forward: y = Wd((Wu x) * silu(Wg x)), no bias
(model/qwen/qwen_kv_cont.py:250-266). silu(z) = z * sigmoid(z), on the gate."""

from __future__ import annotations

import torch

from ..config.specs import SwiGLUSpec
from .registry import TensorDecl, register_part


class SwiGLU:
    @staticmethod
    def tensors(spec: SwiGLUSpec):
        return {"gate_proj.weight": TensorDecl((spec.intermediate, spec.hidden)),
                "up_proj.weight": TensorDecl((spec.intermediate, spec.hidden)),
                "down_proj.weight": TensorDecl((spec.hidden, spec.intermediate))}

    def __init__(self, spec: SwiGLUSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        # One operand for gate and up. Where the width allows, their rows alternate in blocks
        # of 16 (16 gate rows, the 16 up rows of the same columns, ...): a workgroup of the
        # decode product then holds both and applies the activation itself.
        gate, up = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        ff = spec.intermediate
        self.interleave = 16 if ff % 16 == 0 else 0
        if self.interleave:
            self.w_gate_up = torch.stack([gate.view(ff // 16, 16, -1), up.view(ff // 16, 16, -1)],
                                         dim=1).reshape(2 * ff, -1).contiguous()
        else:
            self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]
        # (the activation goes to a product and nowhere else: the kernel set may lay it out as it likes)
        self._free_layout = {"by_tile": True} if getattr(ops, "rows_by_tile", None) is not None else {}

    takes_projection = True     # the block may supply the last product
    takes_norm_owed = True      # x goes to one product only

    def forward(self, x, ctx=None, project=None):
        act = self.ops.linear_swiglu(x, self.w_gate_up, self.interleave, **self._free_layout)
        if project is not None:
            return project(act, self.w_down)
        # the block's next norm adds this output to the residual: partial sums are welcome
        return self.ops.linear(act, self.w_down, allow_partial=True)


register_part(SwiGLUSpec, SwiGLU)
