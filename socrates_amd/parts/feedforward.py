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
        # One operand for gate and up: rows [gate | up].
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]],
                                   dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]

    def forward(self, x, ctx=None):
        gate_up = self.ops.linear(x, self.w_gate_up)
        # the block's next norm adds this output to the residual: partial sums are welcome
        return self.ops.linear(self.ops.swiglu(gate_up), self.w_down, allow_partial=True)


register_part(SwiGLUSpec, SwiGLU)
