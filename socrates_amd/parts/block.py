"""Arrangements of a mixer, a feed-forward and their norms into one layer.

"prenorm" (model/qwen/qwen_kv_paged.py:186-189): h = x + mixer(norm1(x));
y = h + ffn(norm2(h)). The residual stream is a float32 tensor updated in place;
each sum is fused into the norm that follows it, so a block returns its last
branch output un-added ("pending") and the next norm adds it.
"""

from __future__ import annotations

from ..config.specs import BlockSpec
from .registry import build_part, tensors_of

_ARRANGEMENTS = {}


def register_arrangement(name: str, cls) -> None:
    _ARRANGEMENTS[name] = cls


def block_tensors(spec: BlockSpec):
    """{full tensor name: TensorDecl} of one layer."""
    out = {}
    for role in ("norm1", "mixer", "norm2", "ffn"):
        sub = getattr(spec, role)
        for local, decl in tensors_of(sub).items():
            out[f"{spec.name_of(role)}.{local}"] = decl
    return out


def build_block(spec: BlockSpec, weights, ops):
    try:
        cls = _ARRANGEMENTS[spec.arrangement]
    except KeyError:
        raise KeyError(f"unknown block arrangement {spec.arrangement!r}; "
                       f"known: {sorted(_ARRANGEMENTS)}") from None
    return cls(spec, weights, ops)


def _sub_tensors(spec: BlockSpec, role: str, weights):
    sub = getattr(spec, role)
    prefix = spec.name_of(role) + "."
    return {local: weights[prefix + local] for local in tensors_of(sub)}


class PreNormBlock:
    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec = spec
        self.norm1 = build_part(spec.norm1, _sub_tensors(spec, "norm1", weights), ops)
        self.mixer = build_part(spec.mixer, _sub_tensors(spec, "mixer", weights), ops)
        self.norm2 = build_part(spec.norm2, _sub_tensors(spec, "norm2", weights), ops)
        self.ffn = build_part(spec.ffn, _sub_tensors(spec, "ffn", weights), ops)
        # a step through this layer can be captured into a HIP graph unless one of its parts
        # says otherwise (it reads the host's view of the batch, or syncs with the device)
        self.capturable = all(getattr(p, "capturable", True)
                              for p in (self.norm1, self.mixer, self.norm2, self.ffn))

    def forward(self, residual, pending, ctx, slot, write=True):
        """residual: fp32 [N, hidden], updated in place. pending: the previous block's
        un-added output or None. Returns this block's un-added feed-forward output."""
        h = self.norm1.add_norm(residual, pending)
        a = self.mixer.forward(h, ctx, slot, write)
        h = self.norm2.add_norm(residual, a)
        return self.ffn.forward(h, ctx)


register_arrangement("prenorm", PreNormBlock)
