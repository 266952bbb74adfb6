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


class Normed:
    """What a branch returns when its last projection has already added its output to the
    residual stream and computed the following norm: ``rows`` is that norm's output (a
    tensor, or whatever the kernel set hands the next product in its place)."""
    __slots__ = ("rows",)

    def __init__(self, rows):
        self.rows = rows


class PreNormBlock:
    chains = True       # forward takes ``nxt``, the block that runs after this one

    def __init__(self, spec: BlockSpec, weights, ops):
        self.spec, self.ops = spec, ops
        self.norm1 = build_part(spec.norm1, _sub_tensors(spec, "norm1", weights), ops)
        self.mixer = build_part(spec.mixer, _sub_tensors(spec, "mixer", weights), ops)
        self.norm2 = build_part(spec.norm2, _sub_tensors(spec, "norm2", weights), ops)
        self.ffn = build_part(spec.ffn, _sub_tensors(spec, "ffn", weights), ops)
        # a step through this layer can be captured into a HIP graph unless one of its parts
        # says otherwise (it reads the host's view of the batch, or syncs with the device)
        self.capturable = all(getattr(p, "capturable", True)
                              for p in (self.norm1, self.mixer, self.norm2, self.ffn))

    def reserve(self, n_positions):
        """Pass the cache's longest row on to the parts that keep something by position."""
        for part in (self.norm1, self.mixer, self.norm2, self.ffn):
            if hasattr(part, "reserve"):
                part.reserve(n_positions)

    def _branch(self, part, args, residual, norm, consumer):
        """Run a mixer or feed-forward. If the part ends with a projection that it lets the
        block supply (``takes_projection``), the norm after it can be left to the kernel set
        (``fusable``) and the part after that norm takes what the kernel set then returns in
        place of normed rows (``takes_norm_owed``), the part's last product adds to the
        residual stream and prepares the norm itself: one kernel instead of two."""
        ops = self.ops
        if (getattr(part, "takes_projection", False) and norm is not None and hasattr(norm, "fusable")
                and getattr(consumer, "takes_norm_owed", False) and hasattr(ops, "linear_add_norm")):
            gain, eps = norm.fusable()
            return part.forward(*args, project=lambda y, w: Normed(ops.linear_add_norm(y, w, residual, gain, eps)))
        return part.forward(*args)

    @staticmethod
    def _norm(norm, consumer, residual, delta):
        """The sum and the norm before a part. A part that feeds its input to one product of the
        kernel set and nowhere else (``takes_norm_owed``) leaves the layout of that input to the
        kernel set, if the norm can write it so (``free_layout``)."""
        if getattr(norm, "free_layout", False) and getattr(consumer, "takes_norm_owed", False):
            return norm.add_norm(residual, delta, by_tile=True)
        return norm.add_norm(residual, delta)

    def forward(self, residual, pending, ctx, slot, write=True, nxt=None):
        """residual: fp32 [N, hidden], updated in place. pending: the previous block's
        un-added output, None, or a ``Normed`` (already added, and normed by this block's
        first norm). ``nxt``: the block that runs next, if it is of this arrangement.
        Returns this block's feed-forward output, un-added or as a ``Normed``."""
        h = pending.rows if isinstance(pending, Normed) else self._norm(self.norm1, self.mixer, residual, pending)
        a = self._branch(self.mixer, (h, ctx, slot, write), residual, self.norm2, self.ffn)
        h = a.rows if isinstance(a, Normed) else self._norm(self.norm2, self.ffn, residual, a)
        return self._branch(self.ffn, (h, ctx), residual, getattr(nxt, "norm1", None), getattr(nxt, "mixer", None))


register_arrangement("prenorm", PreNormBlock)
