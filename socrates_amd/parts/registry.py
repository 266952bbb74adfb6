"""Registry from a spec type to the class that implements it.

A part is built from its spec (sizes and constants), its tensors (by local
name) and the kernel set. It never learns which model it is in. A new mixer,
feed-forward, norm or position encoding is added by defining a frozen spec
dataclass and an implementation class and calling ``register_part``; no file
of the framework has to change.

Interfaces (duck-typed):

  every part   ``tensors(spec) -> {local_name: TensorDecl}`` (staticmethod)
               ``__init__(spec, tensors, ops)``
  norm         ``add_norm(residual, delta, rows=None) -> normed``: adds ``delta`` (nothing,
               a [N, d] tensor, or float32 partial sums [S, N, d]) into the fp32
               ``residual`` in place and returns the normed activations in the compute
               dtype; with ``rows`` it works on those rows only and leaves ``residual``
               alone
  position     ``rotary() -> (inv_freq, rotary_dim) | None`` for the fused kernel, and
               ``apply(q, k, positions)`` in place on [N, H, D] tensors
  mixer        ``cache_need(spec) -> PagedKV | RowState | None`` (staticmethod)
               ``forward(x, ctx, slot, write) -> y`` with x, y [N, hidden]
  feed-forward ``forward(x, ctx) -> y``

A part whose ``forward`` reads ``ctx.host`` (the host's copy of the step's rows, positions
and sequence starts), or waits for the device, sets ``capturable = False`` (class or
instance attribute): a model with such a part never has its decode steps captured into HIP
graphs, whatever the engine's ``compile`` says. Parts without the attribute are taken to
be capturable: everything they do is device work on the current stream whose launch
shape depends on the step only through ``ctx.n_tokens`` and ``ctx.max_ctx_len``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

_PARTS = {}


@dataclass(frozen=True)
class TensorDecl:
    """Shape of one stored tensor and how it is kept in memory.

    kind "matrix": operand of a matrix product, kept in the compute dtype (a tensor
    stored in 32-bit floats stays 32-bit); "vector": gains and other small
    parameters, kept in float32 (lossless from bfloat16); "int": kept as int32.
    """
    shape: Tuple[int, ...]
    kind: str = "matrix"


@dataclass(frozen=True)
class PagedKV:
    """A mixer that keeps keys and values of every position (or a window of them) in pages."""
    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class RowState:
    """A mixer that keeps a state of fixed size per request: ``shape`` elements of ``dtype``
    ("float32", "int32", or "compute": the model's compute dtype), zero when a row opens."""
    shape: Tuple[int, ...]
    dtype: str = "float32"


def register_part(spec_type, impl) -> None:
    _PARTS[spec_type] = impl


def impl_of(spec):
    try:
        return _PARTS[type(spec)]
    except KeyError:
        raise KeyError(f"no part registered for spec type {type(spec).__name__}; "
                       f"known: {sorted(t.__name__ for t in _PARTS)}") from None


def build_part(spec, tensors, ops):
    return impl_of(spec)(spec, tensors, ops)


def tensors_of(spec):
    return impl_of(spec).tensors(spec)
