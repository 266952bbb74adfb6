"""Architecture-neutral description of a decoder: part specs and the model plan.

A *spec* is a frozen dataclass holding every size and constant one part needs.
A *plan* lists the specs of all layers, the order in which layers run, and the
tensor name each parameter has on disk. An architecture's configuration class
(for example ``Qwen3Config``) produces a plan; nothing below the plan knows
which architecture it came from.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x / sqrt(mean(x^2) + eps) * w  over the last ``dim`` elements."""
    dim: int
    eps: float


@dataclass(frozen=True)
class RopeSpec:
    """Rotate-half rotary encoding over the first ``rotary_dim`` of each head.

    inv_freq[j] = theta ** (-2j / rotary_dim) / factor, pairs are (j, j + rotary_dim/2).
    ``factor`` (1: none; the reference's model has none) stretches the positions a checkpoint was
    trained on by that much (linear position interpolation).
    """
    head_dim: int
    theta: float
    rotary_dim: int = 0          # 0 means the whole head
    factor: float = 1.0

    def __post_init__(self):
        if self.rotary_dim == 0:
            object.__setattr__(self, "rotary_dim", self.head_dim)
        if self.rotary_dim % 2 or self.rotary_dim > self.head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and <= head_dim {self.head_dim}")
        if not self.factor > 0:
            raise ValueError("factor must be positive")


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache.

    ``window`` = None: a query at position p sees keys 0..p. ``window`` = w: it
    sees keys max(0, p-w+1)..p. ``qk_norm`` is applied per head before
    ``position``; either may be None. Terms that other architectures add to the
    scores, all off by default: ``distance_slopes`` (one per query head: slope *
    (key position - query position) is added to the scaled score), ``softcap`` (the
    score becomes softcap * tanh(score / softcap)), ``sinks`` (a stored tensor
    ``sinks`` [n_heads]: one more logit per head that takes part in the softmax's
    sum and has no value).
    """
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float
    qk_norm: Optional[RMSNormSpec] = None
    position: Optional[object] = None
    window: Optional[int] = None
    softcap: Optional[float] = None
    sinks: bool = False
    distance_slopes: Optional[Tuple[float, ...]] = None

    def __post_init__(self):
        if self.softcap is not None and not self.softcap > 0:
            raise ValueError("softcap must be positive")
        if self.distance_slopes is not None and len(self.distance_slopes) != self.n_heads:
            raise ValueError(f"distance_slopes: one per query head ({self.n_heads}), not {len(self.distance_slopes)}")
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads {self.n_heads} is not a multiple of n_kv_heads {self.n_kv_heads}")
        if self.head_dim % 16 or not 16 <= self.head_dim <= 256:
            raise ValueError(f"head_dim {self.head_dim}: the attention kernels take multiples of 16 from 16 to 256")
        if self.window is not None and self.window < 1:
            raise ValueError("window must be at least 1")


@dataclass(frozen=True)
class SwiGLUSpec:
    """y = Wd((Wu x) * silu(Wg x)), no bias."""
    hidden: int
    intermediate: int


@dataclass(frozen=True)
class BlockSpec:
    """One layer: which mixer, feed-forward and norms, how they are arranged,
    and the prefix its tensors carry on disk.

    ``arrangement`` "prenorm": h = x + mixer(norm1(x)); y = h + ffn(norm2(h)).
    ``names`` maps the role of each sub-part to the name segment after
    ``prefix`` (for example {"mixer": "self_attn"}).
    """
    mixer: object
    ffn: object
    norm1: object
    norm2: object
    prefix: str
    names: Tuple[Tuple[str, str], ...] = (
        ("norm1", "input_layernorm"), ("mixer", "self_attn"),
        ("norm2", "post_attention_layernorm"), ("ffn", "mlp"))
    arrangement: str = "prenorm"

    def name_of(self, role: str) -> str:
        return self.prefix + dict(self.names)[role]


@dataclass(frozen=True)
class RunStep:
    """One entry of the execution order.

    ``layer`` indexes ``ModelPlan.layers`` (a layer may appear more than once);
    ``cache`` is the cache slot this execution uses; ``write`` False means the
    execution only reads what an earlier step wrote into that slot.
    """
    layer: int
    cache: int
    write: bool = True


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[BlockSpec, ...]
    order: Tuple[RunStep, ...]
    final_norm: object
    embedding_name: str
    final_norm_prefix: str
    head_name: Optional[str]      # None: the head is the embedding table (tied)
    eos_token_ids: Tuple[int, ...] = field(default=())
    # (stored name, name of an expected tensor): a checkpoint may also store the first if it
    # holds the very same values as the second (a tied head written out beside the embedding)
    duplicates: Tuple[Tuple[str, str], ...] = field(default=())
    # What some architectures put between the parts (none of it in the reference's model, so
    # the defaults leave the step as it is): the embedding's rows times a constant; the logits
    # times a constant, then logit_softcap * tanh(logits / logit_softcap).
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: Optional[float] = None

    def __post_init__(self):
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ValueError("logit_softcap must be positive")
        written = set()
        for step in self.order:
            if not 0 <= step.layer < len(self.layers):
                raise ValueError(f"run step names layer {step.layer}, the plan has {len(self.layers)}")
            if step.write:
                if step.cache in written:
                    raise ValueError(f"cache slot {step.cache} is written by two run steps")
                written.add(step.cache)
            elif step.cache not in written:
                raise ValueError(f"run step reads cache slot {step.cache} before any step wrote it")

    @property
    def n_cache_slots(self) -> int:
        return 1 + max(s.cache for s in self.order) if self.order else 0


def default_order(n_layers: int) -> Tuple[RunStep, ...]:
    """Every layer once, in index order, each with a cache slot of its own."""
    return tuple(RunStep(layer=i, cache=i) for i in range(n_layers))
