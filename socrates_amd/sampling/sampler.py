"""Choosing the next token.

The reference is greedy: argmax of the last position's logits, the lowest index
among equal maxima (model/inference_paged.py:166, 193;
bench/day_8/equivalence.py:105-107). Added here: temperature sampling with a
random stream per request. The uniform number of a draw is a hash of the request's
seed and of how many tokens it has drawn, so the tokens of a request do not depend
on which other requests share its batch, on its cache row, or on a preemption in
between. The state (temperature, seed, draws) is part of the row's fixed-size
state in the cache manager and moves with the row.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np
import torch


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 is greedy. ``max_new_tokens`` None takes the engine's limit;
    ``eos_token_ids`` None takes the model's."""
    temperature: float = 0.0
    seed: int = 0
    max_new_tokens: Optional[int] = None
    eos_token_ids: Optional[Tuple[int, ...]] = None

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")


class Sampler:
    def __init__(self, ops, scalars):
        """ops: the kernel set; scalars: the cache manager's RowScalars."""
        self.ops, self.scalars = ops, scalars

    def sample(self, logits: torch.Tensor, rows: Sequence[int]):
        """One token for each row of ``logits`` (float32 [n, vocab]); ``rows[i]`` is the cache
        row whose sampling state applies. Returns a list of ints and counts the draws."""
        if len(rows) != logits.shape[0]:
            raise ValueError("one cache row per row of logits")
        if not len(rows):
            return []
        idx = np.asarray(rows, dtype=np.int64)
        temperature = self.scalars.temperature[idx]
        if not temperature.any():
            tokens = self.ops.argmax(logits)
        else:
            dev = logits.device
            tokens = self.ops.sample(
                logits, torch.from_numpy(temperature).to(dev),
                torch.from_numpy(self.scalars.seed[idx].astype(np.int64)).to(dev),
                torch.from_numpy(self.scalars.draws[idx]).to(dev))
        self.scalars.draws[idx] += 1
        return [int(t) for t in tokens.tolist()]
