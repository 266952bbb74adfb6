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
    def __init__(self, ops, scalars, upload=None):
        """ops: the kernel set; scalars: the cache manager's RowScalars; upload: int32 numpy
        array -> device tensor (the step function's pinned staging), default a plain copy."""
        self.ops, self.scalars, self.upload = ops, scalars, upload

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
            # one copy for the three arrays: seeds and draws (64-bit, first, so that they are
            # aligned) and the temperatures, as 32-bit words
            n = len(idx)
            words = np.empty(5 * n, dtype=np.int32)
            words[:2 * n] = self.scalars.seed[idx].astype(np.int64).view(np.int32)
            words[2 * n:4 * n] = self.scalars.draws[idx].astype(np.int64).view(np.int32)
            words[4 * n:] = temperature.astype(np.float32).view(np.int32)
            dev = (self.upload(words) if self.upload is not None
                   else torch.from_numpy(words).to(logits.device))
            tokens = self.ops.sample(logits, dev[4 * n:].view(torch.float32),
                                     dev[:2 * n].view(torch.int64), dev[2 * n:4 * n].view(torch.int64))
        self.scalars.draws[idx] += 1
        return [int(t) for t in tokens.tolist()]
