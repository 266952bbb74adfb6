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


@dataclass
class Drawn:
    """The tokens of one call of ``Sampler.launch``: on the device at once (``tokens``, int32
    [n]), on the host once ``ready`` has passed."""
    tokens: torch.Tensor
    host: torch.Tensor
    ready: object = None


class Sampler:
    def __init__(self, ops, scalars, upload=None):
        """ops: the kernel set; scalars: the cache manager's RowScalars; upload: int32 numpy
        array -> device tensor (the step function's pinned staging), default a plain copy."""
        self.ops, self.scalars, self.upload = ops, scalars, upload
        # pinned buffers that the tokens come back through: one more than the calls whose
        # tokens can be outstanding at a time (a step and the one launched ahead of it)
        self._ring = [None, None, None]
        self._turn = 0

    def launch(self, logits: torch.Tensor, rows: Sequence[int]) -> Optional[Drawn]:
        """Queue the choice of one token for each row of ``logits`` (float32 [n, vocab]) and
        count the draws; ``rows[i]`` is the cache row whose sampling state applies. Does not
        wait for the device: ``collect`` does. None if there are no rows."""
        if len(rows) != logits.shape[0]:
            raise ValueError("one cache row per row of logits")
        if not len(rows):
            return None
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
        if tokens.device.type != "cuda":
            return Drawn(tokens, tokens)
        n = tokens.numel()
        self._turn = (self._turn + 1) % len(self._ring)
        slot = self._ring[self._turn]
        if slot is None or slot[0].numel() < n:
            slot = self._ring[self._turn] = (torch.empty(max(64, n), dtype=torch.int32).pin_memory(),
                                             torch.cuda.Event())
        host, ready = slot[0][:n], slot[1]
        host.copy_(tokens, non_blocking=True)
        ready.record()
        return Drawn(tokens, host, ready)

    @staticmethod
    def collect(drawn: Optional[Drawn]):
        """The tokens of a ``launch`` as a list of ints, once the device has them."""
        if drawn is None:
            return []
        if drawn.ready is not None:
            drawn.ready.synchronize()
        return [int(t) for t in drawn.host.tolist()]

    def sample(self, logits: torch.Tensor, rows: Sequence[int]):
        """``launch`` and ``collect`` in one: a list of ints, one token per row."""
        return self.collect(self.launch(logits, rows))
