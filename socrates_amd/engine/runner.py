"""The step function: run one ragged batch through the model, from the cache.

It replaces the reference's separate ``prefill`` and ``decode_step``
(model/inference_paged.py:159-194): one call takes, for each request in the
batch, its next tokens (a portion of its prompt or one decoded token), takes the
pages they need, runs only those tokens, and returns the logits at the wanted
places. Generation, trace replay and the benchmark all go through it.
"""

from __future__ import annotations

from typing import List

import torch

from ..cache import CacheManager
from ..config import load_config
from ..parts import DecoderModel, cache_needs, expected_tensors
from ..weights import load_weights
from .batch import StepEntry, build_context


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager):
        self.model, self.cache = model, cache
        self.ops = model.ops
        self.vocab_size = model.plan.vocab_size

    @classmethod
    def from_folder(cls, folder, dtype, device, max_rows, max_len, block_size, num_blocks, ops=None):
        """Build model and cache for the model folder; the class of the model is chosen by
        its config.json."""
        config = load_config(folder)
        plan = config.plan()
        if ops is None:
            from ..kernels import HipKernels
            ops = HipKernels(dtype, device)
        weights = load_weights(folder, expected_tensors(plan), dtype, device)
        model = DecoderModel(plan, weights, ops)
        cache = CacheManager(cache_needs(plan), max_rows=max_rows, max_len=max_len,
                             block_size=block_size, num_blocks=num_blocks, dtype=dtype,
                             device=device)
        runner = cls(model, cache)
        runner.config = config
        return runner

    @torch.no_grad()
    def step(self, entries: List[StepEntry]) -> torch.Tensor:
        """Returns float32 logits [wanted places, vocab], in the order of the entries and of
        each entry's ``want``. Raises OutOfBlocks if the pages do not suffice (lengths
        are then unchanged; pages already taken stay with their rows)."""
        cache = self.cache
        starts = [cache.length(e.row) for e in entries]
        ctx = build_context(entries, starts, self.ops.device, self.vocab_size)
        for e, start in zip(entries, starts):
            cache.reserve(e.row, start + len(e.tokens))
        cache.sync()
        logits = self.model.forward(ctx, cache)
        for e in entries:
            cache.advance(e.row, len(e.tokens))
        return logits
