"""A request and the engine's limits and exceptions.

Names and meanings are the reference's (model/inference_cont.py:21-24, 36-40,
65-82): MAX_BATCH rows, MAX_NEW_TOKENS per request, MAX_LEN slots per row,
MAX_QUEUE waiting requests; ``QueueFull`` and ``TooLong``; a ``Request`` with its
ids, output, row and timestamps. The values are not the reference's, which are sized
for a 24 GB GPU (18 rows of 2,048 slots): here 64 rows of 4,096 slots, whose worst-case
page pool is 39 GB at Qwen3-4B sizes and 69 GB at Qwen3-32B sizes, beside the weights
in 288 GB.
"""

from __future__ import annotations

import threading
import time
from dataclasses import dataclass, field
from typing import List, Optional

from ..sampling import SamplingParams

MAX_BATCH = 64
MAX_NEW_TOKENS = 1024
MAX_LEN = 4096
MAX_QUEUE = 16 * MAX_BATCH


class QueueFull(Exception):
    pass


class TooLong(Exception):
    pass


@dataclass
class Request:
    prompt: object                       # the text, or the token ids, as submitted
    ids: List[int] = field(default_factory=list)      # prompt token ids
    output: List[int] = field(default_factory=list)   # generated token ids
    sampling: SamplingParams = field(default_factory=SamplingParams)
    max_new_tokens: int = MAX_NEW_TOKENS
    eos_token_ids: tuple = ()
    done: bool = False
    row: int = -1
    submitted: float = field(default_factory=time.perf_counter)
    admitted: float = 0.0                # first given a row: submitted -> admitted is queue wait
    first_token: float = 0.0
    finished: float = 0.0
    cancelled: bool = False
    preemptions: int = 0                 # times its row was taken back and its cache recomputed
    event: threading.Event = field(default_factory=threading.Event)
    stream: Optional[object] = None      # a queue.Queue that receives tokens, None last

    def tokens(self) -> List[int]:
        """Everything the cache must hold before the next token is chosen."""
        return self.ids + self.output
