from .batch import NoHostView, StepContext, StepEntry, build_context
from .engine import KV_BLOCK, PREFILL_CHUNK, Engine
from .request import (MAX_BATCH, MAX_LEN, MAX_NEW_TOKENS, MAX_QUEUE, QueueFull, Request,
                      TooLong)
from .runner import ModelRunner
from .scheduler import Planned, Scheduler

__all__ = ["NoHostView", "StepContext", "StepEntry", "build_context", "Engine", "KV_BLOCK", "PREFILL_CHUNK",
           "MAX_BATCH", "MAX_LEN", "MAX_NEW_TOKENS", "MAX_QUEUE", "QueueFull", "Request", "TooLong",
           "ModelRunner", "Planned", "Scheduler"]
