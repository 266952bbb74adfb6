"""The engine: submit, admit, run portions of prompts beside decoding rows, sample,
finish and free.

The surface follows the reference's ``Engine`` (model/inference_paged.py:54-238):
the same constructor arguments with the same meanings (``model``, ``tok``,
``device``, ``dtype``, ``compile``, ``max_batch``, ``max_len``, ``max_new_tokens``,
``block_size``, ``num_blocks``), ``submit`` returning a ``Request``, ``run`` until
everything is finished, results in ``req.output``. Differences: ``model`` is a
model folder (or a ready ``ModelRunner``), a prompt may be a list of token ids (a
tokenizer is optional), prompts are prefilled in portions of at most ``chunk``
tokens in the same step as the decoding rows, pages are taken lazily, and
``generate`` wraps submit + run.
"""

from __future__ import annotations

import time
from typing import List, Optional, Sequence

import torch

from ..cache import blocks_for
from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .request import MAX_BATCH, MAX_LEN, MAX_NEW_TOKENS, MAX_QUEUE, QueueFull, Request, TooLong  # noqa: F401
from .runner import ModelRunner
from .scheduler import Planned, Scheduler

KV_BLOCK = 16          # model/inference_paged.py:51
PREFILL_CHUNK = 2048   # token budget of one step


class _Flight:
    """A step that is queued on the device and whose tokens have not been taken yet."""
    __slots__ = ("plan", "wanted", "drawn")

    def __init__(self, plan, wanted, drawn):
        self.plan, self.wanted, self.drawn = plan, wanted, drawn


class Engine:
    def __init__(self, model, tok=None, device: str = "cuda:0", dtype=torch.bfloat16,
                 compile: bool = True, max_batch: int = MAX_BATCH, max_len: int = MAX_LEN,
                 max_new_tokens: int = MAX_NEW_TOKENS, block_size: int = KV_BLOCK,
                 num_blocks: Optional[int] = None, chunk: int = PREFILL_CHUNK,
                 max_queue: int = MAX_QUEUE, template=None, lookahead: bool = True):
        """model: a model folder (config.json + safetensors) or a ModelRunner. tok: an
        optional tokenizer with the HF surface the reference uses (``apply_chat_template``,
        ``__call__``, ``all_special_ids``); without one, prompts are token id lists.
        compile: replay decode-only steps from captured HIP graphs. num_blocks: pages in the
        pool; default is the worst case max_batch * ceil(max_len / block_size)
        (model/inference_paged.py:83-84). template: ``template(tok, text) -> token ids`` for
        text prompts; default: what the model's configuration class offers as
        ``chat_prompt`` (the architecture's chat format), else the tokenizer's plain encoding.
        lookahead: queue the next decode step before the last one's tokens are read (see
        ``step``); it needs ``compile``."""
        self.device, self.max_batch = device, max_batch
        self.max_len, self.max_new_tokens = max_len, max_new_tokens
        self.tok = tok
        if isinstance(model, ModelRunner):
            self.runner = model
        else:
            per_row = blocks_for(max_len, block_size)
            self.runner = ModelRunner.from_folder(
                model, dtype, device, max_rows=max_batch, max_len=max_len, block_size=block_size,
                num_blocks=num_blocks or max_batch * per_row)
        self.cache = self.runner.cache
        self.template = template or getattr(getattr(self.runner, "config", None), "chat_prompt", None)
        self.plan_ = self.runner.model.plan
        self.scheduler = Scheduler(self.cache, max_batch, max_len, chunk, max_queue)
        self.sampler = Sampler(self.runner.ops, self.cache.scalars, getattr(self.runner, "_upload", None))
        self.compile = compile
        if compile and hasattr(self.runner, "enable_graphs"):
            self.runner.enable_graphs(max_batch)
        self.lookahead = bool(lookahead and compile and hasattr(self.runner, "feeds"))
        self._flight: Optional[_Flight] = None   # the step queued ahead, if any
        self.n_ahead = 0                # steps that were queued ahead
        self.n_steps = 0
        self.last_portions: List[int] = []      # tokens of each request in the last step (1: a decoded token)
        self.prompt_tokens = 0          # counters in place of the reference's Prometheus ones
        self.output_tokens = 0

    # -- reference-compatible views ------------------------------------------------------------
    @property
    def pending(self):
        return self.scheduler.pending

    @property
    def rows(self):
        return self.scheduler.running

    @property
    def n_active(self) -> int:
        return len(self.scheduler.running)

    # -- submitting ------------------------------------------------------------------------------
    def submit(self, prompt, stream: bool = False, sampling: Optional[SamplingParams] = None) -> Request:
        """Queue a prompt (text if the engine has a tokenizer, else token ids). Raises
        QueueFull or TooLong as the reference does (model/inference_paged.py:132-148)."""
        sampling = sampling or SamplingParams()
        if isinstance(prompt, str):
            if self.tok is None:
                raise ValueError("a text prompt needs a tokenizer; pass token ids instead")
            if self.template is not None:
                ids = [int(t) for t in self.template(self.tok, prompt)]
            else:
                ids = [int(t) for t in self.tok(prompt).input_ids]
        else:
            ids = [int(t) for t in prompt]
        eos = sampling.eos_token_ids
        if eos is None:
            eos = tuple(self.tok.all_special_ids) if self.tok is not None else self.plan_.eos_token_ids
        req = Request(prompt=prompt, ids=ids, sampling=sampling, eos_token_ids=tuple(eos),
                      max_new_tokens=(sampling.max_new_tokens if sampling.max_new_tokens is not None
                                      else self.max_new_tokens))
        if stream:
            import queue
            req.stream = queue.Queue()
        if any(t < 0 or t >= self.plan_.vocab_size for t in ids):
            raise ValueError(f"token ids must lie in [0, {self.plan_.vocab_size})")
        self.scheduler.submit(req)
        return req

    # -- one step --------------------------------------------------------------------------------
    def step(self) -> int:
        """Plan and run one step, and take its tokens. Returns the number of tokens it ran
        (0: nothing to do).

        With ``lookahead``, the step after this one is queued before this one's tokens are
        awaited, where the scheduler knows it without them (``Scheduler.repeats``): the
        device takes the tokens from the sampler's output, so it goes from one decode step
        into the next without waiting for the host to read, record, plan and launch. Each
        call still returns with exactly one more step's tokens recorded; between calls the
        cache manager's lengths (and pages) are then those of the step queued ahead, one
        token further than the recorded outputs. A request that stops at a stop token has
        one place in the step that was queued ahead; that place's token is dropped, and its
        key and value lie beyond the request's end in pages that are freed with it."""
        flight = self._flight
        self._flight = None
        if flight is not None and not any(self._live(p.request) for p in flight.plan):
            flight = None                 # everyone in it was cancelled or retired meanwhile
        if flight is None:
            plan = self.scheduler.plan()
            if not plan:
                return 0
            flight = self._launch(plan, None)
        if self.lookahead and self.runner.feeds(len(flight.plan)) and self.scheduler.repeats(flight.plan):
            ahead = [Planned(p.request, [0], True) for p in flight.plan]
            self._flight = self._launch(ahead, flight.drawn.tokens)
            self.n_ahead += 1
        tokens = self.sampler.collect(flight.drawn)
        for p, token in zip(flight.wanted, tokens):
            if self._live(p.request):
                self.record(p.request, token)
        self.last_portions = [len(p.tokens) for p in flight.plan]
        self.n_steps += 1
        return sum(self.last_portions)

    @staticmethod
    def _live(req: Request) -> bool:
        return req.row >= 0 and not req.done and not req.cancelled

    def _launch(self, plan, fed) -> "_Flight":
        """Queue the step of ``plan`` and the choice of its tokens; ``fed``: the tokens of a
        step planned ahead, on the device."""
        entries = [StepEntry(p.request.row, p.tokens, [len(p.tokens) - 1] if p.wants_logits else [])
                   for p in plan]
        logits = self.runner.step(entries, borrow=True) if fed is None else \
            self.runner.step(entries, borrow=True, fed=fed)
        wanted = [p for p in plan if p.wants_logits]
        drawn = self.sampler.launch(logits, [p.request.row for p in wanted])
        for p in plan:
            if not p.request.output and fed is None:
                self.prompt_tokens += len(p.tokens)
        return _Flight(plan, wanted, drawn)

    def record(self, req: Request, token: int) -> None:
        """A stop token ends the request and is not kept (model/inference_paged.py:200-211);
        the request also ends when ``max_new_tokens`` tokens are kept, without running a
        further step for a token that would be dropped."""
        now = time.perf_counter()
        if not req.first_token:
            req.first_token = now
        if token in req.eos_token_ids:
            req.done = True
        else:
            req.output.append(token)
            self.output_tokens += 1
            if req.stream is not None:
                req.stream.put(token)
            if len(req.output) >= req.max_new_tokens:
                req.done = True
        if req.done:
            req.finished = now
            if req.stream is not None:
                req.stream.put(None)

    def run(self) -> None:
        """Until nothing is pending or running (model/inference_paged.py:231-237)."""
        while not self.scheduler.idle:
            if self.step() == 0 and not self.scheduler.idle:
                raise RuntimeError("requests are waiting but nothing can be scheduled")

    def warmup(self, max_width: Optional[int] = None, max_context: Optional[int] = None) -> int:
        """Before serving: capture the decode graphs of every width bucket up to
        ``max_width`` (default ``max_batch``) and every context bucket up to ``max_context``
        (default ``max_len``), as the reference does when its engine is built
        (model/inference_paged.py:110-130); without it a graph is captured at the first step
        that needs it. Returns the number of graphs held (0: steps are not captured)."""
        if not self.scheduler.idle:
            raise RuntimeError("warmup() runs on an idle engine")
        if not hasattr(self.runner, "warmup"):
            return 0
        return self.runner.warmup(max_width or self.max_batch, max_context or self.max_len)

    def tune(self, token_counts: Optional[Sequence[int]] = None) -> None:
        """Before serving: run a throwaway prompt of each of these lengths with the library
        timing its solutions for the model's products at that many rows (about a second per
        shape), and keep the fastest; up to 16 rows, where this package's own kernel is the
        rule, both are timed and the faster is kept for that shape. Default: a full portion,
        and the largest batch. Steps with other numbers of rows are not affected. Decode
        graphs are captured afterwards, so they replay the kept choices."""
        if not self.scheduler.idle:
            raise RuntimeError("tune() runs on an idle engine")
        ops = self.runner.ops
        if not hasattr(ops, "library_tuning"):
            return
        if token_counts is None:
            token_counts = [self.scheduler.token_budget, self.max_batch]
        kept = (self.n_steps, self.prompt_tokens, self.output_tokens)
        ops.library_tuning(True)
        try:
            for n in token_counts:
                n = max(1, min(int(n), self.scheduler.token_budget, self.max_len - 1))
                self.submit([i % self.plan_.vocab_size for i in range(n)],
                            sampling=SamplingParams(max_new_tokens=1, eos_token_ids=()))
                self.run()
                self.scheduler.retire_finished()
                if n <= 64 and ops.dtype == torch.bfloat16:
                    # a prompt asks for one row of logits; a decode step of n requests for n
                    self.runner.model.head_logits(torch.zeros(
                        (n, self.plan_.hidden), dtype=ops.dtype, device=ops.device))
        finally:
            ops.library_tuning(False)
        self.n_steps, self.prompt_tokens, self.output_tokens = kept

    # -- the Python entry point ------------------------------------------------------------------
    def generate(self, prompts: Sequence, max_new_tokens: Optional[int] = None,
                 temperature: float = 0.0, seed: int = 0,
                 eos_token_ids: Optional[Sequence[int]] = None) -> List[List[int]]:
        """Generate for every prompt; returns the new token ids of each. Request i draws
        from the random stream ``seed + i``."""
        reqs = [self.submit(p, sampling=SamplingParams(
            temperature=temperature, seed=seed + i, max_new_tokens=max_new_tokens,
            eos_token_ids=None if eos_token_ids is None else tuple(eos_token_ids)))
            for i, p in enumerate(prompts)]
        self.run()
        return [r.output for r in reqs]
