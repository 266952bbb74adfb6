"""The step function: run one ragged batch through the model, from the cache.

It replaces the reference's separate ``prefill`` and ``decode_step``
(model/inference_paged.py:159-194): one call takes, for each request in the
batch, its next tokens (a portion of its prompt or one decoded token), takes the
pages they need, runs only those tokens, and returns the logits at the wanted
places. Generation, trace replay and the benchmark all go through it.
"""

from __future__ import annotations

import dataclasses
from typing import List

import numpy as np
import torch

from ..cache import CacheManager
from ..config import load_config
from ..parts import DecoderModel, cache_needs, expected_tensors
from ..weights import load_weights
from .batch import NoHostView, PinnedUploader, StepContext, StepEntry, build_context


class _CapturedStep:
    """A decode step of one width and context bucket, ready to be run again: graphs of the
    pieces that can be captured, in order, and between them the blocks that cannot, run as
    they come, each with its output copied to the place the next graph reads."""

    def __init__(self, model, cache, ctx_seen):
        self.model, self.cache, self.ctx_seen = model, cache, ctx_seen
        self.pieces = []

    def graph(self, graph):
        self.pieces.append(graph)

    def eager(self, residual, pending, lo, hi):
        out = self.model.run(residual, pending, self.ctx_seen, self.cache, lo, hi, last_chains=False)
        if not isinstance(out, torch.Tensor):
            raise TypeError("a block that cannot be captured has to return a tensor")
        fixed = torch.empty_like(out)
        fixed.copy_(out)
        self.pieces.append((residual, pending, lo, hi, fixed))
        return fixed

    def replay(self):
        for piece in self.pieces:
            if isinstance(piece, tuple):
                residual, pending, lo, hi, fixed = piece
                fixed.copy_(self.model.run(residual, pending, self.ctx_seen, self.cache, lo, hi, last_chains=False))
            else:
                piece.replay()


class ModelRunner:
    def __init__(self, model: DecoderModel, cache: CacheManager):
        self.model, self.cache = model, cache
        self.ops = model.ops
        self.vocab_size = model.plan.vocab_size
        self._graphs = None              # (width, context) -> captured decode step, once enable_graphs ran
        self._staging_read = {}          # per captured step: event behind the last copy out of its staging buffer
        self._graph_max = 0
        self._graph_pool = None          # one memory pool for all captures: replays never overlap
        self.graphs_refused = None       # why enable_graphs left the steps eager, if it did
        self._graph_epoch = 0            # the kernel set's ``graph_epoch`` the held graphs were captured under
        if hasattr(model, "reserve"):
            model.reserve(cache.max_len)     # tables by position stand at their final addresses from here on
        # eager steps: the batch's integers go through pinned staging memory, one copy per step
        self._upload = PinnedUploader(self.ops.device) if self.ops.device.type == "cuda" else None

    @classmethod
    def from_folder(cls, folder, dtype, device, max_rows, max_len, block_size, num_blocks, ops=None):
        """Build model and cache for the model folder; the class of the model is chosen by
        its config.json."""
        config = load_config(folder)
        plan = config.plan()
        if ops is None:
            from ..kernels import HipKernels
            ops = HipKernels(dtype, device)
        weights = load_weights(folder, expected_tensors(plan), dtype, device, plan.duplicates)
        model = DecoderModel(plan, weights, ops)
        cache = CacheManager(cache_needs(plan), max_rows=max_rows, max_len=max_len,
                             block_size=block_size, num_blocks=num_blocks, dtype=dtype,
                             device=device)
        runner = cls(model, cache)
        runner.config = config
        return runner

    @torch.no_grad()
    def step(self, entries: List[StepEntry], borrow: bool = False, fed: torch.Tensor = None) -> torch.Tensor:
        """Returns float32 logits [wanted places, vocab], in the order of the entries and of
        each entry's ``want``. Raises OutOfBlocks if the pages do not suffice (lengths
        are then unchanged; pages already taken stay with their rows). ``borrow``: the
        caller uses the logits before the next step, so a captured step may hand out its own
        output buffer instead of a copy. ``fed``: int32 [entries] on the device, the one token
        of each entry where the host does not know it yet (the entries' own tokens are then
        placeholders); only where ``feeds`` says so."""
        cache = self.cache
        if (self._graphs is not None and len(entries) <= self._graph_max
                and all(len(e.tokens) == 1 for e in entries)):
            return self._step_captured(entries, borrow, fed)
        if fed is not None:
            raise ValueError("tokens can be fed from the device only to a step that `feeds` admits")
        starts = [cache.length(e.row) for e in entries]
        ctx = build_context(entries, starts, self.ops.device, self.vocab_size, self._upload)
        for e, start in zip(entries, starts):
            cache.reserve(e.row, start + len(e.tokens))
        cache.sync()
        logits = self.model.forward(ctx, cache)
        for e in entries:
            cache.advance(e.row, len(e.tokens))
        return logits

    # -- decode steps replayed from HIP graphs -----------------------------------------------------
    # The reference compiles its decode step with CUDA graphs, one per batch width
    # (model/inference_paged.py:99-130). Here a step in which every request brings one token
    # is replayed from a graph captured for its width (rounded up to a bucket; the padding
    # rows use the cache's null row, so they read and write the null page only). The graph's
    # inputs live at fixed addresses and are filled by one copy per step; key splits of the
    # attention kernel are planned for a bucket of context lengths (powers of two), so the
    # launch shape depends on a request's length only through that bucket.
    _BUCKETS = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64, 96, 128, 192, 256)

    def enable_graphs(self, max_width: int) -> None:
        """From now on steps in which every request brings one token are replayed from HIP
        graphs, up to ``max_width`` requests. A part that cannot be captured (``capturable =
        False``: it reads the host's view of the batch or waits for the device) is run as it
        comes, between the graphs of the blocks before and after it; a model with no block
        that can be captured, or whose final norm cannot, keeps all its steps eager, and
        ``graphs_refused`` then says so."""
        if self.ops.device.type != "cuda":
            return                       # a stand-in kernel set on the CPU has nothing to capture
        if not getattr(self.model, "capturable", True):
            segments = self.model.segments() if hasattr(self.model, "segments") else []
            if not getattr(self.model.final_norm, "capturable", True):
                self.graphs_refused = "the final norm declares capturable = False"
                return
            if not any(cap for cap, _, _ in segments):
                self.graphs_refused = "no block of the model can be captured (capturable = False)"
                return
        self._graphs = {}
        self._graph_max = max_width
        self._graph_pool = torch.cuda.graph_pool_handle()
        self._graph_epoch = getattr(self.ops, "graph_epoch", 0)

    def _drop_stale_graphs(self) -> None:
        """A captured step holds raw addresses and the choices of the kernel set at its
        capture. The kernel set counts what takes either away (a table made anew, copies of
        weights dropped, products tuned: ``graph_epoch``); graphs captured under another
        count are dropped here and captured anew when a step needs them."""
        epoch = getattr(self.ops, "graph_epoch", 0)
        if epoch != self._graph_epoch:
            if self._graphs:
                torch.cuda.synchronize(self.ops.device)      # no replay is on its way when its graph goes
                self._graphs.clear()
                self._staging_read.clear()
            self._graph_epoch = epoch

    def feeds(self, n_entries: int) -> bool:
        """Whether a step of ``n_entries`` single tokens can take them from the device
        (``step(..., fed=)``): such steps are the ones replayed from graphs, whose inputs
        live at fixed addresses."""
        return self._graphs is not None and n_entries <= self._graph_max

    def _bucket(self, n: int) -> int:
        for b in self._BUCKETS:
            if b >= n:
                return min(b, max(self._graph_max, n))
        return n

    def _context_bucket(self, longest: int) -> int:
        """The context length a graph is planned for: the next power of two (at least 256),
        capped by the cache's longest row."""
        b = 256
        while b < longest:
            b *= 2
        return min(b, self.cache.max_len)

    def warmup(self, max_width: int = None, max_context: int = None) -> int:
        """Capture, before serving, the decode step of every width bucket up to ``max_width``
        (default: what enable_graphs was given) for every context bucket up to
        ``max_context`` (default: the cache's longest row), as the reference captures all
        its widths when the engine is built (model/inference_paged.py:110-130). Returns the
        number of graphs now held. All captures share one memory pool (replays never
        overlap), so what they hold beyond it is one float32 logits buffer [width, vocab]
        per graph."""
        if self._graphs is None:
            return 0
        self._drop_stale_graphs()
        max_width = min(max_width or self._graph_max, self._graph_max)
        contexts, c = [], 256
        longest = min(max_context or self.cache.max_len, self.cache.max_len)
        while True:
            contexts.append(min(c, self.cache.max_len))
            if c >= longest:
                break
            c *= 2
        widths = sorted({self._bucket(n) for n in range(1, max_width + 1)})
        for context in sorted(set(contexts)):
            for width in widths:
                if (width, context) not in self._graphs:
                    self._graphs[(width, context)] = self._capture(width, context)
        return len(self._graphs)

    def _capture(self, width: int, context: int):
        dev = self.ops.device
        # rows of the input buffer: token ids, positions, cache rows, lengths after the step
        inputs = torch.zeros((4, width), dtype=torch.int32, device=dev)
        inputs[2].fill_(self.cache.null_row)
        staging = torch.zeros((4, width), dtype=torch.int32).pin_memory()
        host = staging.numpy()
        host[2] = self.cache.null_row
        arange = torch.arange(width + 1, dtype=torch.int32, device=dev)
        ctx = StepContext(
            n_tokens=width, n_seqs=width, n_want=width, token_ids=inputs[0], positions=inputs[1],
            token_rows=inputs[2], seq_rows=inputs[2], seq_qstart=arange, seq_ctx=inputs[3],
            want_index=arange[:width], max_q_len=1, max_ctx_len=context, host=NoHostView())
        model, cache = self.model, self.cache
        segments = model.segments() if not getattr(model, "capturable", True) else [(True, 0, len(model.plan.order))]
        # What a part that is run as it comes sees of the step: the same device tensors, and
        # the host's arrays of the staging buffer, which is filled before every replay.
        seen = dataclasses.replace(ctx, host={
            "positions": host[1], "token_rows": host[2], "seq_rows": host[2],
            "seq_qstart": np.arange(width + 1, dtype=np.int32), "seq_ctx": host[3]}) if len(segments) > 1 else ctx
        stream = torch.cuda.Stream(device=dev)
        stream.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(stream):
            model.forward(seen, cache)                   # warm up outside the capture
        torch.cuda.current_stream(dev).wait_stream(stream)
        torch.cuda.synchronize(dev)
        # The graphs hold raw addresses: every tensor they read (the inputs, ``arange`` through
        # ctx, what one piece hands to the next) lives as long as the record, which keeps it.
        step = _CapturedStep(model, cache, seen)
        residual = pending = logits = None
        for n, (capturable, lo, hi) in enumerate(segments):
            first, last = n == 0, n == len(segments) - 1
            if capturable or first:
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=self._graph_pool, stream=stream):
                    if first:
                        residual, pending = model.begin(ctx)
                    if capturable:
                        pending = model.run(residual, pending, ctx, cache, lo, hi)
                        if last:
                            logits = model.finish(residual, pending, ctx)
                step.graph(graph)
                if len(segments) > 1:
                    graph.replay()                       # what a block that runs as it comes sees now is a step's values
            if not capturable:
                # as it comes, now and at every replay; what it leaves goes to a fixed place
                # for the graph behind it
                pending = step.eager(residual, pending, lo, hi)
                if last:
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, pool=self._graph_pool, stream=stream):
                        logits = model.finish(residual, pending, ctx)
                    step.graph(graph)
        return step, inputs, staging, logits, ctx

    def _step_captured(self, entries: List[StepEntry], borrow: bool, fed: torch.Tensor = None) -> torch.Tensor:
        cache = self.cache
        n = len(entries)
        rows = [e.row for e in entries]
        if len(set(rows)) != n:
            raise ValueError("a cache row appears twice in one step")
        if fed is not None and (fed.dtype != torch.int32 or fed.shape != (n,) or fed.device.type != self.ops.device.type):
            raise ValueError(f"fed tokens must be int32 [{n}] on {self.ops.device}")
        self._drop_stale_graphs()
        width = self._bucket(n)
        # key splits of the attention kernel are planned per context bucket, so that a short
        # context is not cut into the many splits a long one needs
        context = self._context_bucket(max(cache.length(r) for r in rows) + 1)
        key = (width, context)
        if key not in self._graphs:
            self._graphs[key] = self._capture(width, context)
        graph, inputs, staging, logits, _ctx = self._graphs[key]
        copied = self._staging_read.get(key)
        if copied is not None:
            copied.synchronize()            # the last step's copy has read the staging buffer
        host = staging.numpy()
        host[0, n:], host[1, n:], host[2, n:], host[3, n:] = 0, 0, cache.null_row, 0
        for i, e in enumerate(entries):
            token = int(e.tokens[0])
            if not 0 <= token < self.vocab_size:
                raise ValueError(f"entry {i}: token id outside [0, {self.vocab_size})")
            if any(j != 0 for j in e.want):
                raise ValueError(f"entry {i}: wanted place outside its one token")
            start = cache.length(e.row)
            cache.reserve(e.row, start + 1)
            host[0, i], host[1, i], host[2, i], host[3, i] = token, start, e.row, start + 1
        cache.sync()
        inputs.copy_(staging, non_blocking=True)
        if fed is not None:
            inputs[0, :n].copy_(fed)
        copied = copied or torch.cuda.Event()
        copied.record()
        self._staging_read[key] = copied
        graph.replay()
        for e in entries:
            cache.advance(e.row, 1)
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if len(wanted) == n:
            return logits[:n] if borrow else logits[:n].clone()
        return logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)]
