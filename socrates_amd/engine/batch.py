"""One step's batch: requests with their next tokens, flattened for the kernels.

The reference runs either one whole prompt [1, T] or n single tokens [n, 1]
(model/qwen/qwen_kv_paged.py:207-224). Here a step is a ragged batch: any mix of
prompt portions (any length, starting where the row's cache ends) beside single
decoded tokens. All integers of a step travel to the device in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Sequence

import numpy as np
import torch

from ..cache.staging import PinnedUploader, pageable_upload  # noqa: F401


@dataclass
class StepEntry:
    """``tokens`` continue the request in cache row ``row``; ``want`` lists the places
    among these tokens whose logits are asked for."""
    row: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


class NoHostView(dict):
    """``StepContext.host`` of a step that is being captured into, or replayed from, a HIP
    graph: which rows, positions and lengths the step has is then known on the device only,
    so there is nothing to look up here. A part that walks the host arrays declares
    ``capturable = False`` and its model's steps stay eager."""

    def __missing__(self, key):
        raise KeyError(f"ctx.host[{key!r}]: a captured step has no host-side view of its batch; a part "
                       "that needs one declares `capturable = False`")


@dataclass
class StepContext:
    """``host``: numpy copies of positions, token_rows, seq_rows, seq_qstart and seq_ctx for
    parts that plan on the host (empty, a ``NoHostView``, in a captured step)."""
    n_tokens: int
    n_seqs: int
    n_want: int
    token_ids: torch.Tensor      # int32 [N]
    positions: torch.Tensor      # int32 [N] absolute position of each token
    token_rows: torch.Tensor     # int32 [N] cache row of each token
    seq_rows: torch.Tensor       # int32 [S] cache row of each sequence
    seq_qstart: torch.Tensor     # int32 [S+1] offsets of the sequences among the tokens
    seq_ctx: torch.Tensor        # int32 [S] tokens in the cache after this step
    want_index: torch.Tensor     # int32 [n_want] flat token indices
    max_q_len: int
    max_ctx_len: int
    host: dict = field(default_factory=dict)
    upload: object = None        # int32 numpy array -> device tensor, for kernels that plan on the host


def build_context(entries: List[StepEntry], starts: Sequence[int], device, vocab_size=None,
                  upload=None) -> StepContext:
    """``starts[i]`` is the position of the first token of ``entries[i]``. ``upload`` brings
    the step's integers to the device (default: a plain copy from pageable memory)."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    lens = [len(e.tokens) for e in entries]
    if min(lens) < 1:
        raise ValueError("every entry of a step brings at least one token")
    rows = [e.row for e in entries]
    if len(set(rows)) != len(rows):
        raise ValueError("a cache row appears twice in one step")
    N, S = sum(lens), len(entries)
    n_want = sum(len(e.want) for e in entries)
    total = 3 * N + S + (S + 1) + S + n_want
    buf = np.empty(total, dtype=np.int32)
    o = 0
    ids, o = buf[o:o + N], o + N
    pos, o = buf[o:o + N], o + N
    trow, o = buf[o:o + N], o + N
    srow, o = buf[o:o + S], o + S
    qst, o = buf[o:o + S + 1], o + S + 1
    sctx, o = buf[o:o + S], o + S
    want = buf[o:o + n_want]
    t = w = 0
    for i, e in enumerate(entries):
        n = lens[i]
        toks = np.asarray(e.tokens, dtype=np.int64)
        if toks.min() < 0 or (vocab_size is not None and toks.max() >= vocab_size):
            raise ValueError(f"entry {i}: token ids outside [0, {vocab_size})")
        ids[t:t + n] = toks
        pos[t:t + n] = np.arange(starts[i], starts[i] + n)
        trow[t:t + n] = e.row
        srow[i], qst[i], sctx[i] = e.row, t, starts[i] + n
        for j in e.want:
            if not 0 <= j < n:
                raise ValueError(f"entry {i}: wanted place {j} is outside its {n} tokens")
            want[w] = t + j
            w += 1
        t += n
    qst[S] = N
    upload = upload or pageable_upload(device)
    dev = upload(buf)
    o = 0
    views = []
    for n in (N, N, N, S, S + 1, S, n_want):
        views.append(dev[o:o + n])
        o += n
    return StepContext(
        n_tokens=N, n_seqs=S, n_want=n_want, token_ids=views[0], positions=views[1],
        token_rows=views[2], seq_rows=views[3], seq_qstart=views[4], seq_ctx=views[5],
        want_index=views[6], max_q_len=max(lens), max_ctx_len=int(sctx.max()),
        host={"positions": pos.copy(), "token_rows": trow.copy(), "seq_rows": srow.copy(),
              "seq_qstart": qst.copy(), "seq_ctx": sctx.copy()}, upload=upload)
