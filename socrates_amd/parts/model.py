"""A decoder put together from a plan: embedding, blocks in the plan's order,
final norm, output head (model/qwen/qwen_kv_paged.py:207-224).

The forward pass runs exactly the tokens of one step batch, reads earlier
tokens from the cache, and computes the final norm and the head only at the
wanted places.
"""

from __future__ import annotations

import torch

from ..config.specs import ModelPlan
from .block import block_tensors, build_block
from .registry import TensorDecl, build_part, impl_of, tensors_of


def expected_tensors(plan: ModelPlan):
    """{tensor name on disk: TensorDecl} for the whole model."""
    out = {plan.embedding_name: TensorDecl((plan.vocab_size, plan.hidden))}
    for spec in plan.layers:
        out.update(block_tensors(spec))
    for local, decl in tensors_of(plan.final_norm).items():
        out[f"{plan.final_norm_prefix}.{local}"] = decl
    if plan.head_name is not None:
        out[plan.head_name] = TensorDecl((plan.vocab_size, plan.hidden))
    return out


def cache_needs(plan: ModelPlan):
    """The cache requirement of every cache slot, in slot order."""
    needs = [None] * plan.n_cache_slots
    for step in plan.order:
        mixer = plan.layers[step.layer].mixer
        need = impl_of(mixer).cache_need(mixer)
        if needs[step.cache] is not None and needs[step.cache] != need and step.write:
            raise ValueError(f"cache slot {step.cache} is claimed with two different needs")
        if step.write:
            needs[step.cache] = need
        elif needs[step.cache] != need:
            raise ValueError(f"run step of layer {step.layer} reads cache slot {step.cache}, "
                             f"whose contents {needs[step.cache]} are not what it needs ({need})")
    return needs


class DecoderModel:
    def __init__(self, plan: ModelPlan, weights, ops):
        self.plan, self.ops = plan, ops
        self.embed = weights[plan.embedding_name]
        self.blocks = [build_block(spec, weights, ops) for spec in plan.layers]
        norm_tensors = {local: weights[f"{plan.final_norm_prefix}.{local}"]
                        for local in tensors_of(plan.final_norm)}
        self.final_norm = build_part(plan.final_norm, norm_tensors, ops)
        self.head = self.embed if plan.head_name is None else weights[plan.head_name]
        # False if any part declares `capturable = False`: the runner then captures the runs of
        # blocks between such parts and runs those as they come (``segments``); a final norm
        # that cannot be captured leaves every step eager
        self.capturable = (all(getattr(b, "capturable", True) for b in self.blocks)
                           and getattr(self.final_norm, "capturable", True))

    def reserve(self, n_positions):
        """Before the first step: parts that keep tables by position (a rotation's cosines
        and sines) make them for ``n_positions``, the cache's longest row, so that they
        stand at their final addresses when steps are captured."""
        for block in self.blocks:
            if hasattr(block, "reserve"):
                block.reserve(n_positions)

    def forward(self, ctx, cache):
        """ctx: a StepContext on the device; cache: the CacheManager. Returns float32
        logits [len(ctx.want_index), vocab]."""
        residual, pending = self.begin(ctx)
        pending = self.run(residual, pending, ctx, cache, 0, len(self.plan.order))
        return self.finish(residual, pending, ctx)

    # The forward pass in pieces, for a runner that captures what can be captured and runs
    # the rest as it comes: begin (the embedding), run (some entries of the run order), finish
    # (final norm and head). ``residual`` is one float32 tensor from begin to finish, updated
    # in place; ``pending`` is what the last block left un-added.
    def begin(self, ctx):
        residual = self.ops.embedding(ctx.token_ids, self.embed)
        if self.plan.embedding_scale != 1.0:
            self.ops.scale_softcap_(residual, self.plan.embedding_scale)
        return residual, None

    def run(self, residual, pending, ctx, cache, lo, hi, last_chains=True):
        """Entries lo .. hi - 1 of the run order. ``last_chains``: the last of them may leave
        its sum and the next block's first norm to its last product, as blocks inside the run
        do; without it, it returns its output as a tensor."""
        order = self.plan.order
        for i in range(lo, hi):
            step = order[i]
            block = self.blocks[step.layer]
            if getattr(block, "chains", False):
                # the block may leave its last sum and the next block's first norm to its last product
                follows = i + 1 < len(order) and (i + 1 < hi or last_chains)
                nxt = self.blocks[order[i + 1].layer] if follows else None
                pending = block.forward(residual, pending, ctx, cache.slot(step.cache), step.write,
                                        nxt=nxt if getattr(nxt, "chains", False) else None)
            else:
                pending = block.forward(residual, pending, ctx, cache.slot(step.cache), step.write)
        return pending

    def finish(self, residual, pending, ctx):
        if ctx.n_want == 0:
            # The cache is complete after the last block; no logits are asked for.
            return torch.empty((0, self.plan.vocab_size), dtype=torch.float32, device=self.ops.device)
        # (the normed rows go to the head's product and nowhere else: their layout is the kernel set's)
        if getattr(self.final_norm, "free_layout", False):
            h = self.final_norm.add_norm(residual, pending, rows=ctx.want_index, by_tile=True)
        else:
            h = self.final_norm.add_norm(residual, pending, rows=ctx.want_index)
        return self.head_logits(h)

    def segments(self):
        """The run order cut into runs that a runner may capture and single entries that it
        may not (a part of their block says ``capturable = False``): [(capturable, lo, hi)]."""
        out = []
        for i, step in enumerate(self.plan.order):
            cap = getattr(self.blocks[step.layer], "capturable", True)
            if cap and out and out[-1][0]:
                out[-1] = (True, out[-1][1], i + 1)
            else:
                out.append((cap, i, i + 1))
        return out

    def head_logits(self, h):
        """float32 logits [n, vocab] of normed rows ``h`` [n, hidden]."""
        logits = self.ops.linear(h, self.head, out_dtype=torch.float32)
        if self.plan.logit_scale != 1.0 or self.plan.logit_softcap is not None:
            self.ops.scale_softcap_(logits, self.plan.logit_scale, self.plan.logit_softcap)
        return logits
