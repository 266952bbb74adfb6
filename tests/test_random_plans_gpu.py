"""Model plans drawn at random (seeded) from what the specs allow beyond the reference's model:
windows, a rotation over half a head or over stretched positions or none, heads without their
norm, further score terms, any scale, embedding and logit multipliers, a soft cap on the logits,
tied or untied heads, layers that differ in all of it. Each runs a trace (portions of three
requests side by side, their last tokens one by one, with or without captured steps) through the
HIP kernels in float32 against the same plan and weights over the torch stand-in on the CPU."""

import math
import random

import pytest
import torch

from torch_kernels import TorchKernels
from socrates_amd.cache import CacheManager
from socrates_amd.config import AttentionSpec, BlockSpec, ModelPlan, RMSNormSpec, RopeSpec, RunStep, SwiGLUSpec
from socrates_amd.engine import ModelRunner, StepEntry
from socrates_amd.parts import DecoderModel, cache_needs, expected_tensors
from socrates_amd.weights import random_tensors

pytestmark = pytest.mark.gpu


def draw(case):
    rng = random.Random(900 + case)
    hidden = rng.choice([32, 48, 64, 72, 96])
    vocab = rng.randint(40, 300)
    blocks, said = [], []
    for i in range(rng.randint(1, 3)):
        D = rng.choice([16, 32, 48, 64, 64, 128])
        kv, group = rng.choice([1, 2, 3]), rng.choice([1, 2, 4, 5])
        rot = rng.choice(["whole", "whole", "half", "stretched", "none"])
        position = {"whole": RopeSpec(D, 1e4), "half": RopeSpec(D, 1e4, rotary_dim=D // 2),
                    "stretched": RopeSpec(D, 5e4, factor=rng.choice([2.0, 8.0])), "none": None}[rot]
        qk_norm = RMSNormSpec(D, 1e-6) if rng.random() < 0.7 else None
        window = rng.choice([None, None, 3, 8, 20])
        terms = {}
        if rng.random() < 0.3:
            terms["softcap"] = rng.choice([2.0, 10.0])
        if rng.random() < 0.3:
            terms["sinks"] = True
        if rng.random() < 0.3:
            terms["distance_slopes"] = tuple(-0.5 ** (j % 4 + 1) for j in range(kv * group))
        scale = rng.choice([D ** -0.5, D ** -0.5, 1.0 / D, 0.2])
        attention = AttentionSpec(hidden, kv * group, kv, D, scale, qk_norm, position, window=window, **terms)
        blocks.append(BlockSpec(attention, SwiGLUSpec(hidden, rng.choice([48, 64, 100, 160])), RMSNormSpec(hidden, 1e-6),
                                RMSNormSpec(hidden, 1e-5), prefix=f"model.layers.{i}."))
        said.append(f"[head size {D}, {kv * group}/{kv} heads, rotation {rot}, norm {qk_norm is not None}, window {window}, "
                    f"{sorted(terms)}, scale {scale:.3g}]")
    extras = {}
    if rng.random() < 0.3:
        extras["embedding_scale"] = math.sqrt(hidden)
    if rng.random() < 0.3:
        extras["logit_scale"] = 0.5
    if rng.random() < 0.3:
        extras["logit_softcap"] = 5.0
    plan = ModelPlan(architecture="Toy", vocab_size=vocab, hidden=hidden, layers=tuple(blocks),
                     order=tuple(RunStep(i, i) for i in range(len(blocks))), final_norm=RMSNormSpec(hidden, 1e-6),
                     embedding_name="embed.weight", final_norm_prefix="final_norm",
                     head_name=rng.choice([None, "head.weight"]), **extras)
    page = rng.choice([4, 8, 16, 32])
    lengths = [rng.choice([3, 17, 40, 70]) for _ in range(3)]
    captured = rng.random() < 0.5
    label = f"width {hidden}, vocabulary {vocab}, pages of {page}, lengths {lengths}, captured {captured}, {sorted(extras)} " + " ".join(said)
    return plan, page, lengths, captured, label


def trace(prompts, case):
    """Steps of (request, first token, tokens): portions of changing size side by side, the
    last six tokens of every request one by one."""
    r = random.Random(case)
    at = {i: 0 for i in range(len(prompts))}
    steps = []
    while at:
        batch = []
        for i in r.sample(sorted(at), r.randint(1, len(at))):
            left = len(prompts[i]) - at[i]
            n = 1 if left <= 6 else min(left - 6, r.choice([2, 5, 16, 33]))
            batch.append((i, at[i], n))
            at[i] += n
            if at[i] == len(prompts[i]):
                del at[i]
        steps.append(batch)
    return steps


def run(plan, ops, page, prompts, steps, captured):
    weights = random_tensors(expected_tensors(plan), seed=3, dtype=torch.float32, device="cpu", std=0.2, gain_std=0.1)
    weights = {k: v.to(ops.device) for k, v in weights.items()}
    cache = CacheManager(cache_needs(plan), 4, 128, page, 4 * 128 // page, ops.dtype, ops.device)
    runner = ModelRunner(DecoderModel(plan, weights, ops), cache)
    if captured:
        runner.enable_graphs(4)
    rows = {i: cache.open_row() for i in range(len(prompts))}
    got = {i: [] for i in range(len(prompts))}
    for batch in steps:
        logits = runner.step([StepEntry(rows[i], prompts[i][a:a + n], list(range(n))) for i, a, n in batch]).float().cpu()
        o = 0
        for i, a, n in batch:
            got[i].append(logits[o:o + n])
            o += n
    return {i: torch.cat(v) for i, v in got.items()}


@pytest.mark.parametrize("case", range(12))
def test_a_plan_drawn_at_random(case):
    from socrates_amd.kernels import HipKernels
    plan, page, lengths, captured, label = draw(case)
    g = torch.Generator().manual_seed(case)
    prompts = [[int(t) for t in torch.randint(0, plan.vocab_size, (n,), generator=g)] for n in lengths]
    steps = trace(prompts, case)
    want = run(plan, TorchKernels(torch.float32, "cpu"), page, prompts, steps, False)
    got = run(plan, HipKernels(torch.float32, "cuda:0"), page, prompts, steps, captured)
    for i in want:
        torch.testing.assert_close(got[i], want[i], atol=2e-4, rtol=2e-4, msg=lambda m: f"{label}: request {i}: {m}")
