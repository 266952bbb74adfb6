"""Configurations drawn at random (seeded) from everything config.json allows: head sizes in
steps of 16, any number of heads and groups, widths and vocabularies that are no powers of two
(nor multiples of 8), pages of any size. Each runs one way of cutting its requests through the
step function, in float32 and in bfloat16, against the plain implementation."""

import random

import pytest
import torch

import plain_qwen3 as plain
from helpers import (make_runner, random_prompts, replay, trace_mixed, trace_portions, trace_tail_decode,
                     trace_whole, write_tiny)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: dict(atol=1e-4, rtol=1e-4), torch.bfloat16: dict(atol=6e-2, rtol=5e-2)}


def draw(case):
    rng = random.Random(77 + case)
    head_dim = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 128, 256])
    kv = rng.choice([1, 2, 3, 4, 5])
    group = rng.choice([1, 2, 3, 4, 5, 8]) if head_dim < 256 else rng.choice([1, 2])
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=rng.randint(50, 700),
               hidden_size=rng.choice([40, 44, 50, 64, 72, 88, 96, 120, 136, 200]),
               num_hidden_layers=rng.randint(1, 3), num_attention_heads=kv * group, num_key_value_heads=kv,
               head_dim=head_dim, intermediate_size=rng.choice([24, 50, 64, 100, 136, 160, 192, 232, 300]),
               rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]), rope_theta=rng.choice([1e4, 5e4, 1e6]),
               tie_word_embeddings=rng.random() < 0.5)
    tiny = dict(cfg=cfg, block_size=rng.choice([1, 2, 4, 8, 12, 16, 24, 32, 64]), gain_std=rng.choice([0.01, 0.1, 0.2]))
    cut = rng.choice(["whole", "tail", "portions", "mixed", "mixed, captured"])
    lengths = [rng.choice([1, 2, 5, 16, 17, 31, 33, 64, 70, 100, 129]) for _ in range(5)]
    if cut == "tail":
        lengths = [max(n, 34) for n in lengths]
    return tiny, cut, lengths


@pytest.mark.parametrize("case", range(16))
def test_a_configuration_drawn_at_random(tmp_path, case):
    tiny, cut, lengths = draw(case)
    label = f"{tiny['cfg']} pages of {tiny['block_size']}, {cut}, lengths {lengths}"
    folder = write_tiny(tmp_path / "m", tiny, seed=case)
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts(lengths, cfg["vocab_size"], seed=case)
    want = {f"r{i}": plain.forward(cfg, w, p) for i, p in enumerate(prompts)}
    bs = tiny["block_size"]
    for dtype in (torch.float32, torch.bfloat16):
        from socrates_amd.kernels import HipKernels
        # so few pages that finished requests' pages are used again
        longest = sorted((len(p) for p in prompts), reverse=True)[:4]
        num_blocks = sum(-(-n // bs) for n in longest)
        runner = make_runner(folder, HipKernels(dtype, DEV), max_rows=4, max_len=256, block_size=bs, num_blocks=num_blocks)
        if cut == "mixed, captured":
            runner.enable_graphs(4)
        steps = {"whole": lambda: trace_whole(prompts), "tail": lambda: trace_tail_decode(prompts, 32),
                 "portions": lambda: trace_portions(prompts, seed=case), "mixed": lambda: trace_mixed(prompts, seed=case),
                 "mixed, captured": lambda: trace_mixed(prompts, seed=case, prefill_frac=0.3)}[cut]()
        got = replay(runner, steps)
        tol = TOL[dtype]
        for rid in want:
            have = got[rid][-len(want[rid]):]
            bad = ((have - want[rid]).abs() > tol["atol"] + tol["rtol"] * want[rid].abs()).any(dim=-1)
            assert not bad.any(), (f"{label}, {dtype}: request {rid}, {int(bad.sum())} of {len(bad)} positions are off; "
                                   f"the first is position {int(bad.nonzero()[0])}")
        assert runner.cache.n_free_pages == num_blocks and not runner.cache.open_rows, label
