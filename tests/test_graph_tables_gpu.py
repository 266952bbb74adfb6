"""What a captured decode step reads by address stays where it is, or the step is dropped.

The reference keeps cache and tables in module buffers so that its captured steps find
them (model/qwen/qwen_kv_cont.py:97-127). Here the fused decode attention looks cosines
and sines up in a table by position; these tests run the schedules under which a table
that grows on demand would be freed under a captured step: a long prompt beside a short
request that decodes from a graph, and ``Engine.warmup()`` over all context buckets of
a cache of 4,096 tokens. Head size 64 (and 128 in test_real_sizes_gpu.py): the sizes at
which bfloat16 decode steps take that kernel."""

import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY_D, captured_decode_beside_a_long_prompt, make_runner, random_prompts, write_tiny

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: dict(atol=1e-4, rtol=1e-4), torch.bfloat16: dict(atol=6e-2, rtol=5e-2)}


def assert_every_choice_near_the_best(cfg, w, prompt, got, tol):
    """bfloat16 greedy tokens, each judged behind the tokens the engine chose itself: with
    every logit within ``tol`` of the plain one, the chosen token's plain logit lies within
    twice that of the plain maximum."""
    ids = list(prompt)
    for n, g in enumerate(got):
        logits = plain.forward(cfg, w, ids)[-1]
        best = float(logits.max())
        slack = 2 * (tol["atol"] + tol["rtol"] * abs(best))
        assert best - float(logits[g]) <= slack, (f"token {n} after a {len(prompt)}-token prompt: the engine chose "
                                                  f"{g} ({float(logits[g]):.3f}), the plain maximum is {best:.3f}")
        ids.append(g)


@pytest.fixture(scope="module")
def tiny_d(tmp_path_factory):
    folder = write_tiny(tmp_path_factory.mktemp("tables") / "D", TINY_D, seed=8)
    cfg, w = plain.read_folder(folder)
    short, long_ = random_prompts([70, 2300], cfg["vocab_size"], seed=12)
    return folder, cfg, w, short, long_


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_captured_step_is_right_after_a_long_prompt(tiny_d, dtype):
    from socrates_amd.kernels import HipKernels
    folder, cfg, w, short, long_ = tiny_d
    want_short, want_long = plain.forward(cfg, w, short), plain.forward(cfg, w, long_)
    runner = make_runner(folder, HipKernels(dtype, DEV), max_rows=3, max_len=4096, block_size=32)
    runner.enable_graphs(2)

    def close(got, want, what):
        torch.testing.assert_close(got, want, **TOL[dtype], msg=lambda m: f"{what}: {m}")

    captured_decode_beside_a_long_prompt(runner, short, long_, want_short, want_long, close, first_decoded=40)
    if dtype == torch.bfloat16:
        assert runner.ops.last_attention_kernel == ("fused", 1)


def test_a_table_made_anew_drops_the_captured_steps(tiny_d):
    """Should a table be made anew after all (a caller that steps beyond what was reserved),
    the kernel set says so and the runner captures its steps again instead of replaying
    them over the freed one."""
    from socrates_amd.engine import StepEntry
    from socrates_amd.kernels import HipKernels
    from socrates_amd.parts.rope import shared_table
    folder, cfg, w, short, _ = tiny_d
    want = plain.forward(cfg, w, short)
    ops = HipKernels(torch.bfloat16, DEV)
    ops.pack_min_elements = 0                             # the products read copies of the weights by tile
    runner = make_runner(folder, ops, max_rows=2, max_len=512, block_size=32)
    table = shared_table(ops, cfg["rope_theta"], cfg["head_dim"])
    assert table.rows.shape[0] == 512                     # reserved for the cache's longest row, once
    layers = [b.mixer.position.shared for b in runner.model.blocks]
    assert all(t is table for t in layers)                # one table for all layers
    runner.enable_graphs(2)
    row = runner.cache.open_row()
    runner.step([StepEntry(row, short[:60], [])])
    got = runner.step([StepEntry(row, short[60:61], [0])]).float().cpu()
    torch.testing.assert_close(got[0], want[60], **TOL[torch.bfloat16])
    first = runner._graphs[(1, 256)][0]
    address = table.rows.data_ptr()
    table.reserve(2048)
    assert table.rows.data_ptr() != address and ops.graph_epoch == 1
    junk = torch.full((512 * 64,), 3.0e4, dtype=torch.float32, device=DEV)     # takes the freed block
    got = runner.step([StepEntry(row, short[61:62], [0])]).float().cpu()
    torch.testing.assert_close(got[0], want[61], **TOL[torch.bfloat16])
    assert runner._graphs[(1, 256)][0] is not first
    del junk
    # dropping the weights' copies by tile does the same
    second = runner._graphs[(1, 256)][0]
    assert ops._packed
    ops.forget_packed()
    assert ops.graph_epoch == 2
    got = runner.step([StepEntry(row, short[62:63], [0])]).float().cpu()
    torch.testing.assert_close(got[0], want[62], **TOL[torch.bfloat16])
    assert runner._graphs[(1, 256)][0] is not second and runner._graph_epoch == 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_warmup_over_all_context_buckets_then_generation(tiny_d, dtype):
    """``Engine.warmup()`` with a cache of 4,096 tokens captures the buckets 256 .. 4,096 one
    after the other; short and long requests generated afterwards give the plain run's
    tokens."""
    from socrates_amd.engine import Engine
    folder, cfg, w, short, long_ = tiny_d
    cfg64, w64 = plain.read_folder(folder, torch.float64)
    prompts = [short[:30], long_[:2100], short[:9], long_[100:700]]
    want = [plain.greedy(cfg64, w64, p, 5) for p in prompts]
    engine = Engine(str(folder), dtype=dtype, max_batch=2, max_len=4096, max_new_tokens=5, block_size=32, chunk=1024)
    assert engine.warmup() == 2 * 5                       # widths 1, 2 x contexts 256 .. 4,096
    got = engine.generate(prompts)
    if dtype == torch.float32:
        assert got == want
    else:
        assert all(len(g) == 5 for g in got)
        for p, g in zip(prompts, got):
            assert_every_choice_near_the_best(cfg64, w64, p, g, TOL[dtype])
    assert len(engine.runner._graphs) == 10               # nothing was captured anew
