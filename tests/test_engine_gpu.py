"""Generation through the entry points on the GPU: the Python ``Engine.generate`` and the
command line, greedy and with temperature, against the plain implementation."""

import subprocess
import sys
from pathlib import Path

import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY_A, TINY_B, random_prompts, write_tiny
from torch_kernels import uniform_of

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


def assert_same_where_clear(cfg, w, prompt, want, got, min_margin=0.05):
    """bfloat16 greedy tokens ``got`` against the plain run's ``want``: every token must be the
    same up to the first choice that the plain run won by less than ``min_margin`` (a bf16
    argmax may flip there under any change of summation order, as the reference notes,
    docs/day_8_docs.md:262-297; what follows such a token is another sequence). Returns the
    number of tokens that had to agree, so that callers can insist that the test checks
    something."""
    assert len(got) == len(want)
    ids, n = list(prompt), 0
    for t, g in zip(want, got):
        top = plain.forward(cfg, w, ids)[-1].topk(2).values
        if float(top[0] - top[1]) < min_margin:
            break
        assert g == t, f"token {n} after a {len(prompt)}-token prompt: {g}, the plain run has {t}"
        ids.append(t)
        n += 1
    return n


def test_greedy_tiny_a_workload(tmp_path):
    """Tiny A: prompts of 5, 17 and 33 ids (seed 0), 8 greedy tokens each."""
    from socrates_amd.engine import Engine
    folder = write_tiny(tmp_path / "A", TINY_A, seed=0)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([5, 17, 33], cfg["vocab_size"], seed=0)
    want = [plain.greedy(cfg, w, p, 8) for p in prompts]
    engine = Engine(str(folder), dtype=torch.float32, max_batch=4, max_len=64, max_new_tokens=8, block_size=16)
    assert engine.generate(prompts) == want
    assert engine.cache.n_free_pages == 4 * 4 and not engine.cache.open_rows
    for compile_ in (True, False):
        engine = Engine(str(folder), dtype=torch.bfloat16, max_batch=4, max_len=64, max_new_tokens=8,
                        block_size=16, compile=compile_)
        got = engine.generate(prompts)
        checked = [assert_same_where_clear(cfg, w, p, x, g) for p, g, x in zip(prompts, got, want)]
        assert sum(checked) >= 20 and sum(c == 8 for c in checked) >= 2, checked


def test_temperature_tiny_b_workload(tmp_path):
    """Tiny B: prompts of 1, 9, 24 and 40 ids (seed 1), prefill chunk 7, temperature 0.8
    seeded; in float32 the draws equal an inverse-CDF draw from the plain logits."""
    from socrates_amd.engine import Engine
    folder = write_tiny(tmp_path / "B", TINY_B, seed=1)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([1, 9, 24, 40], cfg["vocab_size"], seed=1)
    engine = Engine(str(folder), dtype=torch.float32, max_batch=4, max_len=64, max_new_tokens=6, block_size=8, chunk=7)
    got = engine.generate(prompts, temperature=0.8, seed=50)
    again = Engine(str(folder), dtype=torch.float32, max_batch=2, max_len=64, max_new_tokens=6, block_size=8,
                   chunk=64).generate(prompts, temperature=0.8, seed=50)
    assert got == again                                   # seeded, whatever the batching
    for i, (p, out) in enumerate(zip(prompts, got)):
        ids = list(p)
        for draw, tok in enumerate(out):
            logits = plain.forward(cfg, w, ids)[-1]
            cdf = torch.cumsum(torch.softmax(logits / 0.8, -1), -1)
            u = uniform_of(50 + i, draw)
            lo = float(cdf[tok - 1]) if tok else 0.0
            assert lo - 1e-4 <= u <= float(cdf[tok]) + 1e-4, (i, draw)
            ids.append(tok)


def test_tuned_library_products_leave_the_tokens_alone(tmp_path, request):
    """``Engine.tune``: the library picks its fastest solution for the products of a 33-token
    portion (bfloat16, more than 16 rows); greedy tokens stay those of the plain run, the
    counters and the cache are as before, and nothing is written to the working folder."""
    import os
    from socrates_amd.engine import Engine
    request.addfinalizer(lambda: torch.cuda.tunable.enable(False))     # what is tuned here stays here
    folder = write_tiny(tmp_path / "A", TINY_A, seed=0)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([33, 20], cfg["vocab_size"], seed=3)
    want = [plain.greedy(cfg, w, p, 6) for p in prompts]
    engine = Engine(str(folder), dtype=torch.bfloat16, max_batch=4, max_len=64, max_new_tokens=6, block_size=16)
    before = set(os.listdir("."))
    engine.tune([33, 20])
    assert (engine.n_steps, engine.prompt_tokens, engine.output_tokens) == (0, 0, 0)
    assert engine.cache.n_free_pages == 4 * 4 and not engine.cache.open_rows
    got = engine.generate(prompts)
    checked = [assert_same_where_clear(cfg, w, p, x, g) for p, g, x in zip(prompts, got, want)]
    assert checked[1] == 6, checked
    with pytest.raises(RuntimeError):
        engine.submit(prompts[0])
        engine.tune()
    engine.run()
    assert set(os.listdir(".")) == before
    # up to 16 rows both ways of a product are timed and the faster is noted per shape; the
    # tokens are the same whichever way the table points
    ops = engine.runner.ops
    engine.tune([2])
    two_rows = [k for k in ops.product_choice if k[0] == 2]
    # (with the norms left to the products, most products of a short step are not up for
    # choice: the first layer's input, the last layer's output and the head are)
    assert len(two_rows) >= 3 and set(ops.product_choice.values()) <= {"own", "library"}
    ops.fuse_norms = False
    engine.tune([2])
    assert len([k for k in ops.product_choice if k[0] == 2]) >= 4
    ops.fuse_norms = True
    for way in ("library", "own"):
        ops.product_choice = {k: way for k in ops.product_choice}
        ops.invalidate_graphs()                          # captured steps hold the way they were captured with
        got = engine.generate(prompts[:2])
        checked = [assert_same_where_clear(cfg, w, p, x, g) for p, g, x in zip(prompts, got, want)]
        assert checked[1] == 6, checked


def test_command_line(tmp_path):
    folder = write_tiny(tmp_path / "A", TINY_A, seed=0)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([5, 17], cfg["vocab_size"], seed=2)
    want = [plain.greedy(cfg, w, p, 5) for p in prompts]
    cmd = [sys.executable, "-m", "socrates_amd.generate", "--model", str(folder), "--dtype", "float32",
           "--max-new-tokens", "5", "--max-len", "64", "--max-batch", "2"]
    for p in prompts:
        cmd += ["--prompt-ids", ",".join(map(str, p))]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(ROOT))
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().split("\n")
    assert lines[0].startswith("2 requests, 2 rows")
    shown = [l for i, l in enumerate(lines) if i > 0 and lines[i - 1].startswith("> ")]
    assert shown == [" ".join(map(str, x)) for x in want]
    assert lines[-1].endswith("tok/s") and "| 10 tok |" in lines[-1]


def test_command_line_with_a_preset(tmp_path):
    """``--preset tiny-b``: the command line writes a seeded random model of that configuration
    into --model and generates from it; the plain implementation reads the same folder."""
    folder = tmp_path / "B"
    cmd = [sys.executable, "-m", "socrates_amd.generate", "--model", str(folder), "--preset", "tiny-b", "--seed", "4",
           "--dtype", "float32", "--max-new-tokens", "4", "--max-len", "64", "--max-batch", "2", "--block-size", "8",
           "--prompt-ids", "7,300,12,5,9"]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300, cwd=str(ROOT))
    assert proc.returncode == 0, proc.stderr[-2000:]
    cfg, w = plain.read_folder(folder, torch.float64)
    assert (cfg["num_hidden_layers"], cfg["head_dim"], cfg["vocab_size"]) == (3, 32, 384)
    want = plain.greedy(cfg, w, [7, 300, 12, 5, 9], 4)
    lines = proc.stdout.strip().split("\n")
    shown = [l for i, l in enumerate(lines) if i > 0 and lines[i - 1].startswith("> ")]
    assert shown == [" ".join(map(str, want))]


def test_steps_queued_ahead_change_no_token(tmp_path):
    """The engine queues the next decode step before it has read the last one's tokens.
    Requests that stop at a stop token in the middle (the step queued ahead then has a
    wasted place), limits of different lengths, a request submitted while a step is ahead,
    a cancelled one, temperature, and a pool in which the step ahead does not always find
    its pages: the tokens are those of an engine that never queues ahead, and in float32
    the plain run's."""
    from socrates_amd.engine import Engine
    from socrates_amd.sampling import SamplingParams
    folder = write_tiny(tmp_path / "A", TINY_A, seed=2)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([5, 17, 33, 2, 21], cfg["vocab_size"], seed=3)
    free = [plain.greedy(cfg, w, p, 20) for p in prompts]
    # request i stops at the token that the plain run has at place stops[i] (if it does not
    # appear earlier, which the expected output below accounts for)
    stops, limits = [6, 11, None, 3, None], [20, 20, 9, 20, 14]
    want, eos = [], []
    for out, stop, limit in zip(free, stops, limits):
        eos.append(() if stop is None else (out[stop],))
        cut = out.index(out[stop]) if stop is not None else len(out)
        want.append(out[:min(cut, limit)])

    def run(lookahead, num_blocks=None):
        engine = Engine(str(folder), dtype=torch.float32, max_batch=4, max_len=64, max_new_tokens=20,
                        block_size=16, num_blocks=num_blocks, lookahead=lookahead)
        reqs = [engine.submit(p, sampling=SamplingParams(max_new_tokens=n, eos_token_ids=e))
                for p, n, e in list(zip(prompts, limits, eos))[:4]]
        for _ in range(4):
            engine.step()
        reqs.append(engine.submit(prompts[4], sampling=SamplingParams(max_new_tokens=limits[4], eos_token_ids=eos[4])))
        doomed = engine.submit(prompts[0], sampling=SamplingParams(max_new_tokens=20, eos_token_ids=()))
        while not doomed.output:
            engine.step()
        doomed.cancelled = True
        engine.run()
        engine.cache.check()
        assert not engine.cache.open_rows and engine.cache.n_free_pages == (num_blocks or 16)
        return [r.output for r in reqs], engine

    got, engine = run(True)
    assert got == want
    assert engine.n_ahead >= 8, engine.n_ahead
    plainly, engine = run(False)
    assert plainly == want and engine.n_ahead == 0
    tight, engine = run(True, num_blocks=7)
    assert tight == want

    outs = []
    for lookahead in (True, False):
        engine = Engine(str(folder), dtype=torch.bfloat16, max_batch=4, max_len=64, max_new_tokens=16,
                        block_size=16, lookahead=lookahead)
        outs.append(engine.generate(prompts, temperature=0.7, seed=11, eos_token_ids=()))
        assert (engine.n_ahead > 0) == lookahead
    assert outs[0] == outs[1]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_engine_under_page_pressure(tmp_path, dtype):
    """Pools so small that requests wait, have their portions shortened and are preempted,
    on the HIP kernels with captured decode steps (the reference's engine test runs its
    schedules against the model too, tests/test_engine_paged.py:33-71; the decisions
    themselves are tested on the CPU). float32 tokens equal the plain run's; bfloat16 tokens
    wherever the choice is clear."""
    from socrates_amd.engine import Engine
    folder = write_tiny(tmp_path / "B", TINY_B, seed=4)
    cfg, w = plain.read_folder(folder, torch.float64)
    prompts = random_prompts([5, 17, 33, 9, 24, 40, 1, 12], cfg["vocab_size"], seed=1)
    # four requests of two pages each that outgrow a pool of six pages while they decode
    prompts += random_prompts([15, 15, 14, 13], cfg["vocab_size"], seed=8)
    n_new = 12
    want = [plain.greedy(cfg, w, p, n_new) for p in prompts]
    preempted = 0
    for num_blocks, chunk, picks in ((13, 7, range(8)), (7, 5, range(8)), (4, 64, (7, 3)), (6, 64, range(8, 12))):
        engine = Engine(str(folder), dtype=dtype, max_batch=4, max_len=64, max_new_tokens=n_new, block_size=8,
                        num_blocks=num_blocks, chunk=chunk, compile=True)
        got = engine.generate([prompts[i] for i in picks], max_new_tokens=n_new)
        if dtype == torch.float32:
            assert got == [want[i] for i in picks], (num_blocks, chunk)
        else:
            checked = [assert_same_where_clear(cfg, w, prompts[i], want[i], g) for i, g in zip(picks, got)]
            assert sum(checked) >= 8, checked
        engine.cache.check()
        assert engine.cache.n_free_pages == num_blocks and not engine.cache.open_rows
        assert engine.runner._graphs                      # decode-only steps were replayed from graphs
        preempted += engine.scheduler.n_preemptions
        if num_blocks in (4, 6):
            assert engine.scheduler.n_preemptions > 0
    assert preempted >= 3
