"""Logits at the layer sizes the benchmark times: two layers with the widths of Qwen3-4B
(hidden 2,560, 32 query and 8 kv heads of 128, feed-forward 9,728, vocabulary 151,936, tied
head), seeded weights written as a folder that the plain implementation reads on the CPU.
The reference compares every logit of its model at every step (tests/test_paged_model.py:35-76);
here the same at real widths, where the decode products split K, the feed-forward's
activation sits in a product's epilogue, the head has 151,936 rows and the attention kernels
run with 32 / 8 heads of 128 and many key splits."""

import pytest
import torch

import plain_qwen3 as plain
from helpers import captured_decode_beside_a_long_prompt, make_runner, random_prompts

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# float32: 1e-4 of the logit scale (the reference's bound for whole-model logits); bfloat16 as
# in the replay tests
TOL = {torch.float32: dict(atol=4e-4, rtol=1e-4), torch.bfloat16: dict(atol=6e-2, rtol=5e-2)}
WIDE = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=2560, num_hidden_layers=2,
            num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=9728,
            rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True)


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    from socrates_amd.config import Qwen3Config
    from socrates_amd.weights import write_random_model
    folder = write_random_model(tmp_path_factory.mktemp("wide") / "m", Qwen3Config.from_dict(WIDE), 21,
                                dtype=torch.bfloat16, std=0.02, gain_std=0.1)
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts([300, 2200, 90, 500, 33], cfg["vocab_size"], seed=5)
    return folder, cfg, w, prompts


def close(got, want, dtype, what):
    tol = TOL[dtype]
    bad = (got - want).abs() > tol["atol"] + tol["rtol"] * want.abs()
    assert not bad.any(), (f"{what}: {int(bad.sum())} logits off, largest error "
                           f"{float((got - want).abs().max()):.3g} at scale {float(want.abs().max()):.3g}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_whole_prompt_then_captured_decode(wide, dtype):
    """A 300-token prompt: most of it in two steps, then its last 32 tokens one by one
    through captured graphs (one row: the skinny products with K splits, the SwiGLU epilogue,
    the float32-output head of 151,936 rows, decode attention with key splits)."""
    from socrates_amd.engine import StepEntry
    from socrates_amd.kernels import HipKernels
    folder, cfg, w, prompts = wide
    prompt = prompts[0]
    head_rows = [0, 1, 15, 16, 17, 100, 255, 256, 267]
    want = plain.forward(cfg, w, prompt, rows=head_rows + list(range(268, 300)))
    runner = make_runner(folder, HipKernels(dtype, DEV), max_rows=2, max_len=512, block_size=16)
    runner.enable_graphs(2)
    row = runner.cache.open_row()
    # 218 tokens in one step, then a portion of 50: in bfloat16 the two projections into the
    # residual sum of that step split K over sweeping workgroups (17 to 64 rows)
    first = [r for r in head_rows if r < 218]
    got = runner.step([StepEntry(row, prompt[:218], first)]).float().cpu()
    close(got, want[:len(first)], dtype, "the prompt's first 218 tokens in one step")
    got = runner.step([StepEntry(row, prompt[218:268], [r - 218 for r in head_rows[len(first):]])]).float().cpu()
    close(got, want[len(first):len(head_rows)], dtype, "the next 50 tokens in one step")
    for t in range(268, 300):
        logits = runner.step([StepEntry(row, prompt[t:t + 1], [0])]).float().cpu()
        close(logits[0], want[len(head_rows) + t - 268], dtype, f"decoded token at position {t}")
    assert list(runner._graphs) == [(1, 512)]           # every decoded token came from the one captured step
    runner.cache.close_row(row)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_long_portion_beside_decoded_tokens(wide, dtype):
    """A mixed step at real widths: a 2,100-token portion of one request (the eight-wave
    attention form, library or plain products of 2,100 rows) beside one decoded token of three
    other requests behind contexts of 89, 499 and 32 tokens, then the rest of the long request
    in a second mixed step."""
    from socrates_amd.engine import StepEntry
    from socrates_amd.kernels import HipKernels
    folder, cfg, w, prompts = wide
    ops = HipKernels(dtype, DEV)
    runner = make_runner(folder, ops, max_rows=4, max_len=2304, block_size=16)
    rows = {}
    for i in (2, 3, 4):                                   # everything but their last two tokens
        rows[i] = runner.cache.open_row()
        runner.step([StepEntry(rows[i], prompts[i][:-2], [])])
    rows[1] = runner.cache.open_row()
    long_prompt = prompts[1]
    wanted = {1: [0, 700, 2099, 2100, 2150, 2199], 2: [88, 89], 3: [498, 499], 4: [31, 32]}
    oracle = {i: plain.forward(cfg, w, prompts[i], rows=r) for i, r in wanted.items()}
    cuts = [(0, 2100, [0, 700, 2099]), (2100, 100, [0, 50, 99])]
    for j, (start, n, want_here) in enumerate(cuts):
        batch = [StepEntry(rows[2], [prompts[2][-2 + j]], [0]),
                 StepEntry(rows[1], long_prompt[start:start + n], want_here),
                 StepEntry(rows[3], [prompts[3][-2 + j]], [0]),
                 StepEntry(rows[4], [prompts[4][-2 + j]], [0])]
        logits = runner.step(batch).float().cpu()
        if dtype == torch.bfloat16 and j == 0:
            assert ops.last_attention_kernel == ("workgroup", 64)   # the long portion; the short ones by key splits
        close(logits[0], oracle[2][j], dtype, f"step {j}: decoded token of the 90-token request")
        close(logits[1:4], oracle[1][3 * j:3 * j + 3], dtype, f"step {j}: the long portion")
        close(logits[4], oracle[3][j], dtype, f"step {j}: decoded token of the 500-token request")
        close(logits[5], oracle[4][j], dtype, f"step {j}: decoded token of the 33-token request")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_captured_step_is_right_after_a_long_prompt(wide, dtype):
    """Head size 128, a cache of 4,096 tokens: the 90-token request's decode step is captured
    for contexts up to 256, the 2,200-token prompt then runs in three eager portions, and the
    step captured first is replayed (the reference's captured steps read module buffers that
    never move, model/qwen/qwen_kv_cont.py:97-127)."""
    from socrates_amd.kernels import HipKernels
    folder, cfg, w, prompts = wide
    short, long_ = prompts[2], prompts[1]
    want_short = plain.forward(cfg, w, short)
    want_long = plain.forward(cfg, w, long_, rows=[0, 733, 734, 1467, 1468, 2199])
    at = {0: 0, 733: 1, 734: 2, 1467: 3, 1468: 4, 2199: 5}

    class Rows:                      # the oracle's rows of the long request, by position
        def __getitem__(self, position):
            return want_long[at[position]]

    runner = make_runner(folder, HipKernels(dtype, DEV), max_rows=3, max_len=4096, block_size=16)
    runner.enable_graphs(2)
    captured_decode_beside_a_long_prompt(runner, short, long_, want_short, Rows(),
                                         lambda got, want, what: close(got, want, dtype, what), first_decoded=70)


# ---- the benchmark's own batch sizes -----------------------------------------------------------
# Lengths on both sides of a page (16), of a 256-key context bucket and of the split plans; the
# first 8, 16 and 24 of them each hold short and long ones.
BATCH_LENGTHS = [19, 262, 35, 130, 255, 50, 257, 18, 100, 270, 31, 258, 66, 20, 200, 34,
                 140, 259, 21, 36, 70, 256, 23, 260] + [24 + (7 * i) % 90 for i in range(40)]
DECODED = 3       # tokens of every request that are decoded, all rows in one step


def decode_rows_through_graphs(folder, cfg, w, prompts, want, dtype, live, expect_forms=()):
    """``live`` requests: their prompts but the last DECODED tokens in eager steps, then those
    tokens one per step, all rows in one captured step; every logit against ``want[i]``
    [DECODED, V]. Returns the kernel set (its ``forms`` say what was launched)."""
    from socrates_amd.engine import StepEntry
    from socrates_amd.kernels import HipKernels
    ops = HipKernels(dtype, DEV)
    runner = make_runner(folder, ops, max_rows=live, max_len=512, block_size=16)
    runner.enable_graphs(live)
    rows = [runner.cache.open_row() for _ in range(live)]
    for lo in range(0, live, 8):                                  # prompts, eight requests a step
        runner.step([StepEntry(rows[i], prompts[i][:-DECODED], []) for i in range(lo, min(lo + 8, live))])
    ops.forms.clear()
    for t in range(DECODED):
        batch = [StepEntry(rows[i], [prompts[i][len(prompts[i]) - DECODED + t]], [0]) for i in range(live)]
        logits = runner.step(batch).float().cpu()
        for i in range(live):
            close(logits[i], want[i][t], dtype,
                  f"{live} rows, step {t}, request {i} ({len(prompts[i])} tokens)")
    assert all(k[0] == runner._bucket(live) for k in runner._graphs) and runner._graphs
    for form in expect_forms:
        assert any(k.startswith(form) for k in ops.forms), (form, dict(ops.forms))
    return ops


@pytest.fixture(scope="module")
def wide_batch(wide):
    folder, cfg, w, _ = wide
    prompts = random_prompts(BATCH_LENGTHS, cfg["vocab_size"], seed=77)
    want = [plain.forward(cfg, w, p, rows=list(range(len(p) - DECODED, len(p)))) for p in prompts]
    return prompts, want


@pytest.mark.parametrize("live", [8, 16, 24, 64])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_every_logit_at_the_benchmarks_batch_sizes(wide, wide_batch, dtype, live):
    """The reference compares every logit of every step of its batched decode
    (tests/test_paged_model.py:35-76). 8 and 16 rows: the sweep form of QKV, gate / up and the
    head, the fused attention with key splits that meet in memory, rows handed on by tile, the
    two projections with the residual sum and the next norm in their epilogue, chained over
    both layers. 24 and 64 rows: the products with K outermost (QKV, gate / up with its activation,
    the head at 24 rows) from rows that the norm lays out by tile, beside the sweep over parts
    of K and, at 64 rows, the library's product for the head."""
    folder, cfg, w, _ = wide
    prompts, want = wide_batch
    forms = () if dtype == torch.float32 else \
        ("sweep", "sweep_swiglu", "add_norm", "fused_attention") if live <= 16 else \
        ("parts_of_k", "stream", "stream_swiglu", "fused_attention")
    ops = decode_rows_through_graphs(folder, cfg, w, prompts, want, dtype, live, forms)
    if dtype == torch.bfloat16 and live == 8:
        splits = [int(k.split(":")[1]) for k in ops.forms if k.startswith("fused_attention")]
        assert max(splits) > 4, dict(ops.forms)              # the key splits met in memory


# One or two layers at the widths of the larger models (random weights; a vocabulary of 8,192
# keeps the head in the sweep form at K = 4,096 and 5,120).
WIDER = {
    "8b": dict(architectures=["Qwen3ForCausalLM"], vocab_size=8192, hidden_size=4096, num_hidden_layers=2,
               num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288,
               rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False),
    "32b": dict(architectures=["Qwen3ForCausalLM"], vocab_size=8192, hidden_size=5120, num_hidden_layers=1,
                num_attention_heads=64, num_key_value_heads=8, head_dim=128, intermediate_size=25600,
                rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=False),
}


@pytest.fixture(scope="module", params=["8b", "32b"])
def wider(request, tmp_path_factory):
    from socrates_amd.config import Qwen3Config
    from socrates_amd.weights import write_random_model
    folder = write_random_model(tmp_path_factory.mktemp(request.param) / "m", Qwen3Config.from_dict(WIDER[request.param]),
                                31, dtype=torch.bfloat16, std=0.02, gain_std=0.1)
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts(BATCH_LENGTHS[:40], cfg["vocab_size"], seed=78)
    want = [plain.forward(cfg, w, p, rows=list(range(len(p) - DECODED, len(p)))) for p in prompts]
    return request.param, folder, cfg, w, prompts, want


@pytest.mark.parametrize("live", [1, 8, 40])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_layers_of_the_larger_models(wider, dtype, live):
    """Widths 4,096 (K of 4,096 and 12,288) and 5,120 with 64 query heads (K of 5,120 in two
    halves per wave, 8,192 into 5,120 outputs as 512 workgroups of 10 weight rows, and 25,600): decode steps of
    1, 8 and 40 rows through captured graphs, every logit against the plain implementation."""
    name, folder, cfg, w, prompts, want = wider
    forms = () if dtype == torch.float32 else \
        ("sweep", "sweep_swiglu", "add_norm", "fused_attention") if live <= 16 else ("parts_of_k", "fused_attention")
    ops = decode_rows_through_graphs(folder, cfg, w, prompts, want, dtype, live, forms)
    if dtype == torch.bfloat16 and live <= 16:
        assert any(k.startswith("add_norm") for k in ops.forms), dict(ops.forms)
