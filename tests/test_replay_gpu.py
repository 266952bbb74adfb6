"""The engine's step function on the GPU against the plain implementation, under every
way of cutting the same requests into steps, in float32 and in bfloat16."""

import pytest
import torch

import plain_qwen3 as plain
from helpers import (TINIES, make_runner, random_prompts, replay, trace_mixed, trace_portions,
                     trace_tail_decode, trace_whole, write_tiny)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# float32: the reference's own bound for whole-model logits (tests/test_paged_model.py: 1e-4).
# bfloat16: activations are rounded to 8 bits of mantissa between kernels; logits of size ~2
# come out within a few hundredths of the float32 oracle that uses the same weights.
TOL = {torch.float32: dict(atol=1e-4, rtol=1e-4), torch.bfloat16: dict(atol=6e-2, rtol=5e-2)}
LENGTHS = [5, 17, 33, 70, 64, 129]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("replay_models")
    return {name: write_tiny(base / name, tiny, seed=3 + i) for i, (name, tiny) in enumerate(TINIES.items())}


@pytest.fixture(scope="module")
def oracle(folders):
    out = {}
    for name, folder in folders.items():
        cfg, w = plain.read_folder(folder)
        prompts = random_prompts(LENGTHS, cfg["vocab_size"], seed=len(name))
        out[name] = (prompts, {f"r{i}": plain.forward(cfg, w, p) for i, p in enumerate(prompts)})
    return out


def runner_for(folder, tiny, dtype, num_blocks):
    from socrates_amd.kernels import HipKernels
    return make_runner(folder, HipKernels(dtype, DEV), max_rows=4, max_len=256,
                       block_size=tiny["block_size"], num_blocks=num_blocks)


def compare(got, want, dtype, label):
    tol = TOL[dtype]
    for rid in want:
        assert got[rid].shape == want[rid].shape, (label, rid)
        bad = ((got[rid] - want[rid]).abs() > tol["atol"] + tol["rtol"] * want[rid].abs()).any(dim=-1)
        if bad.any():
            first = int(bad.nonzero()[0])
            err = (got[rid][first] - want[rid][first]).abs().max().item()
            raise AssertionError(f"{label} request {rid}: {int(bad.sum())} of {len(bad)} positions are "
                                 f"off; the first is position {first} (max error {err:.3g})")


CUTS = {
    "whole": lambda prompts: trace_whole(prompts),
    "tail32": lambda prompts: trace_tail_decode(prompts, 32),
    "portions": lambda prompts: trace_portions(prompts, seed=1),
    "mixed": lambda prompts: trace_mixed(prompts, seed=2),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", list(TINIES))
def test_cut_matches_plain(folders, oracle, name, cut, dtype):
    prompts, want = oracle[name]
    bs = TINIES[name]["block_size"]
    # so few pages that finished requests' pages are used again: the four longest
    # requests together, rounded up to pages, and nothing more
    longest = sorted((len(p) for p in prompts), reverse=True)[:4]
    num_blocks = sum(-(-n // bs) for n in longest)
    runner = runner_for(folders[name], TINIES[name], dtype, num_blocks)
    got = replay(runner, CUTS[cut](prompts))
    compare(got, want, dtype, f"{name}/{cut}")
    assert runner.cache.n_free_pages == num_blocks and not runner.cache.open_rows


@pytest.mark.parametrize("name", list(TINIES))
def test_bf16_cuts_agree_with_each_other(folders, oracle, name):
    """Cutting changes only the order of a few float32 sums, so bfloat16 logits of the
    same position differ between cuts by a few bfloat16 roundings, far less than they
    differ from the float32 oracle."""
    prompts, _ = oracle[name]
    results = {}
    for cut in ("whole", "mixed"):
        runner = runner_for(folders[name], TINIES[name], torch.bfloat16, 64)
        results[cut] = replay(runner, CUTS[cut](prompts))
    for rid in results["whole"]:
        torch.testing.assert_close(results["mixed"][rid], results["whole"][rid], atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("name", list(TINIES))
def test_short_steps_with_the_norms_in_kernels_of_their_own(folders, oracle, name):
    """Steps of at most 16 tokens fold the residual sums and norms into the products around
    them; with that switched off the same steps run product, sum and norm one after the other.
    Both ways match the oracle, and agree with each other far more closely than with it; the
    arrival counts that workgroups meet through are back at zero afterwards."""
    prompts, want = oracle[name]
    results = {}
    for fused in (True, False):
        runner = runner_for(folders[name], TINIES[name], torch.bfloat16, 64)
        runner.ops.fuse_norms = fused
        results[fused] = replay(runner, trace_tail_decode(prompts, 32))
        compare(results[fused], want, torch.bfloat16, f"{name}/tail32/fused={fused}")
        assert int(runner.ops._split_count.abs().sum()) == 0
    for rid in results[True]:
        torch.testing.assert_close(results[True][rid], results[False][rid], atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_first_tokens_and_long_decode(folders, dtype):
    """The first tokens of a sequence one by one (positions 0, 1, 2 ...), then a long
    decode across many page edges."""
    cfg, w = plain.read_folder(folders["B"])
    prompt = random_prompts([200], cfg["vocab_size"], seed=9)[0]
    want = plain.forward(cfg, w, prompt)
    runner = runner_for(folders["B"], TINIES["B"], dtype, 32)
    steps = [([("r0", prompt[t:t + 1], [0])], []) for t in range(len(prompt))]
    got = replay(runner, steps)["r0"]
    torch.testing.assert_close(got, want, **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("hidden,inter", [(50, 300), (44, 24)])
def test_widths_that_are_no_multiple_of_eight(tmp_path, hidden, inter, dtype):
    """A width of 50 or 44: the bfloat16 products that read eight elements at a time do not
    apply, and a short step must not leave rows owed their norm to a product that cannot take
    them (it once did, and the step stopped with an error). Portions, then tokens one by one."""
    tiny = dict(cfg=dict(architectures=["Qwen3ForCausalLM"], vocab_size=211, hidden_size=hidden,
                         num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=32,
                         intermediate_size=inter, rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=True),
                block_size=8, gain_std=0.1)
    folder = write_tiny(tmp_path / "m", tiny, seed=hidden)
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts([40, 7, 70], cfg["vocab_size"], seed=2)
    want = {f"r{i}": plain.forward(cfg, w, p) for i, p in enumerate(prompts)}
    for steps in (trace_portions(prompts, seed=3), trace_tail_decode(prompts, 32)):
        runner = runner_for(folder, tiny, dtype, 40)
        compare(replay(runner, steps), want, dtype, f"hidden {hidden}")


@pytest.mark.parametrize("which", ["all", "some", "head"])
def test_matrices_stored_in_32_bit_under_a_bfloat16_run(tmp_path, which):
    """A file that holds all, some, or the first and last of its matrices in 32-bit floats: they
    stay so, and a bfloat16 run multiplies with them through the float32 product. Short steps
    must not hand such a product rows that are owed their norm (they once did, and the step
    stopped with an error). Mixed steps, then tokens one by one, against the plain run."""
    import random
    import warnings
    from safetensors.torch import load_file, save_file
    tiny = TINIES["B"]
    folder = write_tiny(tmp_path / "m", tiny, seed=9)
    tensors = load_file(str(folder / "model.safetensors"))
    rng = random.Random(3)
    for k in list(tensors):
        if tensors[k].dim() == 2 and (which == "all" or (which == "some" and rng.random() < 0.4) or
                                      (which == "head" and ("lm_head" in k or "embed" in k))):
            tensors[k] = tensors[k].float()
    save_file(tensors, str(folder / "model.safetensors"))
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts([5, 17, 40, 70], cfg["vocab_size"], seed=4)
    want = {f"r{i}": plain.forward(cfg, w, p) for i, p in enumerate(prompts)}
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")                     # "stored in 32-bit": known here
        runner = runner_for(folder, tiny, torch.bfloat16, 64)
    for steps in (trace_mixed(prompts, seed=1), trace_tail_decode(prompts, 32)):
        compare(replay(runner, steps), want, torch.bfloat16, f"{which} in 32-bit")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_captured_decode_steps_follow_the_data(folders, oracle, dtype):
    """Decode-only steps replayed from HIP graphs: every replay is compared with the plain
    oracle, with eager work (prompt portions, other widths, synchronisations) between the
    replays, rows joining and leaving, and widths that need padding rows."""
    prompts, want = oracle["B"]
    runner = runner_for(folders["B"], TINIES["B"], dtype, 80)
    runner.enable_graphs(4)
    steps = trace_mixed(prompts, seed=5, prefill_frac=0.3) + trace_tail_decode(prompts[:2], 40)
    decode_only = sum(all(len(t) == 1 for _, t, _ in entries) for entries, _ in steps)
    assert decode_only > 30
    got = replay(runner, steps)
    assert len(runner._graphs) >= 3                       # several widths were captured
    compare({k: v[-len(want[k]):] for k, v in got.items()}, want, dtype, "captured")
    # the same trace without graphs gives the same logits up to summation order
    eager = runner_for(folders["B"], TINIES["B"], dtype, 80)
    ref = replay(eager, steps)
    for rid in ref:
        torch.testing.assert_close(got[rid], ref[rid], **TOL[dtype])


def test_long_portion_beside_decoded_tokens_at_middle_size(tmp_path):
    """A step of a size at which the kernels for long prompts are chosen by themselves: a
    portion of 2,100 tokens (the eight-wave workgroup attention form, a wave per token in the
    rotation kernel, library products) beside one decoded token of three other requests (the
    per-wave attention kernel with key splits, in the same step), then shorter portions
    behind that context. Head size 64, eight query heads per kv head, bfloat16."""
    from socrates_amd.config import Qwen3Config
    from socrates_amd.kernels import HipKernels
    from socrates_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], vocab_size=1000, hidden_size=256, num_hidden_layers=2,
               num_attention_heads=16, num_key_value_heads=2, head_dim=64, intermediate_size=512,
               rms_norm_eps=1e-6, rope_theta=1e6, tie_word_embeddings=True)
    folder = write_random_model(tmp_path / "mid", Qwen3Config.from_dict(cfg), 11, dtype=torch.bfloat16, std=0.05, gain_std=0.05)
    pcfg, w = plain.read_folder(folder)
    prompts = random_prompts([2300, 300, 700, 40], pcfg["vocab_size"], seed=4)
    hip = HipKernels(torch.bfloat16, DEV)
    runner = make_runner(folder, hip, max_rows=4, max_len=2304, block_size=16)
    cuts = [2100, 184, 16]
    steps = [([(f"r{i}", prompts[i][:-len(cuts)], [])], []) for i in (1, 2, 3)]
    t = 0
    kernels = []
    got = {}
    rows = {}
    from socrates_amd.engine import StepEntry
    for entries, _ in steps:
        rid, toks, want = entries[0]
        rows[rid] = runner.cache.open_row()
        runner.step([StepEntry(rows[rid], toks, want)])
    rows["r0"] = runner.cache.open_row()
    long_want = {}
    for j, n in enumerate(cuts):
        want_here = sorted({0, n // 3, n - 1})
        batch = [StepEntry(rows[f"r{i}"], [prompts[i][len(prompts[i]) - len(cuts) + j]], [0]) for i in (1, 2, 3)]
        batch.insert(1, StepEntry(rows["r0"], prompts[0][t:t + n], want_here))
        logits = runner.step(batch).float().cpu()
        kernels.append(hip.last_attention_kernel)
        got[("r1", j)] = logits[0]
        for a, p in enumerate(want_here):
            long_want[t + p] = logits[1 + a]
        got[("r2", j)], got[("r3", j)] = logits[1 + len(want_here)], logits[2 + len(want_here)]
        t += n
    assert kernels[0] == ("workgroup", 64) and kernels[1][0] == "wave"
    tol = TOL[torch.bfloat16]
    ref = plain.forward(pcfg, w, prompts[0])
    for p, row in long_want.items():
        torch.testing.assert_close(row, ref[p], **tol)
    for i in (1, 2, 3):
        ref = plain.forward(pcfg, w, prompts[i])
        for j in range(len(cuts)):
            torch.testing.assert_close(got[(f"r{i}", j)], ref[len(prompts[i]) - len(cuts) + j], **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
@pytest.mark.parametrize("name,live,longest", [("B", 5, 120), ("B", 11, 400), ("D", 23, 120), ("D", 40, 400),
                                              ("C", 40, 300)])
def test_captured_steps_of_padded_widths_and_long_contexts(folders, name, live, longest, dtype):
    """Decode steps of 5, 11, 23 and 40 live rows replay the graphs of the width buckets 6,
    12, 24 and 48 (the padding rows use the null row), with contexts inside the 256-key bucket
    and beyond it. Every replay is compared with the plain implementation; between replays
    there is eager work (a portion of another request) and rows leave one by one, so the same
    graph is replayed with other rows, other lengths and more padding."""
    import random
    from socrates_amd.engine import StepEntry
    tiny = TINIES[name]
    cfg, w = plain.read_folder(folders[name])
    rng = random.Random(live)
    lengths = [longest] + [rng.randrange(12, longest) for _ in range(live - 1)]
    prompts = random_prompts(lengths, cfg["vocab_size"], seed=live)
    tail = 6
    want = [plain.forward(cfg, w, p)[-tail:] for p in prompts]
    from socrates_amd.kernels import HipKernels
    runner = make_runner(folders[name], HipKernels(dtype, DEV), max_rows=live + 1, max_len=512,
                         block_size=tiny["block_size"])
    runner.enable_graphs(64)
    rows = []
    for p in prompts:
        rows.append(runner.cache.open_row())
        runner.step([StepEntry(rows[-1], p[:-tail], [])])
    extra = runner.cache.open_row()
    extra_prompt = random_prompts([40], cfg["vocab_size"], seed=99)[0]
    extra_want = plain.forward(cfg, w, extra_prompt)
    alive = list(range(live))
    for t in range(tail):
        batch = [StepEntry(rows[i], [prompts[i][len(prompts[i]) - tail + t]], [0]) for i in alive]
        logits = runner.step(batch).float().cpu()
        for j, i in enumerate(alive):
            torch.testing.assert_close(logits[j], want[i][t], **TOL[dtype],
                                       msg=lambda m: f"step {t}, request {i} of {len(alive)} live: {m}")
        # eager work between the replays: a portion of another request, checked as well
        got = runner.step([StepEntry(extra, extra_prompt[6 * t:6 * t + 6], [5])]).float().cpu()
        torch.testing.assert_close(got[0], extra_want[6 * t + 5], **TOL[dtype])
        if t >= 2 and len(alive) > 2:
            runner.cache.close_row(rows[alive.pop(1)])    # a row leaves: same bucket, one more padding row
    widths = {k[0] for k in runner._graphs}
    contexts = {k[1] for k in runner._graphs}
    assert runner._bucket(live) in widths and runner._bucket(live) >= live
    assert (512 in contexts) == (longest > 256), (contexts, longest)
