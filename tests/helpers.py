"""Tiny configurations and trace helpers shared by the tests."""

import random

import torch

from socrates_amd.cache import CacheManager
from socrates_amd.config import Qwen3Config
from socrates_amd.engine import ModelRunner, StepEntry
from socrates_amd.parts import DecoderModel, cache_needs, expected_tensors
from socrates_amd.weights import load_weights, write_random_model

# Two configurations that differ in every size and option: head counts and groups, a
# head size decoupled from the width, sizes that are no power of two, number of
# layers, vocabulary, eps, theta, tied or separate head, and the cache's block size.
TINY_A = dict(cfg=dict(architectures=["Qwen3ForCausalLM"], vocab_size=256, hidden_size=64,
                       num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                       head_dim=16, intermediate_size=128, rms_norm_eps=1e-6, rope_theta=10000.0,
                       tie_word_embeddings=True),
              block_size=16, gain_std=0.01)
TINY_B = dict(cfg=dict(architectures=["Qwen3ForCausalLM"], vocab_size=384, hidden_size=96,
                       num_hidden_layers=3, num_attention_heads=8, num_key_value_heads=2,
                       head_dim=32, intermediate_size=160, rms_norm_eps=1e-5, rope_theta=1e6,
                       tie_word_embeddings=False),
              block_size=8, gain_std=0.2)
# A third one with awkward sizes: three kv heads with three query heads each, head size 48,
# odd widths. It differs from A and from B in every size and option.
TINY_C = dict(cfg=dict(architectures=["Qwen3ForCausalLM"], vocab_size=331, hidden_size=72,
                       num_hidden_layers=4, num_attention_heads=9, num_key_value_heads=3,
                       head_dim=48, intermediate_size=200, rms_norm_eps=3e-6, rope_theta=50000.0,
                       tie_word_embeddings=True),
              block_size=4, gain_std=0.1)

# A fourth with the head size of real checkpoints' small models (64: the kernels' 32-element
# product steps, the wide rotation kernel) and one kv head for eight query heads.
TINY_D = dict(cfg=dict(architectures=["Qwen3ForCausalLM"], vocab_size=500, hidden_size=128,
                       num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=1,
                       head_dim=64, intermediate_size=192, rms_norm_eps=1e-6, rope_theta=1e5,
                       tie_word_embeddings=False),
              block_size=32, gain_std=0.05)

TINIES = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def write_tiny(folder, tiny, seed, dtype=torch.bfloat16, std=0.05):
    """A model folder with weights large enough that attention is far from uniform."""
    config = Qwen3Config.from_dict(tiny["cfg"])
    return write_random_model(folder, config, seed, dtype=dtype, std=std, gain_std=tiny["gain_std"])


def make_runner(folder, ops, max_rows=4, max_len=512, block_size=16, num_blocks=None):
    """A ModelRunner over ``folder`` with the given kernel set (HIP or the torch stand-in)."""
    from socrates_amd.config import load_config
    config = load_config(folder)
    plan = config.plan()
    weights = load_weights(folder, expected_tensors(plan), ops.dtype, ops.device)
    model = DecoderModel(plan, weights, ops)
    if num_blocks is None:
        num_blocks = max_rows * ((max_len + block_size - 1) // block_size)
    cache = CacheManager(cache_needs(plan), max_rows=max_rows, max_len=max_len,
                         block_size=block_size, num_blocks=num_blocks, dtype=ops.dtype,
                         device=ops.device)
    return ModelRunner(model, cache)


def random_prompts(lengths, vocab, seed):
    rng = random.Random(seed)
    return [[rng.randrange(vocab) for _ in range(n)] for n in lengths]


# ---- ways of cutting requests into steps ---------------------------------------------------
# A trace is a list of steps; a step is (entries, ends) with entries = [(id, tokens, want)].

def trace_whole(prompts):
    """Each request alone, whole, every logit wanted."""
    return [([(f"r{i}", p, list(range(len(p))))], [f"r{i}"]) for i, p in enumerate(prompts)]


def trace_tail_decode(prompts, tail=32):
    """Most of each request in one step, the last ``tail`` tokens one by one."""
    steps = []
    for i, p in enumerate(prompts):
        head = max(len(p) - tail, 1)
        steps.append(([(f"r{i}", p[:head], list(range(head)))], []))
        for t in range(head, len(p)):
            steps.append(([(f"r{i}", p[t:t + 1], [0])], []))
        steps[-1] = (steps[-1][0], [f"r{i}"])
    return steps


def trace_portions(prompts, seed, sizes=(2, 3, 5, 7, 16, 17, 33)):
    """Each request alone in portions of changing size, down to two tokens."""
    rng = random.Random(seed)
    steps = []
    for i, p in enumerate(prompts):
        t = 0
        while t < len(p):
            n = min(rng.choice(sizes), len(p) - t)
            steps.append(([(f"r{i}", p[t:t + n], list(range(n)))], []))
            t += n
        steps[-1] = (steps[-1][0], [f"r{i}"])
    return steps


def trace_mixed(prompts, seed, max_live=4, prefill_frac=0.6):
    """Up to ``max_live`` requests at once: portions of some beside single tokens of
    others; a request may sit out a step; finished ones end so their pages come back."""
    rng = random.Random(seed)
    waiting = list(range(len(prompts)))
    live, done_at = {}, {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.7):
            live[waiting.pop(0)] = 0
        entries, ends = [], []
        for i in list(live):
            if len(live) > 1 and rng.random() < 0.2:
                continue                                    # sits this step out
            p, t = prompts[i], live[i]
            cut = int(len(p) * prefill_frac)
            if t < cut:
                n = min(rng.choice((2, 3, 5, 8, 13, 21)), cut - t)
            else:
                n = 1
            n = min(n, len(p) - t)
            entries.append((f"r{i}", p[t:t + n], list(range(n))))
            live[i] = t + n
            if live[i] == len(p):
                ends.append(f"r{i}")
                del live[i]
        if entries:
            steps.append((entries, ends))
    return steps


def replay(runner, steps):
    """Run a trace through a ModelRunner. Returns {request id: logits [T, V]} on the CPU."""
    rows, got = {}, {}
    for entries, ends in steps:
        batch = []
        for rid, tokens, want in entries:
            if rid not in rows:
                rows[rid] = runner.cache.open_row()
            batch.append(StepEntry(rows[rid], tokens, want))
        logits = runner.step(batch).float().cpu()
        o = 0
        for rid, tokens, want in entries:
            got.setdefault(rid, []).append(logits[o:o + len(want)])
            o += len(want)
        for rid in ends:
            runner.cache.close_row(rows.pop(rid))
        runner.cache.check()
    return {rid: torch.cat(parts) for rid, parts in got.items()}


def captured_decode_beside_a_long_prompt(runner, short, long_, want_short, want_long, close, first_decoded):
    """A short request's decode step is captured for a small context bucket; then a prompt
    that reaches far beyond it runs eagerly in portions, with other allocations between
    the steps (whatever a captured step reads by address and a long step replaced would be
    handed out again here); then the short request replays the step captured first.
    ``want_*``: the plain implementation's logits for every position of the two requests;
    ``close(got, want, what)`` compares. Every logit the engine computes is compared."""
    import torch
    from socrates_amd.engine import StepEntry
    dev = runner.ops.device
    a = runner.cache.open_row()
    n = len(short)
    mid = first_decoded + (n - first_decoded) // 2
    got = runner.step([StepEntry(a, short[:first_decoded], [first_decoded - 1])]).float().cpu()
    close(got[0], want_short[first_decoded - 1], "short request, end of its prompt")
    for t in range(first_decoded, mid):
        got = runner.step([StepEntry(a, short[t:t + 1], [0])]).float().cpu()
        close(got[0], want_short[t], f"short request, decoded position {t} (first capture)")
    bucket = runner._context_bucket(mid)
    held = runner._graphs[(1, bucket)][0]
    b = runner.cache.open_row()
    junk = []
    portion = (len(long_) + 2) // 3
    for start in range(0, len(long_), portion):
        tokens = long_[start:start + portion]
        got = runner.step([StepEntry(b, tokens, [0, len(tokens) - 1])]).float().cpu()
        close(got[0], want_long[start], f"long request, position {start}")
        close(got[1], want_long[start + len(tokens) - 1], f"long request, position {start + len(tokens) - 1}")
        # blocks of the sizes that tables and activations have, filled with what no cosine is
        junk = [torch.full((s,), 3.0e4, dtype=torch.float32, device=dev) for s in (1 << 15, 1 << 17, 1 << 18, 1 << 19)]
    del junk
    for t in range(mid, n - 2):
        got = runner.step([StepEntry(a, short[t:t + 1], [0])]).float().cpu()
        close(got[0], want_short[t], f"short request, decoded position {t} (replayed after the long prompt)")
    assert runner._graphs[(1, bucket)][0] is held, "the step captured first was not the one replayed"
    # both requests in one captured step, whose positions reach as far as the long request's
    c = runner.cache.open_row()
    runner.step([StepEntry(c, long_[:len(long_) - 1], [])])
    got = runner.step([StepEntry(a, short[n - 2:n - 1], [0]), StepEntry(c, long_[-1:], [0])]).float().cpu()
    close(got[0], want_short[n - 2], "short request beside the long one")
    close(got[1], want_long[len(long_) - 1], "long request, decoded last position")
    assert (2, runner._context_bucket(len(long_))) in runner._graphs
    junk = [torch.full((s,), 3.0e4, dtype=torch.float32, device=dev) for s in (1 << 15, 1 << 17, 1 << 18, 1 << 19)]
    # and the short one alone again, from the step captured first (unless the kernel set
    # said that it was stale: then from one captured anew)
    got = runner.step([StepEntry(a, short[n - 1:], [0])]).float().cpu()
    close(got[0], want_short[n - 1], "short request, last position, after a captured step that reached far")
    del junk
    for row in (a, b, c):
        runner.cache.close_row(row)
