"""The scheduler's decisions and the engine loop, on the CPU with the torch stand-in for
the kernels: admission, portions under a token budget, decode beside prefill, finishing
and freeing, and what happens when pages run out (wait, shorten, preempt and recompute)."""

import pytest
import torch

import plain_qwen3 as plain
from helpers import TINY_A, TINY_B, make_runner, random_prompts, write_tiny
from socrates_amd.cache import CacheManager
from socrates_amd.engine import Engine, QueueFull, Request, Scheduler, TooLong
from socrates_amd.parts import PagedKV
from socrates_amd.sampling import SamplingParams
from torch_kernels import TorchKernels, uniform_of


def sched(rows=4, max_len=64, bs=8, pages=8, budget=16, queue=6):
    cache = CacheManager([PagedKV(1, 16)], rows, max_len, bs, pages, torch.float32, "cpu")
    return Scheduler(cache, rows, max_len, budget, queue), cache


def req(n, max_new=4):
    return Request(prompt=None, ids=list(range(1, n + 1)), max_new_tokens=max_new)


def run_plan(s, cache, plan, token=7):
    """What the engine does with a plan, without a model: take pages, advance, append a token."""
    for p in plan:
        start = cache.length(p.request.row)
        cache.reserve(p.request.row, start + len(p.tokens))
        cache.advance(p.request.row, len(p.tokens))
        if p.wants_logits:
            p.request.output.append(token)
            if len(p.request.output) >= p.request.max_new_tokens:
                p.request.done = True
    cache.check()


def test_submit_limits():
    s, _ = sched(queue=2)
    with pytest.raises(TooLong):
        s.submit(req(61, 4))                    # 65 > max_len 64, as model/inference_paged.py:144-146
    s.submit(req(60, 4))
    s.submit(req(3))
    with pytest.raises(QueueFull):
        s.submit(req(3))
    small, _ = sched(pages=2)                   # the whole pool holds 16 tokens
    with pytest.raises(TooLong):
        small.submit(req(14, 4))
    with pytest.raises(ValueError):
        small.submit(Request(prompt=None, ids=[]))


def test_portions_under_a_budget_and_decode_beside_prefill():
    s, cache = sched(budget=16, pages=20, max_len=128)
    a, b = req(5), req(40, max_new=3)
    s.submit(a), s.submit(b)
    plan = s.plan()
    # a whole (5, wants logits) and the first 11 tokens of b (no logits yet)
    assert [(p.request, len(p.tokens), p.wants_logits) for p in plan] == [(a, 5, True), (b, 11, False)]
    assert plan[1].tokens == b.ids[:11]
    run_plan(s, cache, plan)
    plan = s.plan()
    # a decodes one token beside the next 15 of b
    assert [(p.request, len(p.tokens), p.wants_logits) for p in plan] == [(a, 1, True), (b, 15, False)]
    assert plan[0].tokens == [7]
    run_plan(s, cache, plan)
    plan = s.plan()
    assert [(len(p.tokens), p.wants_logits) for p in plan] == [(1, True), (14, True)]
    run_plan(s, cache, plan)
    while not s.idle:
        plan = s.plan()
        if plan:
            run_plan(s, cache, plan)
    assert len(a.output) == 4 and len(b.output) == 3 and a.row == b.row == -1
    assert cache.n_free_pages == 20 and not cache.open_rows


def test_admission_waits_for_rows_and_pages():
    s, cache = sched(rows=2, pages=4, budget=64)
    a, b, c = req(16, 1), req(9, 1), req(3, 1)
    for r in (a, b, c):
        s.submit(r)
    plan = s.plan()
    assert [p.request for p in plan] == [a, b] and list(s.pending) == [c]      # two rows only
    run_plan(s, cache, plan)
    plan = s.plan()                                                            # a and b are done: freed
    assert [p.request for p in plan] == [c] and cache.n_free_pages == 4
    # pages: a prompt that does not fit whole is shortened to the free pages
    s2, cache2 = sched(rows=3, pages=3, budget=64)
    x, y = req(17, 2), req(12, 2)
    s2.submit(x), s2.submit(y)
    plan = s2.plan()
    assert [(p.request, len(p.tokens)) for p in plan] == [(x, 17)]             # 3 pages: nothing left for y
    run_plan(s2, cache2, plan)
    assert [(p.request, len(p.tokens)) for p in s2.plan()] == [(x, 1)] and list(s2.pending) == [y]


def test_preempts_the_youngest_when_a_running_request_needs_a_page():
    s, cache = sched(rows=3, pages=4, budget=64, max_len=32)
    old, young = req(15, 8), req(15, 8)
    s.submit(old), s.submit(young)
    run_plan(s, cache, s.plan())                  # both prefilled: 2 + 2 pages, pool full
    assert cache.n_free_pages == 0
    run_plan(s, cache, s.plan())                  # token 16 of each still fits its second page
    plan = s.plan()                               # position 16 needs a third page each
    assert [p.request for p in plan] == [old]     # the older one goes on ...
    assert young.row == -1 and young.preemptions == 1 and s.pending[0] is young   # ... the younger is put back
    assert len(young.output) == 2                 # with its output kept
    run_plan(s, cache, plan)
    while not old.done:
        plan = s.plan()
        assert all(p.request is old for p in plan)    # nobody is admitted while the pool is short
        run_plan(s, cache, plan)
    plan = s.plan()                               # old retired: young comes back and recomputes
    assert [(p.request, len(p.tokens), p.wants_logits) for p in plan] == [(young, 17, True)]
    assert plan[0].tokens == young.ids + young.output
    assert cache.scalars.draws[young.row] == 2    # its random stream continues where it stopped
    run_plan(s, cache, plan)
    while not s.idle:
        run_plan(s, cache, s.plan())
    assert len(young.output) == 8 and cache.n_free_pages == 4 and s.n_preemptions == 1


def test_when_the_next_step_is_known_before_the_tokens():
    """``repeats``, asked as the engine asks it (the plan's step is queued, its tokens are not
    there yet): the step after a plan is one token for each of the same requests, whatever
    the plan's tokens are, only if every running request is in the plan and gets a token
    from it, none reaches its limit with that token, nobody who waits could be given a row,
    nobody is cancelled and the pages for one more token each are free. It changes nothing."""
    def queue(cache, plan):
        for p in plan:
            start = cache.length(p.request.row)
            cache.reserve(p.request.row, start + len(p.tokens))
            cache.advance(p.request.row, len(p.tokens))

    def tokens(plan, token=7):
        for p in plan:
            if p.wants_logits:
                p.request.output.append(token)
                p.request.done = len(p.request.output) >= p.request.max_new_tokens

    s, cache = sched(rows=2, pages=8, budget=16, bs=8)
    a, b = req(5, max_new=3), req(20, max_new=6)
    s.submit(a), s.submit(b)
    plan = s.plan()                             # a whole, 11 tokens of b: b gets no token yet
    queue(cache, plan)
    assert not s.repeats(plan)
    tokens(plan)
    plan = s.plan()                             # a decodes, b's last 9 tokens: both get a token
    queue(cache, plan)
    free = cache.free_pages()
    assert s.repeats(plan) and cache.free_pages() == free and len(s.running) == 2
    c = req(3)
    s.submit(c)                                 # both rows are taken: c cannot be admitted anyway
    assert s.repeats(plan)
    a.cancelled = True
    assert not s.repeats(plan)
    a.cancelled = False
    tokens(plan)                                # a has 2 of 3
    plan = s.plan()
    queue(cache, plan)
    assert len(a.output) == 2 and not s.repeats(plan)       # this step's token is a's last
    tokens(plan)
    assert a.done
    plan = s.plan()                             # a retired, c admitted beside b
    queue(cache, plan)
    assert [p.request for p in plan] == [b, c] and s.repeats(plan)
    # pages: two requests that fill the pool's two pages; the next token of the first needs a third
    s, cache = sched(rows=2, pages=2, budget=16, bs=8, max_len=16)
    a, b = req(8, max_new=8), req(7, max_new=8)
    s.submit(a), s.submit(b)
    plan = s.plan()
    assert [len(p.tokens) for p in plan] == [8, 7]
    queue(cache, plan)
    assert not s.repeats(plan)
    cache.check()


def test_cancelled_requests_are_dropped_and_freed():
    s, cache = sched(pages=8)
    a, b, c = req(9), req(9), req(9)
    for r in (a, b, c):
        s.submit(r)
    c.cancelled = True
    run_plan(s, cache, s.plan())
    assert c.row == -1 and c.event.is_set() and len(s.running) == 2
    a.cancelled = True
    plan = s.plan()
    assert [p.request for p in plan] == [b] and a.row == -1 and a.event.is_set()
    assert cache.n_free_pages == 8 - 1             # b holds one page (7 of its tokens so far)


@pytest.fixture(scope="module")
def tiny_b(tmp_path_factory):
    folder = write_tiny(tmp_path_factory.mktemp("sched") / "B", TINY_B, seed=4)
    cfg, w = plain.read_folder(folder, torch.float64)
    return folder, cfg, w


def engine_on_cpu(folder, num_blocks, chunk, max_batch=4, max_new=8, max_len=64):
    ops = TorchKernels(torch.float64, "cpu", acc=torch.float64)
    runner = make_runner(folder, ops, max_rows=max_batch, max_len=max_len, block_size=8, num_blocks=num_blocks)
    return Engine(runner, max_batch=max_batch, max_len=max_len, max_new_tokens=max_new, chunk=chunk,
                  compile=False)


def test_engine_tokens_do_not_depend_on_batching_or_pool_size(tiny_b):
    """tests/test_engine_paged.py:61-71 of the reference: batched == each alone, token for
    token (in float64, where argmax ties do not flip). Here also: with portions, and with a
    pool so small that requests wait and are preempted."""
    folder, cfg, w = tiny_b
    prompts = random_prompts([5, 17, 33, 9, 24, 40, 1, 12], cfg["vocab_size"], seed=1)
    want = [plain.greedy(cfg, w, p, 8) for p in prompts]
    for num_blocks, chunk in ((64, 2048), (64, 7), (13, 7), (7, 5)):
        engine = engine_on_cpu(folder, num_blocks, chunk)
        got = engine.generate(prompts, max_new_tokens=8)
        assert got == want, (num_blocks, chunk)
        engine.cache.check()
        assert engine.cache.n_free_pages == num_blocks and not engine.cache.open_rows
    alone = [engine_on_cpu(folder, 64, 2048, max_batch=1).generate([p], max_new_tokens=8)[0] for p in prompts[:3]]
    assert alone == want[:3]
    # two requests that fit at admission (2 + 2 pages of 4) and outgrow the pool while decoding:
    # the younger one is preempted, recomputed later, and still yields the same tokens
    engine = engine_on_cpu(folder, 4, 64)
    assert engine.generate([prompts[7], prompts[3]], max_new_tokens=8) == [want[7], want[3]]
    assert engine.scheduler.n_preemptions > 0 and engine.cache.n_free_pages == 4


def test_engine_stops_on_eos_and_counts(tiny_b):
    folder, cfg, w = tiny_b
    prompt = random_prompts([11], cfg["vocab_size"], seed=2)[0]
    full = plain.greedy(cfg, w, prompt, 8)
    engine = engine_on_cpu(folder, 64, 2048)
    stop = full[3]
    first = full.index(stop)
    r = engine.submit(prompt, sampling=SamplingParams(eos_token_ids=(stop,)), stream=True)
    engine.run()
    assert r.output == full[:first] and r.done                 # the stop token is not kept
    streamed = []
    while True:
        t = r.stream.get_nowait()
        if t is None:
            break
        streamed.append(t)
    assert streamed == r.output
    assert engine.prompt_tokens == 11 and engine.output_tokens == first
    assert r.submitted <= r.admitted <= r.first_token <= r.finished
    with pytest.raises(ValueError):
        engine.submit([cfg["vocab_size"]])
    with pytest.raises(ValueError):
        engine.submit("text without a tokenizer")


def test_temperature_sampling_is_seeded_and_batch_independent(tiny_b):
    folder, cfg, w = tiny_b
    prompts = random_prompts([9, 24, 40, 1], cfg["vocab_size"], seed=3)

    def expected(prompt, seed, n=6, T=0.8):
        ids, out = list(prompt), []
        for draw in range(n):
            logits = plain.forward(cfg, w, ids)[-1]
            cdf = torch.cumsum(torch.softmax(logits / T, -1), -1)
            tok = int(torch.searchsorted(cdf, torch.tensor(uniform_of(seed, draw) * float(cdf[-1]),
                                                           dtype=cdf.dtype), right=True))
            out.append(tok)
            ids.append(tok)
        return out

    want = [expected(p, 100 + i) for i, p in enumerate(prompts)]
    together = engine_on_cpu(folder, 64, 7).generate(prompts, max_new_tokens=6, temperature=0.8, seed=100)
    assert together == want
    squeezed = engine_on_cpu(folder, 9, 5)                      # waits and preemptions in between
    assert squeezed.generate(prompts, max_new_tokens=6, temperature=0.8, seed=100) == want
    other_seed = engine_on_cpu(folder, 64, 7).generate(prompts, max_new_tokens=6, temperature=0.8, seed=7)
    assert other_seed != want
