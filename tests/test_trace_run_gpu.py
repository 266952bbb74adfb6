"""bin/trace_run as a user runs it: a subprocess fed JSON steps on standard input, logits
read back from <step>.f32 files and compared with the plain implementation. One trace holds
the same requests cut four ways: whole; most in one step and the last 32 tokens one by one;
portions of changing size; mixed with other requests in a pool so small that pages are
used again."""

import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
from helpers import (TINY_A, TINY_B, random_prompts, trace_mixed, trace_portions, trace_tail_decode,
                     trace_whole, write_tiny)

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]
TOL = {"float32": dict(atol=1e-4, rtol=1e-4), "bfloat16": dict(atol=6e-2, rtol=5e-2)}


def build_trace(prompts):
    """[(tag, steps)] -> one list of JSON steps with request ids made unique per cut."""
    cuts = [("whole", trace_whole(prompts)), ("tail", trace_tail_decode(prompts, 32)),
            ("portions", trace_portions(prompts, seed=3)), ("mixed", trace_mixed(prompts, seed=4))]
    lines, wanted = [], []          # wanted: (step number, [(request key, positions)])
    step = 0
    for tag, steps in cuts:
        fed = {}
        for entries, ends in steps:
            msg = {"step": step, "entries": [], "end": [f"{tag}-{r}" for r in ends]}
            here = []
            for rid, tokens, want in entries:
                msg["entries"].append({"id": f"{tag}-{rid}", "tokens": tokens, "want": want})
                start = fed.get(rid, 0)
                here.append((int(rid[1:]), [start + j for j in want]))
                fed[rid] = start + len(tokens)
            lines.append(json.dumps(msg))
            wanted.append((step, here))
            step += 1
    return lines, wanted


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tiny,seed,options", [(TINY_A, 1, []), (TINY_B, 2, []),
                                               (TINY_B, 2, ["--block-size", "8", "--max-rows", "4"])],
                         ids=["A", "B", "B-pages-of-8"])
def test_trace_run_matches_plain(tmp_path, tiny, seed, options, dtype):
    folder = write_tiny(tmp_path / "model", tiny, seed=seed)
    cfg, w = plain.read_folder(folder)
    prompts = random_prompts([5, 33, 70, 64, 100, 41], cfg["vocab_size"], seed=seed)
    oracle = [plain.forward(cfg, w, p) for p in prompts]
    lines, wanted = build_trace(prompts)
    # the four longest requests, each rounded up to 64 tokens: pages are used again
    max_tokens = sum(-(-len(p) // 64) * 64 for p in sorted(prompts, key=len)[-4:])
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(max_tokens)] + options,
                          input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {i}" for i in range(len(lines))]
    V = cfg["vocab_size"]
    for step, here in wanted:
        n = sum(len(pos) for _, pos in here)
        path = out / f"{step}.f32"
        if n == 0:
            assert not path.exists()
            continue
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(n, V).copy())
        want = torch.cat([oracle[i][pos] for i, pos in here])
        torch.testing.assert_close(got, want, **TOL[dtype], msg=lambda m: f"step {step}: {m}")


def test_trace_run_reports_a_bad_line(tmp_path):
    folder = write_tiny(tmp_path / "model", TINY_A, seed=1)
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype",
                           "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                          input='{"step": 0, "entries": [{"id": "a", "tokens": [1, 2], "want": [1]}], "end": []}\nnot json\n',
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 2 and "done 0" in proc.stdout and "line 2" in proc.stderr
