"""Another architecture, added from this file alone: a configuration class with keys of its
own, a plan whose layers differ (one with a window, feed-forwards of different sizes, one layer
in an arrangement of its own and a norm of its own that this file registers, tensor names of
its own, an untied head), registered under its name. From there on everything is
the framework's: the random-weights folder, the loader, the cache groups (the windowed layer
gets pages of its own and gives them back), the step function with captured decode steps,
and generation through ``Engine``. The oracle is put together from the plain implementation's
functions, layer by layer, over whole sequences."""

import json
from dataclasses import dataclass
from typing import Tuple

import pytest
import torch

import plain_qwen3 as plain
from helpers import make_runner, random_prompts

DEV = "cuda:0"
# the torch stand-in for the kernels on the CPU, the HIP kernels in both precisions on the GPU
KINDS = [pytest.param("torch", torch.float32, id="cpu-fp32"),
         pytest.param("hip", torch.float32, id="gpu-fp32", marks=pytest.mark.gpu),
         pytest.param("hip", torch.bfloat16, id="gpu-bf16", marks=pytest.mark.gpu)]
# the tolerances and the weights' scale of the replay tests
TOL = {torch.float32: dict(atol=1e-4, rtol=1e-4), torch.bfloat16: dict(atol=6e-2, rtol=5e-2)}


class ParallelBlock:
    """An arrangement from outside: y = x + mixer(norm1(x)) + ffn(norm1(x)). Like every block it
    gets the float32 residual stream and the previous block's output not yet added to it, and
    returns its own output un-added; the second norm of the spec is not used."""

    def __init__(self, spec, weights, ops):
        from socrates_amd.parts.registry import build_part, tensors_of

        def sub(role):
            part = getattr(spec, role)
            return build_part(part, {name: weights[f"{spec.name_of(role)}.{name}"] for name in tensors_of(part)}, ops)
        self.norm1, self.mixer, self.ffn = sub("norm1"), sub("mixer"), sub("ffn")

    def forward(self, residual, pending, ctx, slot, write=True):
        h = self.norm1.add_norm(residual, pending)
        both = (self.mixer.forward(h, ctx, slot, write), self.ffn.forward(h, ctx))
        # either may come as float32 partial sums [S, N, d]; so does what this block returns,
        # and the norm that runs next adds them to the residual stream in order
        return torch.cat([t if t.dim() == 3 else t.float().unsqueeze(0) for t in both])


@dataclass(frozen=True)
class CenterNormSpec:
    """y = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias over the last ``dim`` elements."""
    dim: int
    eps: float


class CenterNorm:
    """A norm from outside, written with library routines: it has no ``fusable``, so the blocks
    around it run product, sum and norm one after the other."""

    @staticmethod
    def tensors(spec):
        from socrates_amd.parts.registry import TensorDecl
        return {"weight": TensorDecl((spec.dim,), "vector"), "bias": TensorDecl((spec.dim,), "vector")}

    def __init__(self, spec, tensors, ops):
        self.spec, self.ops, self.weight, self.bias = spec, ops, tensors["weight"], tensors["bias"]

    def add_norm(self, residual, delta, rows=None):
        if delta is not None:
            delta = delta.sum(0) if delta.dim() == 3 else delta.float()
        if rows is None:
            if delta is not None:
                residual += delta
            h = residual
        else:
            h = residual[rows.long()] + (delta[rows.long()] if delta is not None else 0)
        return self(h)

    def __call__(self, x):
        y = torch.nn.functional.layer_norm(x.float(), (self.spec.dim,), self.weight, self.bias, self.spec.eps)
        return y.to(self.ops.dtype)


@dataclass(frozen=True)
class HybridConfig:
    """config.json of the toy: ``windows[i]`` 0 means that layer i sees every key; layers
    listed in ``parallel`` run mixer and feed-forward side by side."""
    vocab: int
    width: int
    heads: int
    kv_heads: int
    head_size: int
    ff_sizes: Tuple[int, ...]
    windows: Tuple[int, ...]
    parallel: Tuple[int, ...]
    eps: float
    theta: float

    @classmethod
    def from_dict(cls, d):
        return cls(d["vocab"], d["width"], d["heads"], d["kv_heads"], d["head_size"], tuple(d["ff_sizes"]),
                   tuple(d["windows"]), tuple(d["parallel"]), float(d["eps"]), float(d["theta"]))

    def to_dict(self):
        return dict(architectures=["ToyHybridLM"], vocab=self.vocab, width=self.width, heads=self.heads,
                    kv_heads=self.kv_heads, head_size=self.head_size, ff_sizes=list(self.ff_sizes),
                    windows=list(self.windows), parallel=list(self.parallel), eps=self.eps, theta=self.theta)

    def plan(self):
        from socrates_amd.config.specs import (AttentionSpec, BlockSpec, ModelPlan, RMSNormSpec, RopeSpec,
                                               SwiGLUSpec, default_order)
        norm, centred = RMSNormSpec(self.width, self.eps), CenterNormSpec(self.width, self.eps)
        layers = tuple(
            BlockSpec(mixer=AttentionSpec(hidden=self.width, n_heads=self.heads, n_kv_heads=self.kv_heads,
                                          head_dim=self.head_size, scale=self.head_size ** -0.5,
                                          qk_norm=RMSNormSpec(self.head_size, self.eps),
                                          position=RopeSpec(self.head_size, self.theta), window=w or None),
                      ffn=SwiGLUSpec(self.width, ff), norm1=centred if i in self.parallel else norm, norm2=norm,
                      prefix=f"blocks.{i}.",
                      names=(("norm1", "ln_a"), ("mixer", "attn"), ("norm2", "ln_b"), ("ffn", "ff")),
                      arrangement="parallel" if i in self.parallel else "prenorm")
            for i, (ff, w) in enumerate(zip(self.ff_sizes, self.windows)))
        return ModelPlan(architecture="ToyHybridLM", vocab_size=self.vocab, hidden=self.width, layers=layers,
                         order=default_order(len(layers)), final_norm=centred, embedding_name="tok.weight",
                         final_norm_prefix="ln_out", head_name="out.weight")


TOY = HybridConfig(vocab=301, width=96, heads=6, kv_heads=2, head_size=32, ff_sizes=(136, 72, 200),
                   windows=(0, 7, 0), parallel=(2,), eps=3e-6, theta=5e4)


def oracle(cfg, w, ids, rows):
    """Logits at ``rows`` of the whole sequence, from the plain implementation's parts."""
    ids = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(len(ids))
    part = dict(num_attention_heads=cfg["heads"], num_key_value_heads=cfg["kv_heads"], head_dim=cfg["head_size"],
                rms_norm_eps=cfg["eps"], rope_theta=cfg["theta"])
    x = w["tok.weight"][ids]
    for i, window in enumerate(cfg["windows"]):
        p = f"blocks.{i}."
        if i in cfg["parallel"]:
            h = torch.nn.functional.layer_norm(x, (cfg["width"],), w[p + "ln_a.weight"], w[p + "ln_a.bias"], cfg["eps"])
        else:
            h = plain.rms_norm(x, w[p + "ln_a.weight"], cfg["eps"])
        x = x + plain.attention_layer(h, w, p + "attn.", part, positions, window or None)
        if i not in cfg["parallel"]:
            h = plain.rms_norm(x, w[p + "ln_b.weight"], cfg["eps"])
        x = x + plain.swiglu_mlp(h, w, p + "ff.")
    x = torch.nn.functional.layer_norm(x[torch.as_tensor(rows)], (cfg["width"],), w["ln_out.weight"],
                                       w["ln_out.bias"], cfg["eps"])
    return x @ w["out.weight"].T


def register():
    """All that the framework has to be told."""
    from socrates_amd.config import register_architecture
    from socrates_amd.parts import register_part
    from socrates_amd.parts.block import register_arrangement
    register_architecture("ToyHybridLM", HybridConfig)
    register_arrangement("parallel", ParallelBlock)
    register_part(CenterNormSpec, CenterNorm)


@pytest.fixture(scope="module")
def toy_folder(tmp_path_factory):
    from socrates_amd.config import load_config
    from socrates_amd.weights import write_random_model
    register()
    folder = write_random_model(tmp_path_factory.mktemp("hybrid") / "m", TOY, 9, dtype=torch.bfloat16,
                                std=0.05, gain_std=0.1)
    assert json.loads((folder / "config.json").read_text())["windows"] == [0, 7, 0]
    assert load_config(folder) == TOY
    cfg, w = plain.read_folder(folder)
    return folder, cfg, w


@pytest.mark.parametrize("kind,dtype", KINDS)
def test_portions_and_decode_of_the_new_architecture(toy_folder, kind, dtype):
    """Two requests: prompts in portions of changing size beside each other, then decoded
    tokens one by one (through captured graphs on the GPU); every logit against the oracle.
    The windowed layer is a cache group of its own whose pages come back while the request
    is alive."""
    from socrates_amd.engine import StepEntry
    folder, cfg, w = toy_folder
    if kind == "hip":
        from socrates_amd.kernels import HipKernels
        ops = HipKernels(dtype, DEV)
    else:
        from torch_kernels import TorchKernels
        ops = TorchKernels(dtype, "cpu")
    a, b = random_prompts([45, 30], cfg["vocab"], seed=3)
    runner = make_runner(folder, ops, max_rows=2, max_len=64, block_size=4)
    groups = runner.cache.groups
    assert sorted(g.need.window or 0 for g in groups) == [0, 7]
    assert [len(g.pools) for g in groups if not g.need.window] == [2]       # the two layers that see every key share a group
    if kind == "hip":
        runner.enable_graphs(2)
    ra, rb = runner.cache.open_row(), runner.cache.open_row()
    want_a, want_b = oracle(cfg, w, a, list(range(45))), oracle(cfg, w, b, list(range(30)))

    def check(got, want, what):
        tol = TOL[dtype]
        torch.testing.assert_close(got.float().cpu(), want, msg=lambda m: f"{what}: {m}", **tol)

    cuts_a, cuts_b = [(0, 17), (17, 19), (19, 33)], [(0, 2), (2, 20), (20, 22)]
    for (a0, a1), (b0, b1) in zip(cuts_a, cuts_b):
        got = runner.step([StepEntry(ra, a[a0:a1], list(range(a1 - a0))), StepEntry(rb, b[b0:b1], list(range(b1 - b0)))])
        check(got[:a1 - a0], want_a[a0:a1], f"a[{a0}:{a1}]")
        check(got[a1 - a0:], want_b[b0:b1], f"b[{b0}:{b1}]")
    windowed = next(g for g in groups if g.need.window)
    full = next(g for g in groups if not g.need.window)
    assert len(windowed.held_by(ra)) < len(full.held_by(ra))           # pages behind the window went back
    for t in range(8):
        got = runner.step([StepEntry(ra, [a[33 + t]], [0]), StepEntry(rb, [b[22 + t]], [0])])
        check(got[0], want_a[33 + t], f"a, decoded at {33 + t}")
        check(got[1], want_b[22 + t], f"b, decoded at {22 + t}")
    assert kind != "hip" or runner._graphs                              # the decode steps were captured ones
    runner.cache.close_row(ra)
    runner.cache.close_row(rb)
    assert not runner.cache.open_rows


@pytest.mark.gpu
def test_greedy_generation_of_the_new_architecture_through_the_engine(toy_folder):
    """``Engine(folder)`` finds the architecture by its name; float32 tokens are the oracle's."""
    from socrates_amd.engine import Engine
    folder, cfg, w = toy_folder
    prompts = random_prompts([11, 4, 19], cfg["vocab"], seed=4)
    engine = Engine(str(folder), device=DEV, dtype=torch.float32, max_batch=4, max_len=64, block_size=4)
    got = engine.generate(prompts, max_new_tokens=9)
    for prompt, out in zip(prompts, got):
        seq = list(prompt)
        for _ in range(9):
            seq.append(int(oracle(cfg, w, seq, [len(seq) - 1])[0].argmax()))
        assert out == seq[len(prompt):]


@pytest.mark.gpu
def test_the_replay_program_serves_it_as_a_plug_in(toy_folder, tmp_path):
    """``bin/trace_run`` in a process of its own knows nothing of the toy until the module
    named in SOCRATES_AMD_PLUGINS registers it; then the folder's config.json chooses it as
    it chooses any architecture, and the logits are the oracle's."""
    import os
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    folder, cfg, w = toy_folder
    root = Path(__file__).resolve().parent.parent
    (tmp_path / "toy_plugin.py").write_text("import test_another_architecture\ntest_another_architecture.register()\n")
    (prompt,) = random_prompts([21], cfg["vocab"], seed=6)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:13], "want": [0, 12]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[13:], "want": list(range(8))}], "end": ["a"]}]
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([str(tmp_path), str(Path(__file__).resolve().parent),
                                                       os.environ.get("PYTHONPATH", "")]))
    cmd = [sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32",
           "--out", str(tmp_path / "out"), "--max-tokens", "64"]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    unknown = subprocess.run(cmd, input=text, capture_output=True, text=True, env=env, timeout=300)
    assert unknown.returncode != 0 and "unknown architecture 'ToyHybridLM'" in unknown.stderr
    proc = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=300,
                          env=dict(env, SOCRATES_AMD_PLUGINS="toy_plugin"))
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == ["done", "0", "done", "1"]
    want = oracle(cfg, w, prompt, [0, 12] + list(range(13, 21)))
    got = np.concatenate([np.fromfile(tmp_path / "out" / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for i in (0, 1)])
    torch.testing.assert_close(torch.from_numpy(got), want, **TOL[torch.float32])
