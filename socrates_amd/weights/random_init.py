"""Seeded random weights: in memory, or written as a model folder.

The reference's tests draw every parameter from one seeded generator with
non-trivial norm gains (tests/tiny.py:24-32). Here: matrices N(0, std), gains
1 + N(0, gain_std), tensor by tensor in the order of ``expected`` so that a seed
fixes every value; a folder written this way (config.json + model.safetensors)
loads like any other.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors.torch import save_file


def random_tensors(expected, seed: int, dtype=torch.bfloat16, device="cpu",
                   std: float = 0.02, gain_std: float = 0.01):
    """{name: tensor} for ``expected`` ({name: TensorDecl}); vectors are float32 gains
    near one, matrices have ``dtype``."""
    gen = torch.Generator(device=device).manual_seed(seed)
    out = {}
    for name, decl in expected.items():
        if decl.kind == "vector":
            t = 1.0 + gain_std * torch.randn(decl.shape, generator=gen, device=device,
                                             dtype=torch.float32)
            out[name] = t
        elif decl.kind == "int":
            out[name] = torch.zeros(decl.shape, dtype=torch.int32, device=device)
        else:
            # drawn in float32 then rounded, so a bfloat16 and a float32 folder of one
            # seed hold the same values up to that rounding
            t = torch.empty(decl.shape, device=device, dtype=torch.float32)
            t.normal_(0.0, std, generator=gen)
            out[name] = t.to(dtype)
    return out


def write_random_model(folder, config, seed: int, dtype=torch.bfloat16,
                       std: float = 0.02, gain_std: float = 0.01):
    """Write ``folder/config.json`` and ``folder/model.safetensors`` for ``config``
    (a typed configuration with ``to_dict()`` and ``plan()``). Gains are stored in
    ``dtype`` too, as checkpoints of this architecture do."""
    from ..parts import expected_tensors

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    expected = expected_tensors(config.plan())
    tensors = random_tensors(expected, seed, dtype=dtype, device="cpu", std=std, gain_std=gain_std)
    tensors = {n: t.to(dtype).contiguous() if t.is_floating_point() else t
               for n, t in tensors.items()}
    (folder / "config.json").write_text(json.dumps(config.to_dict(), indent=2))
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
