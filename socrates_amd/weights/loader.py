"""Weights from safetensors, by tensor name.

The reference reads every shard named in model.safetensors.index.json into one
dict and loads it strictly (model/qwen/qwen_kv_cont.py:35-42,
model/inference_paged.py:73-75): a missing or unexpected name raises. Here a
local folder holds either ``model.safetensors`` or an index with shards, names
are the ones on disk (no renaming), and everything that is wrong is reported in
one error: missing names, unexpected names and wrong shapes.

Kept dtypes: matrix operands in the compute dtype, except that a tensor stored in
32-bit floats stays 32-bit; gains and other vectors in float32 (exact from
bfloat16); integer tables as int32.
"""

from __future__ import annotations

import json
from pathlib import Path

import torch
from safetensors import safe_open


class WeightError(ValueError):
    """Lists every missing tensor, unexpected tensor and wrong shape at once."""

    def __init__(self, folder, missing, unexpected, wrong_shape, wrong_dtype=()):
        self.missing, self.unexpected = sorted(missing), sorted(unexpected)
        self.wrong_shape, self.wrong_dtype = list(wrong_shape), list(wrong_dtype)
        lines = [f"weights in {folder} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, got in self.wrong_shape:
            lines.append(f"  wrong shape: {name} expected {list(want)}, found {list(got)}")
        for name, got in self.wrong_dtype:
            lines.append(f"  wrong dtype: {name} is {got}")
        super().__init__("\n".join(lines))


def _files_of(folder: Path):
    """{tensor name: file} for a folder with one file or an index and shards."""
    single, index = folder / "model.safetensors", folder / "model.safetensors.index.json"
    if single.is_file():
        files = [single]
    elif index.is_file():
        shards = sorted(set(json.loads(index.read_text())["weight_map"].values()))
        files = [folder / s for s in shards]
        absent = [str(f) for f in files if not f.is_file()]
        if absent:
            raise FileNotFoundError(f"shards named by {index} are absent: {absent}")
    else:
        raise FileNotFoundError(f"{folder} holds neither model.safetensors nor model.safetensors.index.json")
    where = {}
    for f in files:
        with safe_open(str(f), framework="pt") as sf:
            for name in sf.keys():
                where[name] = f
    return where


_FLOATS = {"F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16}
_INTS = {"I64", "I32", "I16", "I8", "U8"}


def kept_dtype(kind: str, stored: str, compute_dtype):
    """The dtype a stored tensor is kept in; None if the stored dtype cannot serve."""
    if kind == "int":
        return torch.int32 if stored in _INTS else None
    if stored not in _FLOATS:
        return None
    if kind == "vector":
        return torch.float32
    if compute_dtype == torch.float32 or stored in ("F32", "F64"):
        return torch.float32
    return compute_dtype


def _same_stored(where, a, b) -> bool:
    """Whether the stored tensors ``a`` and ``b`` hold the same values in the same dtype."""
    with safe_open(str(where[a]), framework="pt") as fa, safe_open(str(where[b]), framework="pt") as fb:
        ta, tb = fa.get_tensor(a), fb.get_tensor(b)
    return ta.dtype == tb.dtype and ta.shape == tb.shape and torch.equal(ta, tb)


def load_weights(folder, expected, compute_dtype, device, duplicates=()):
    """Read the tensors named in ``expected`` ({name: TensorDecl}) from ``folder``.

    Returns {name: tensor on device}. Raises WeightError naming everything that
    does not fit. As under the reference's strict load, an ``lm_head.weight`` in
    the folder of a tied model is unexpected, unless ``duplicates`` ((stored name,
    expected name) pairs, ``ModelPlan.duplicates``) names it and it holds the very
    values of the embedding table; it is then not read.
    """
    folder = Path(folder)
    where = _files_of(folder)
    missing = [n for n in expected if n not in where]
    unexpected = [n for n in where if n not in expected]
    for stored, same_as in duplicates:
        if stored in unexpected and same_as in where and _same_stored(where, stored, same_as):
            unexpected.remove(stored)
    wrong_shape, wrong_dtype = [], []
    by_file = {}
    for name, decl in expected.items():
        if name in where:
            by_file.setdefault(where[name], []).append((name, decl))
    # First pass: shapes and dtypes only, nothing is read.
    for f, items in by_file.items():
        with safe_open(str(f), framework="pt") as sf:
            for name, decl in items:
                sl = sf.get_slice(name)
                shape = tuple(sl.get_shape())
                if shape != tuple(decl.shape):
                    wrong_shape.append((name, decl.shape, shape))
                if kept_dtype(decl.kind, sl.get_dtype(), compute_dtype) is None:
                    wrong_dtype.append((name, sl.get_dtype()))
    if missing or unexpected or wrong_shape or wrong_dtype:
        raise WeightError(folder, missing, unexpected, wrong_shape, wrong_dtype)
    out = {}
    kept_wide = []
    for f, items in by_file.items():
        with safe_open(str(f), framework="pt") as sf:
            for name, decl in items:
                stored = sf.get_slice(name).get_dtype()
                t = sf.get_tensor(name)
                dtype = kept_dtype(decl.kind, stored, compute_dtype)
                if decl.kind not in ("int", "vector") and dtype != compute_dtype:
                    kept_wide.append(name)
                out[name] = t.to(device=device, dtype=dtype).contiguous()
    if kept_wide:
        # a matrix stored in 32-bit stays 32-bit: said aloud, because its products then take
        # the plain float32 kernel and the matrix twice the memory
        import warnings
        warnings.warn(f"{folder}: {len(kept_wide)} matrices are stored in 32-bit floats and are kept so under "
                      f"{compute_dtype} (first: {kept_wide[0]}); their products run in the float32 kernel. "
                      "Store the checkpoint in bfloat16 for the fast path.", stacklevel=2)
    return out
