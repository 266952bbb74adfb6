"""The HIP kernels are the only compute path: without a GPU the kernel set refuses to
exist, and a library that cannot be built is an error, never a fallback."""

import pytest
import torch

from socrates_amd.kernels import HipKernels
from socrates_amd.kernels import build as kbuild


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the behaviour without a GPU")
def test_no_gpu_is_an_error_not_a_cpu_path():
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        HipKernels(torch.float32, "cuda:0")


def test_missing_compiler_is_an_error(monkeypatch, tmp_path):
    monkeypatch.setenv("HIPCC", str(tmp_path / "nope"))
    monkeypatch.setattr(kbuild.shutil, "which", lambda name: None)
    monkeypatch.setattr(kbuild, "_hipcc", lambda: (_ for _ in ()).throw(kbuild.KernelBuildError("hipcc not found")))
    monkeypatch.setattr(kbuild, "_build_dir_cache", tmp_path)
    with pytest.raises(kbuild.KernelBuildError, match="hipcc not found"):
        kbuild.compile_library("sampling", force=True, quiet=True)


def test_library_names_carry_a_source_hash():
    a = kbuild.library_path("attention", 128).name
    b = kbuild.library_path("attention", 64).name
    assert a.startswith("libsoc_attention_d128.") and b.startswith("libsoc_attention_d64.") and a != b
    with pytest.raises(ValueError):
        kbuild.library_path("attention")
