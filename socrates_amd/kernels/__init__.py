"""The kernel set: thin, checked Python wrappers over the HIP entry points.

``HipKernels(dtype, device)`` is what every part computes with. It is the only
kernel set in the package: there is no CPU or library path behind it, and it
raises at construction if the GPU or a library is missing (the reference's
``require_cuda_kernel``, model/kernels/__init__.py:82-92, has the same purpose).
Wrappers check devices, dtypes, contiguity and shapes on the host before a kernel
is launched, so that a wrong operand is an exception and not a memory fault.

This module holds the class, its switches and thresholds, and the small kernels (embedding,
norms, sampling); ``products.py`` the matrix products in all their forms, ``attention.py``
attention and what prepares it, ``planning.py`` the host arithmetic of key splits,
``common.py`` what they share, ``build.py`` the compiler and loader.
"""

from __future__ import annotations

import collections
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from .attention import Attention
from .build import KernelBuildError, build_all, compile_library, load_library
from .common import (_ATTENTION_SIGNATURES, _DTYPE_CODE, _EW_SIGNATURES, _GEMM_SIGNATURES, _SAMPLING_SIGNATURES, KernelError,
                     NormOwed, RowsByTile, _check, _declare, _ptr)
from .planning import MAX_KEY_SPLITS, plan_key_splits
from .products import Products

__all__ = ["HipKernels", "KernelBuildError", "KernelError", "MAX_KEY_SPLITS", "NormOwed", "RowsByTile", "build_all",
           "compile_library", "load_library", "plan_key_splits"]


class HipKernels(Products, Attention):
    def __init__(self, dtype=torch.bfloat16, device="cuda:0"):
        if dtype not in _DTYPE_CODE:
            raise ValueError(f"compute dtype must be float32 or bfloat16, not {dtype}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the HIP kernels are the only compute path "
                              "(there is no CPU fallback)")
        self.dtype, self.device = dtype, torch.device(device)
        self.code = _DTYPE_CODE[dtype]
        self._ew = load_library("elementwise")
        self._gemm = load_library("gemm")
        self._sampling = load_library("sampling")
        self._attn = {}
        _declare(self._ew, _EW_SIGNATURES)
        _declare(self._gemm, _GEMM_SIGNATURES)
        _declare(self._sampling, _SAMPLING_SIGNATURES)
        self.attention_splits = None        # (split_len, n_splits) override, for tests and capture
        self.attention_row_tiles = None     # row tiles per wave of the MFMA kernel, override
        self.last_attention_kernel = None   # (kernel, row tiles) the last bfloat16 call went to
        # (rows, N, K, out dtype, partial sums welcome) -> "own" | "library" for bfloat16 products
        # of at most 16 rows; filled while ``library_tuning`` is on, by timing both
        self.product_choice = {}
        self._tuning = False
        self.attention_mfma = True          # bfloat16 takes the MFMA kernels
        self.attention_workgroup = True     # prompt portions take the kernel that shares K/V through LDS
        # Which form of the prompt-portion attention a step takes, by the number of workgroups
        # its long portions give (of 32 rows x 4 waves for the first three, of the chosen form
        # for the last). Measured on an MI355X (256 compute units) at 8 kv heads of 4 x 128 and
        # 4 x 64; another head layout or another GPU may want other values: set them here.
        self.prompt_form_thresholds = {
            "workgroup_kernel": 256,          # below: the per-wave kernel with key splits
            "eight_waves": 256,               # from here: 32 rows per wave, keys in two halves
            "four_waves_of_32_rows": 768,     # from here (head sizes over 64): four waves of 32 rows
            "two_tiles_of_16_rows": 512,      # head sizes that are no multiple of 32, up to 64
        }
        # bfloat16 products with more than 16 rows go to the library (hipBLASLt through
        # torch.mm), as the reference's all do (nn.Linear); False keeps them on this
        # package's tiled MFMA kernel
        self.library_gemm = True
        self.swiglu_waves = 8           # waves of the fused gate+up product (measured: 4, 8, 16 within 5 %)
        # The sweep form of the skinny product (one workgroup per compute unit keeps its slices
        # of x in registers and walks over the weight tiles): from this many rows of x on, for
        # products of at least ``sweep_min_items`` weight tiles (pairs of them with SwiGLU).
        # Measured on an MI355X at 4B-sized layers with the weights laid out by tile: a decode
        # step of one request takes 2.42 ms with it and 2.52 ms without, of 8 requests 2.87
        # against 3.2 ms, of 16 requests 3.66 against 4.3 ms. (With the weights row by row it
        # lost at one row and won from three on.)
        self.sweep_rows = 1             # 0: never
        self.sweep_min_items = 256
        # Products of at most 16 rows read a second copy of their weight, laid out by tile
        # ([N / 16, K / 32, 16, 32]: a wave's load of 16 rows x 32 k is 1 KB in one piece instead
        # of sixteen pieces of 64 bytes, which streams 5 to 15 % faster), made the first time
        # such a product meets the weight and kept as long as this kernel set. It costs the
        # weight's memory once more; weights below ``pack_min_elements`` elements, or whose N
        # is no multiple of 16 or K of 32, are read row by row.
        self.pack_weights = True
        self.pack_min_elements = 1 << 20
        # what a decode step's attention and gate / up product hand to the projection behind
        # them may lie by tile too (``RowsByTile``); measured: 0.8 and 0.6 us less for O and
        # down of a 4B-sized layer at 8 rows, 1.9 and 1.5 us at 16
        self.rows_by_tile = True
        self._packed = {}               # (address, N, K) -> (the weight, its copy by tile, the weight's version)
        # Products of 17 to ``parts_rows`` rows whose consumer takes float32 partial sums (the
        # projections that end a branch): K split over sweeping workgroups instead of the
        # library's product, for K of at least ``parts_min_k`` (measured at 4B-sized layers, cold
        # weights, 64 rows: down 17 against 28 us, O 10 against 11 us; 32 rows: 14 against 21 us
        # and 7.5 against 9 us). 0 rows: never.
        self.parts_rows, self.parts_min_k = 64, 2048
        # Products of 17 to ``stream_rows`` rows whose consumer wants whole sums (QKV, gate / up
        # with its activation, the output head): K outermost, a workgroup's sums in registers
        # and x read once per workgroup, instead of the library's product. 0 rows: never.
        self.stream_rows, self.stream_min_items = 64, 256
        # steps of at most 16 rows: a branch's last projection adds to the residual and leaves
        # the norm's factor to the next product (linear_add_norm) instead of a norm kernel
        self.fuse_norms = True
        # decode steps: per-head norm, rotation and the page write inside the attention kernel
        self.fuse_rope = True
        # key splits of the MFMA decode attention: waves aimed at, and the fewest keys of a split
        # (measured at 8 kv heads of 128, context 2,048, in ms per step of a 4B-sized model at
        # 1,024 / 2,048 / 4,096 waves: batch 4: 2.92 / 2.97 / 2.97; 8: 3.36 / 3.41 / 3.59; 16:
        # 4.49 / 4.37 / -; 24: 5.09 / 5.15 / 5.16; 32: 5.32 / 5.51 / 5.57: more splits mean more
        # workgroups that have to meet in memory)
        self.split_target_waves, self.split_min_keys = 1024, 64
        self.addnorm_waves = 0          # waves of such a projection, override
        self.addnorm_splits = 0         # workgroups that share one tile's K in it, override
        self.addnorm_tile_rows = 0      # weight rows of a workgroup in it (8 to 16), override
        # arrival counts of those workgroups, one per tile of 16 outputs: zero between launches
        # (the last to arrive leaves it so). All launches of this kernel set share them, so
        # they must not overlap: one stream, as everywhere in this package.
        self._split_count = torch.zeros(16384, dtype=torch.int32, device=self.device)
        # Counts what takes away something a captured step relies on (an address it reads,
        # a choice it was captured with); whoever holds graphs over this kernel set compares
        # it with the count at their capture and drops them when it has moved.
        self.graph_epoch = 0
        # how often each form of a product or of the attention was launched (a replayed graph
        # launches without coming by here): for tests and for whoever asks what a step ran
        self.forms = collections.Counter()

    def invalidate_graphs(self) -> None:
        """Say that steps captured over this kernel set so far must not be replayed."""
        self.graph_epoch += 1

    # -- helpers -----------------------------------------------------------------------------
    def _stream(self):
        return c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def _want(self, t, name, dtype=None, shape=None):
        if t.device.type != "cuda":
            raise KernelError(f"{name} is on {t.device}, the kernels need it on the GPU")
        if not t.is_contiguous():
            raise KernelError(f"{name} is not contiguous")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")
        return t

    def _attention_lib(self, head_dim: int):
        lib = self._attn.get(head_dim)
        if lib is None:
            if head_dim % 16 or not 16 <= head_dim <= 256:
                raise KernelError(f"head size {head_dim}: the attention kernels take multiples of "
                                  "16 from 16 to 256")
            lib = load_library("attention", head_dim)
            _declare(lib, _ATTENTION_SIGNATURES)
            if lib.soc_attention_head_dim() != head_dim:
                raise KernelError("attention library was built for another head size")
            self._attn[head_dim] = lib
        return lib

    def prepare(self, head_dims=()):
        """Compile and load, ahead of the first step, what a model with these head sizes needs."""
        for d in head_dims:
            self._attention_lib(d)

    # -- embedding, norms, activation -------------------------------------------------------------
    def embedding(self, ids, table):
        self._want(ids, "ids", torch.int32)
        self._want(table, "embedding table")
        N, (V, d) = ids.numel(), table.shape
        out = torch.empty((N, d), dtype=torch.float32, device=self.device)
        _check(self._ew.soc_embedding(_ptr(ids), _ptr(table), _ptr(out), c_int(N), c_int(d), c_int(V),
                                      c_int(_DTYPE_CODE[table.dtype]), self._stream()), "embedding")
        return out

    def add_rmsnorm(self, residual, delta, weight, eps, rows=None, by_tile=False):
        """``delta``: None, a [N, d] tensor of the compute dtype, or float32 partial sums
        [S, N, d] (what ``linear(..., allow_partial=True)`` returns) that are added in order.
        ``by_tile``: the caller hands the result to ``linear`` or ``linear_swiglu`` and nowhere
        else, so 17 to 64 rows may come as a ``RowsByTile``."""
        N, d = residual.shape
        self._want(residual, "residual", torch.float32)
        self._want(weight, "norm weight", torch.float32, (d,))
        whole = partials = None
        n_partials = 0
        if delta is not None and delta.dim() == 3:
            partials, n_partials = self._want(delta, "partial sums", torch.float32, (delta.shape[0], N, d)), delta.shape[0]
        elif delta is not None:
            whole = self._want(delta, "delta", self.dtype, (N, d))
        if rows is not None:
            self._want(rows, "rows", torch.int32)
        n_out = N if rows is None else rows.numel()
        tile_rows = 0
        if (by_tile and self.rows_by_tile and self.dtype == torch.bfloat16 and 16 < n_out <= min(self.stream_rows, 64)
                and d % 32 == 0 and d <= 8192):
            tile_rows = (n_out + 15) // 16 * 16
        out = torch.empty((d // 32, tile_rows, 32) if tile_rows else (n_out, d), dtype=self.dtype, device=self.device)
        _check(self._ew.soc_add_rmsnorm(_ptr(residual), _ptr(whole), _ptr(partials), c_int(n_partials),
                                        c_longlong(N * d), _ptr(weight), _ptr(out), _ptr(rows),
                                        c_int(n_out), c_int(d), c_float(eps), c_int(self.code), c_int(tile_rows),
                                        self._stream()), "add_rmsnorm")
        return RowsByTile(out, n_out, d) if tile_rows else out

    def rmsnorm(self, x, weight, eps):
        dim = x.shape[-1]
        self._want(x, "x", self.dtype)
        self._want(weight, "norm weight", torch.float32, (dim,))
        out = torch.empty_like(x)
        _check(self._ew.soc_rmsnorm(_ptr(x), _ptr(weight), _ptr(out), c_int(x.numel() // dim), c_int(dim),
                                    c_float(eps), c_int(self.code), self._stream()), "rmsnorm")
        return out

    def scale_softcap_(self, x, scale=1.0, softcap=None):
        """In place on float32 ``x``: x * scale, then softcap * tanh(x / softcap) if a soft cap
        is given."""
        self._want(x, "x", torch.float32)
        if softcap is not None and not softcap > 0:
            raise KernelError("a soft cap is positive")
        _check(self._ew.soc_scale_softcap(_ptr(x), c_longlong(x.numel()), c_float(scale), c_float(softcap or 0.0),
                                          self._stream()), "scale_softcap")
        return x

    # -- sampling ------------------------------------------------------------------------------
    def argmax(self, logits):
        """Greedy tokens, the lowest index among equal maxima; int32 [n]."""
        n, V = logits.shape
        self._want(logits, "logits", torch.float32)
        n_chunks = max(1, min(64, V // 2048))
        partial = torch.empty((n, n_chunks, 2), dtype=torch.float32, device=self.device)
        out = torch.empty((n,), dtype=torch.int32, device=self.device)
        _check(self._sampling.soc_argmax(_ptr(logits), _ptr(partial), _ptr(out), c_int(n), c_int(V),
                                         c_int(n_chunks), self._stream()), "argmax")
        return out

    def sample(self, logits, temperature, seed, draws):
        """logits [n, V] float32; temperature [n] float32 (0: greedy), seed and draws [n] int64.
        Returns int32 [n]."""
        n, V = logits.shape
        self._want(logits, "logits", torch.float32)
        if temperature is not None:
            self._want(temperature, "temperature", torch.float32, (n,))
            self._want(seed, "seed", torch.int64, (n,))
            self._want(draws, "draws", torch.int64, (n,))
        out = torch.empty((n,), dtype=torch.int32, device=self.device)
        _check(self._sampling.soc_sample(_ptr(logits), _ptr(temperature), _ptr(seed), _ptr(draws), _ptr(out),
                                         c_int(n), c_int(V), self._stream()), "sample")
        return out
