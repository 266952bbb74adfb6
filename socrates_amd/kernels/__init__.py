"""The kernel set: thin, checked Python wrappers over the HIP entry points.

``HipKernels(dtype, device)`` is what every part computes with. It is the only
kernel set in the package: there is no CPU or library path behind it, and it
raises at construction if the GPU or a library is missing (the reference's
``require_cuda_kernel``, model/kernels/__init__.py:82-92, has the same purpose).
Wrappers check devices, dtypes, contiguity and shapes on the host before a kernel
is launched, so that a wrong operand is an exception and not a memory fault.
"""

from __future__ import annotations

import collections
import ctypes
from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

from .build import KernelBuildError, build_all, compile_library, load_library

__all__ = ["HipKernels", "KernelBuildError", "KernelError", "MAX_KEY_SPLITS", "NormOwed", "RowsByTile", "build_all",
           "compile_library", "load_library", "plan_key_splits"]

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


def _ptr(t):
    return None if t is None else c_void_p(t.data_ptr())


def _check(err, what):
    if err != 0:
        raise KernelError(f"{what}: HIP error {err}")


P, I, F = c_void_p, c_int, c_float
_EW_SIGNATURES = {
    "soc_embedding": [P, P, P, I, I, I, I, P],
    "soc_add_rmsnorm": [P, P, P, I, c_longlong, P, P, P, I, I, F, I, I, P],
    "soc_rmsnorm": [P, P, P, I, I, F, I, P],
    "soc_swiglu": [P, P, I, I, I, I, P],
    "soc_scale_softcap": [P, c_longlong, F, F, P],
    "soc_qk_norm_rope": [P] * 7 + [I] + [P] * 5 + [I] * 6 + [F, I, P],
    "soc_rope": [P, P, P, I, I, I, I, I, P],
    "soc_kv_write": [P] * 5 + [I, P, P, I, I, I, I, I, P],
    "soc_rope_table": [P, I, I, I, P, P],
}
_GEMM_SIGNATURES = {
    "soc_gemm_generic": [P, P, P, I, I, I, I, I, I, P],
    "soc_gemm_bf16_mfma": [P, P, P, I, I, I, I, P],
    "soc_gemm_bf16_skinny": [P, P, P, P, I, I, I, I, I, I, I, I, P],
    "soc_gemm_skinny_plan": [I, I, I, I, P, P, P],
    "soc_gemm_bf16_skinny_swiglu": [P, P, P, I, I, I, I, I, P, I, I, F, I, P],
    "soc_gemm_bf16_skinny_norm": [P, P, P, I, I, I, I, P, I, I, F, P, P, P, P, I, P, P, I, I, P],
    "soc_gemm_bf16_sweep": [P, P, P, I, I, I, I, I, I, I, P, I, I, F, I, P],
    "soc_gemm_sweep_plan": [I, I, I, P, P],
    "soc_gemm_bf16_sweep_parts": [P, P, P, I, I, I, I, I, I, I, P],
    "soc_gemm_sweep_parts_plan": [I, I, I, P, P, P],
    "soc_gemm_bf16_stream": [P, P, P, I, I, I, I, I, I, I, I, P],
    "soc_gemm_stream_plan": [I, I, I, I, P, P],
}
_SAMPLING_SIGNATURES = {"soc_sample": [P, P, P, P, P, I, I, P], "soc_argmax": [P, P, P, I, I, I, P]}
_ATTENTION_SIGNATURES = {
    "soc_paged_attention_tokens": [P, P, P, P, I, P, P, P, P, P, I, I, I, I, F, I, I, I, I, F, P, P, P],
    "soc_paged_attention_mfma": [P, P, P, P, I, P, P, P, I, P, P, P, P, I, I, I, I, F, I, I, I, I, I, I, P],
    "soc_paged_attention_prefill": [P, P, P, P, I, P, P, P, I, P, I, I, I, I, F, I, I, I, P],
    "soc_paged_attention_decode_fused": [P, I, P, P, P, I, P, P, P, P, P, P, I, I, I, I, F, I, I, I, I, P, P, P, F, I, I, P],
    "soc_attention_head_dim": [],
}


def _declare(lib, signatures):
    for name, argtypes in signatures.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = argtypes, (None if name == "soc_gemm_skinny_plan" else c_int)


MAX_KEY_SPLITS = 256    # of the MFMA attention: 64 workgroups of four splits meet per task


def plan_key_splits(n_blocks, n_kv_heads, group, max_keys, target_waves=1024, min_keys=64, n_units=256):
    """(split_len, n_splits) for the MFMA attention kernel: enough waves to fill the GPU, no
    split shorter than 64 keys, at most MAX_KEY_SPLITS of them (a longer context gets longer
    splits), one split or a multiple of four (four share a workgroup; some of the last four
    may lie beyond the keys and are empty). Splits are over absolute key indices, a multiple of
    16 keys long, and cover keys 0 .. max_keys - 1. Host arithmetic only."""
    waves = n_blocks * n_kv_heads * ((group + 15) // 16)
    # from one wave per SIMD on (1,024) no split: a split costs a trip through LDS, or memory
    n = 1 if waves >= 1024 else max(1, min((target_waves + waves - 1) // waves,
                                           (max_keys + min_keys - 1) // min_keys, MAX_KEY_SPLITS))
    if n > 1:
        # splits that would each stream more than 2,048 keys are halved: twice the waves keep
        # more loads on their way, and walks that long pay for the larger meeting (measured
        # at 8 rows of 8 kv heads, 32,768 keys: a step of 8.86 ms with 32 splits of 1,024 keys
        # against 9.28 ms with 16 of 2,048; at 8,192 keys 16 splits of 512 stay the faster)
        twice = min((2 * target_waves + waves - 1) // waves, MAX_KEY_SPLITS)
        if twice > n and max_keys >= twice * 1024:
            n = twice
    if n == 1:
        return ((max_keys + 15) // 16 * 16), 1
    n = (n + 3) // 4 * 4
    # Four splits make a workgroup, and a compute unit holds two such workgroups. A launch a
    # little over a whole number of workgroups per compute unit (288 of them: 32 of the 256
    # units get a second one and finish last) is cut down to that whole number; measured on
    # an MI355X at 8 kv heads, ms per step of a 4B-sized model: 12 rows behind 2,048 keys 3.29
    # with 12 splits (288 workgroups) against 3.16 with 8 (192), behind 8,192 keys 5.82 against
    # 4.97; 6 rows 2.75 with 24 splits (288) against 2.65 with 16 (192), 3.96 against 3.55; 24
    # rows 4.40 with 8 splits (384) against 4.20 with 4 (192).
    tasks = waves                                   # (row block, kv head, chunk of heads)
    groups = tasks * (n // 4)
    if groups > n_units and groups % n_units and (groups % n_units) * 4 < n_units * 3:
        fewer = (n_units * (groups // n_units) // tasks) * 4
        if fewer >= 4:
            n = fewer
    split_len = ((max_keys + n - 1) // n + 15) // 16 * 16
    return split_len, ((max_keys + split_len - 1) // split_len + 3) // 4 * 4


class NormOwed:
    """Rows that are still owed their RMSNorm factor: ``x`` [M, dim] = bfloat16(h * gain) of the
    rows h of the residual stream, and ``ssq`` [M, tiles rounded up to 4], float32 partial sums
    of h^2 over ``tiles`` runs of columns (16 each, or fewer where the product that made them gave its workgroups fewer weight rows; the padding is never read). The factor 1 / sqrt(sum(ssq) / dim + eps) is one number per row, so the
    product that consumes the rows applies it to its sums (``HipKernels.linear`` and
    ``linear_swiglu`` take a NormOwed where they take x). Made by ``linear_add_norm``."""
    __slots__ = ("x", "ssq", "dim", "eps", "tiles")

    def __init__(self, x, ssq, dim, eps, tiles=None):
        self.x, self.ssq, self.dim, self.eps = x, ssq, dim, eps
        self.tiles = tiles if tiles is not None else (dim + 15) // 16      # partial sums per row

    @property
    def shape(self):
        return self.x.shape


class RowsByTile:
    """Rows of bfloat16 activations laid out by tile, ``data`` [dim / 32, R, 32] with R the rows
    rounded up to a multiple of 16 (element (row, col) at [col // 32, row,
    col % 32]; rows from ``rows`` on are never written, and what is read of them goes nowhere),
    for the product that takes them next: it then asks the L2 for one piece of rows x 64 bytes
    per load where rows laid out one after the other give it that many pieces. Made by
    ``decode_attention``, ``linear_swiglu`` and ``add_rmsnorm`` where the caller allows it
    (``by_tile``: the caller hands the result to ``linear``, ``linear_swiglu`` or
    ``linear_add_norm`` and nowhere else), taken by those."""
    __slots__ = ("data", "rows", "dim")

    def __init__(self, data, rows, dim):
        self.data, self.rows, self.dim = data, rows, dim

    @property
    def shape(self):
        return (self.rows, self.dim)

    def by_rows(self):
        """The rows as an ordinary [rows, dim] tensor (a copy)."""
        return self.data[:, :self.rows].permute(1, 0, 2).reshape(self.rows, self.dim)


class HipKernels:
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

    def swiglu(self, gate_up, interleave=0):
        """silu(gate) * up from a [N, 2 ff] tensor holding [gate | up] (interleave 0) or gate and
        up columns alternating in blocks of ``interleave``."""
        self._want(gate_up, "gate_up", self.dtype)
        N, two_ff = gate_up.shape
        if two_ff % 2 or (interleave and (two_ff // 2) % interleave):
            raise KernelError("gate_up needs an even last dimension that the interleave divides")
        out = torch.empty((N, two_ff // 2), dtype=self.dtype, device=self.device)
        _check(self._ew.soc_swiglu(_ptr(gate_up), _ptr(out), c_int(N), c_int(two_ff // 2), c_int(interleave),
                                   c_int(self.code), self._stream()), "swiglu")
        return out

    def linear_swiglu(self, x, w_gate_up, interleave=0, by_tile=False):
        """swiglu(x @ w_gate_up^T). With rows interleaved in blocks of 16 and at most 16 rows of
        x in bfloat16, one kernel: the skinny product applies silu(gate) * up in its epilogue.
        ``by_tile``: the caller hands the result to ``linear_add_norm`` or ``linear`` only, so
        it may come as a ``RowsByTile``."""
        owed = x if isinstance(x, NormOwed) else None
        if owed is not None:
            x = owed.x
        if isinstance(x, RowsByTile):
            # 17 to 64 rows by tile (from ``add_rmsnorm``): the product with K outermost reads them so
            M, K = x.shape
            N = w_gate_up.shape[0]
            plan = self._stream_plan(M, N, K, swiglu=True) if (
                interleave == 16 and w_gate_up.dtype == torch.bfloat16 and N % 32 == 0 and self.library_gemm
                and x.data.shape[1] > 16) else None
            if plan is not None:
                self._want(w_gate_up, "weight", None, (N, K))
                key, xt = (M, N, K, "swiglu", False), x
                choice = self.product_choice.get(key)
                if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                    xr = x.by_rows()
                    choice = self.product_choice[key] = self._faster(
                        lambda: self._k_outermost(plan, xt, w_gate_up, torch.empty((M, N // 2), dtype=self.dtype, device=self.device), True),
                        lambda: self.swiglu(torch.mm(xr, w_gate_up.t()), interleave))
                if choice != "library" and (choice == "own" or self._stream_default(M, N, K, plan, True)):
                    out = self._swiglu_out(M, N, by_tile)
                    self._k_outermost(plan, x, w_gate_up, out, True, what="linear_swiglu")
                    return out
            x = x.by_rows()
        M, K = x.shape
        N = w_gate_up.shape[0]
        if (interleave == 16 and x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
                and 0 < M <= 16 and K % 8 == 0 and K >= 8 and N % 32 == 0):
            self._want(x, "x")
            self._want(w_gate_up, "weight", None, (N, K))
            tiled_out = bool(by_tile and self.rows_by_tile and N % 64 == 0)
            out = torch.empty((N // 64, 16, 32) if tiled_out else (M, N // 2), dtype=self.dtype, device=self.device)
            result = RowsByTile(out, M, N // 2) if tiled_out else out
            plan = self._sweep_plan(M, N, K, swiglu=True)
            if plan is not None:
                self._sweep(plan, x, w_gate_up, out, self._SK_SWIGLU, self._owed_args(owed, M, K), what="linear_swiglu",
                            layout=4 if tiled_out else 0)
                return result
            n_waves = self.swiglu_waves          # half of them per tile (gate, up), splitting K
            while n_waves > 2 and K // (n_waves // 2) < 128:
                n_waves //= 2
            ssq, tiles, dim, eps = self._owed_args(owed, M, K)
            wt, tiled = self._by_tile(w_gate_up)
            self.forms["skinny_swiglu"] += 1
            _check(self._gemm.soc_gemm_bf16_skinny_swiglu(_ptr(x), _ptr(wt), _ptr(out), c_int(M), c_int(N),
                                                          c_int(K), c_int(self.code), c_int(n_waves),
                                                          ssq, c_int(tiles), c_int(dim), c_float(eps),
                                                          c_int(tiled | (4 if tiled_out else 0)),
                                                          self._stream()), "linear_swiglu")
            return result
        if (owed is None and interleave == 16 and x.dtype == torch.bfloat16 and w_gate_up.dtype == torch.bfloat16
                and N % 32 == 0 and self.library_gemm):
            plan = self._stream_plan(M, N, K, swiglu=True)
            if plan is not None:
                self._want(x, "x")
                self._want(w_gate_up, "weight", None, (N, K))
                key = (M, N, K, "swiglu", False)
                choice = self.product_choice.get(key)
                if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                    choice = self.product_choice[key] = self._faster(
                        lambda: self._k_outermost(plan, x, w_gate_up, torch.empty((M, N // 2), dtype=self.dtype, device=self.device), True),
                        lambda: self.swiglu(torch.mm(x, w_gate_up.t()), interleave))
                if choice != "library" and (choice == "own" or self._stream_default(M, N, K, plan, True, by_tile=False)):
                    out = self._swiglu_out(M, N, by_tile)
                    self._k_outermost(plan, x, w_gate_up, out, True, what="linear_swiglu")
                    return out
        return self.swiglu(self.linear(owed if owed is not None else x, w_gate_up), interleave)

    _SK_SWIGLU, _SK_SCALED = 1, 2

    def _swiglu_out(self, M, N, by_tile):
        """Where the activation of 17 to 64 rows goes: [M, N / 2], or by tile where the caller
        hands it to one projection and nowhere else."""
        if by_tile and self.rows_by_tile and N % 64 == 0:
            rows = (M + 15) // 16 * 16
            return RowsByTile(torch.empty((N // 64, rows, 32), dtype=self.dtype, device=self.device), M, N // 2)
        return torch.empty((M, N // 2), dtype=self.dtype, device=self.device)

    def _by_tile(self, w, h=16):
        """(the tensor a skinny product reads, 1 if it lies by tile else 0) for weight ``w``
        [N, K] bfloat16, in tiles of ``h`` rows: [N / h, K / 32, h, 32]. The copy by tile is made
        at the first call for a weight and a tile height (not while a graph is being captured:
        such a call reads the weight row by row); the entry keeps the weight alive, so its
        address cannot come to mean another tensor."""
        N, K = w.shape
        if N % h or K % 32 or w.dtype != torch.bfloat16 or not w.is_contiguous():
            return w, 0
        key = (w.data_ptr(), N, K, h)
        entry = self._packed.get(key)
        if entry is not None and entry[2] == w._version:
            return entry[1], 1
        # (a weight written to in place is copied anew)
        if (not self.pack_weights or N * K < self.pack_min_elements or torch.cuda.is_current_stream_capturing()):
            return w, 0
        try:
            tiled = w.view(N // h, h, K // 32, 32).permute(0, 2, 1, 3).contiguous()
        except torch.cuda.OutOfMemoryError:
            # no room for second copies (weights and cache fill the GPU): no new ones from now
            # on; the weights that have one keep using it
            import warnings
            warnings.warn("no memory for a copy of a weight laid out by tile; products of few rows read the "
                          "rows of the weights that have none (HipKernels.pack_weights = False says so up front)")
            self.pack_weights = False
            return w, 0
        self._packed[key] = (w, tiled, w._version)
        return tiled, 1

    def forget_packed(self) -> None:
        """Drop the copies by tile (to free memory). Steps captured with this kernel set read
        the copies by address, so they are declared stale (``invalidate_graphs``): the runner
        drops them before its next captured step and captures anew."""
        if self._packed:
            self.invalidate_graphs()
        self._packed.clear()

    def _sweep_plan(self, M, N, K, swiglu=False):
        """(waves, workgroups) if this product of at most 16 rows takes the sweep form."""
        if not self.sweep_rows or M < self.sweep_rows or M > 16 or K % 8 or K < 8:
            return None
        nw, wgs = c_int(0), c_int(0)
        if not self._gemm.soc_gemm_sweep_plan(c_int(N), c_int(K), c_int(1 if swiglu else 0), ctypes.byref(nw),
                                              ctypes.byref(wgs)):
            return None
        items = N // 32 if swiglu else (N + 15) // 16
        if items < self.sweep_min_items or (N + 32) * K * 2 >= 0xfffffff0:
            return None
        return nw.value, wgs.value

    def _sweep(self, plan, x, w, out, mode, owed_args=(None, 0, 0, 0.0), what="linear", layout=0):
        (M, K), N = x.shape, w.shape[0]
        ssq, tiles, dim, eps = owed_args
        if ssq is not None:
            mode |= self._SK_SCALED
        wt, tiled = self._by_tile(w)
        self.forms["sweep" + ("_swiglu" if mode & self._SK_SWIGLU else "")] += 1
        _check(self._gemm.soc_gemm_bf16_sweep(
            _ptr(x), _ptr(wt), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(_DTYPE_CODE[out.dtype]), c_int(mode),
            c_int(plan[0]), c_int(plan[1]), ssq, c_int(tiles), c_int(dim), c_float(eps), c_int(tiled | layout),
            self._stream()),
            f"{what} (sweep) [{M}x{K}] x [{N}x{K}]^T")

    def _stream_plan(self, M, N, K, swiglu=False):
        """(workgroups, items per workgroup) if this product of 17 to ``stream_rows`` rows takes
        the form with K outermost."""
        if not 16 < M <= min(self.stream_rows, 64) or K % 8 or K < 8 or (N + 32) * K * 2 >= 0xfffffff0:
            return None
        wgs, per = c_int(0), c_int(0)
        if not self._gemm.soc_gemm_stream_plan(c_int(M), c_int(N), c_int(K), c_int(1 if swiglu else 0),
                                               ctypes.byref(wgs), ctypes.byref(per)):
            return None
        if wgs.value * per.value < self.stream_min_items:
            return None
        return wgs.value, per.value

    @staticmethod
    def _stream_default(M, N, K, plan, swiglu=False, by_tile=True):
        """Whether the product with K outermost is taken where no tuning pass has timed it
        against the library. Measured on an MI355X inside replayed graphs, weights from memory
        (us, own with x by tile / own with x row by row / library, with the activation kernel
        where there is one): QKV of 4B-sized layers [6,144 x 2,560] at 32 rows 10.1 / 12.6 / 11.5,
        at 64 rows 13.3 / 19.4 / 15.7; gate and up [19,456 x 2,560] 23.5 / 24.7 / 27.5 and
        28.2 / 32.1 / 31.0; 8B-sized [6,144 x 4,096] 14.6 / 17.7 / 15.4 and 19.3 / 26.3 / 18.0,
        [24,576 x 4,096] 40.3 / 40.6 / 50.0 and 42.9 / 47.4 / 50.6; 32B-sized [51,200 x 5,120],
        three passes of a workgroup: 106.5 / 118.0 / 102.1 and 118.4 / 153.2 / 112.1; the output
        head [151,936 x 2,560], seven passes: 160 / 170 / 174 and 199 / 225 / 186. So: up to 32 rows
        where x comes by tile or the workgroup needs one pass; beyond, one pass with more
        weights than rows of x per workgroup, or a short K."""
        tiles = plan[1] * (2 if swiglu else 1)
        one_pass = tiles <= 6
        if M <= 32:
            return one_pass or by_tile
        return one_pass and by_tile and (16 * tiles >= M or K <= 3072)

    def _k_outermost(self, plan, x, w, out, swiglu=False, what="linear"):
        (M, K), N = x.shape, w.shape[0]
        wt, tiled = self._by_tile(w)
        if isinstance(out, RowsByTile):                  # the activation by tile, for the projection behind it
            out, tiled = out.data, tiled | 4
        if isinstance(x, RowsByTile):
            self._want(x.data, "x by tile", torch.bfloat16, (K // 32, (M + 15) // 16 * 16, 32))
            x, tiled = x.data, tiled | 2
        self.forms["stream" + ("_swiglu" if swiglu else "")] += 1
        _check(self._gemm.soc_gemm_bf16_stream(
            _ptr(x), _ptr(wt), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(_DTYPE_CODE[out.dtype]),
            c_int(self._SK_SWIGLU if swiglu else 0), c_int(plan[0]), c_int(plan[1]), c_int(tiled), self._stream()),
            f"{what} (K outermost) [{M}x{K}] x [{N}x{K}]^T")
        return out

    def _parts_plan(self, M, N, K):
        """(parts of K, K per wave, groups) if this product of 17 to 64 rows, whose consumer
        takes partial sums, is swept with K split over workgroups."""
        if not 16 < M <= self.parts_rows or K % 8 or K < self.parts_min_k or (N + 32) * K * 2 >= 0xfffffff0:
            return None
        parts, kpw, groups = c_int(0), c_int(0), c_int(0)
        if not self._gemm.soc_gemm_sweep_parts_plan(c_int(M), c_int(N), c_int(K), ctypes.byref(parts),
                                                    ctypes.byref(kpw), ctypes.byref(groups)):
            return None
        return parts.value, kpw.value, groups.value

    def _sweep_parts(self, plan, x, w):
        (M, K), N = x.shape, w.shape[0]
        parts, kpw, groups = plan
        out = torch.empty((parts, M, N), dtype=torch.float32, device=self.device)
        wt, tiled = self._by_tile(w)
        if isinstance(x, RowsByTile):
            rows = x.data.shape[1]
            self._want(x.data, "x by tile", torch.bfloat16, (K // 32, rows, 32))
            x, tiled = x.data, tiled | 2 | (rows << 8)
        self.forms[f"parts_of_k:{parts}"] += 1
        _check(self._gemm.soc_gemm_bf16_sweep_parts(_ptr(x), _ptr(wt), _ptr(out), c_int(M), c_int(N), c_int(K),
                                                    c_int(parts), c_int(kpw), c_int(groups), c_int(tiled),
                                                    self._stream()),
               f"linear (parts of K) [{M}x{K}] x [{N}x{K}]^T")
        return out

    def _owed_args(self, owed, M, K):
        """(ssq pointer, tiles, dim, eps) of a NormOwed input, checked; nulls for a plain one."""
        if owed is None:
            return None, 0, 0, 0.0
        if owed.dim != K:
            raise KernelError(f"rows owed a norm over {owed.dim} elements meet a product over {K}")
        tiles = owed.tiles
        self._want(owed.ssq, "sums of squares", torch.float32, (M, (tiles + 3) // 4 * 4))
        return _ptr(owed.ssq), tiles, owed.dim, owed.eps

    def linear_add_norm(self, y, w, residual, gain, eps):
        """residual += y @ w^T, then the RMSNorm (``gain``, ``eps``) of the new residual: what
        ``add_rmsnorm(residual, linear(y, w), gain, eps)`` returns. For bfloat16 steps of at most
        16 rows it is one kernel: the product's epilogue adds to the residual and leaves the
        rows as a NormOwed, whose factor the next product applies (``y`` may be one itself)."""
        owed = y if isinstance(y, NormOwed) else None
        tiled_y = y if isinstance(y, RowsByTile) else None
        yx = owed.x if owed is not None else (tiled_y.data if tiled_y is not None else y)
        (M, K), N = (tiled_y.shape if tiled_y is not None else yx.shape), w.shape[0]
        if not (self.dtype == torch.bfloat16 and yx.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
                and 0 < M <= 16 and K % 8 == 0 and K >= 8 and N % 8 == 0 and N <= 65536 and self.fuse_norms):
            # (65,536: the sums of squares of a row are summed by one wave per 256 tiles of 16;
            # N % 8: the product that takes the owed rows has N as its K, and reads 8 at a time)
            # (the rows go to one product and nowhere else, as a NormOwed would: they may lie by tile)
            return self.add_rmsnorm(residual, self.linear(y, w, allow_partial=True), gain, eps, by_tile=True)
        if tiled_y is not None:
            self._want(yx, "y", torch.bfloat16, (K // 32, 16, 32))
            yx_layout = 2
        else:
            self._want(yx, "y", None, (M, K))
            yx_layout = 0
        self._want(w, "weight", None, (N, K))
        self._want(residual, "residual", torch.float32, (M, N))
        self._want(gain, "norm weight", torch.float32, (N,))
        tile_h, k_splits = self._addnorm_shape(N, K, M)
        if self.addnorm_tile_rows:
            tile_h = self.addnorm_tile_rows
        if self.addnorm_splits:
            k_splits = self.addnorm_splits
        if (N + tile_h - 1) // tile_h > 4096:
            tile_h = 16                     # a row's sums of squares are at most 16 segments of 256 tiles
        tiles = (N + tile_h - 1) // tile_h
        x_out = torch.empty((M, N), dtype=torch.bfloat16, device=self.device)
        ssq_out = torch.empty((M, (tiles + 3) // 4 * 4), dtype=torch.float32, device=self.device)
        n_waves = self.addnorm_waves or 8
        while n_waves > 1 and K // n_waves < 128:
            n_waves //= 2
        ssq, in_tiles, dim, in_eps = self._owed_args(owed, M, K)
        while k_splits > 1 and K // (k_splits * n_waves) < 128:
            k_splits //= 2
        sums = count = None
        if k_splits > 1:
            if tiles > self._split_count.numel():
                raise KernelError(f"linear_add_norm: {N} outputs are more than the {16 * self._split_count.numel()} "
                                  "that K can be split for")
            sums = torch.empty((tiles, k_splits, 256), dtype=torch.float32, device=self.device)
            count = self._split_count
        wt, tiled = self._by_tile(w, tile_h)
        self.forms[f"add_norm:{k_splits}"] += 1
        _check(self._gemm.soc_gemm_bf16_skinny_norm(
            _ptr(yx), _ptr(wt), None, c_int(M), c_int(N), c_int(K), c_int(n_waves), ssq, c_int(in_tiles),
            c_int(dim), c_float(in_eps), _ptr(residual), _ptr(gain), _ptr(x_out), _ptr(ssq_out),
            c_int(k_splits), _ptr(sums), _ptr(count), c_int(tiled | yx_layout), c_int(tile_h), self._stream()),
            f"linear_add_norm [{M}x{K}] x [{N}x{K}]^T")
        return NormOwed(x_out, ssq_out, N, eps, tiles)

    def _addnorm_shape(self, N, K, M):
        """(weight rows of a workgroup, workgroups that share a tile's K) of ``linear_add_norm``.
        A workgroup's 16-row product may hold fewer than 16 weight rows: a narrow output then
        spreads over more compute units (2,560 outputs are 160 tiles of 16 rows, which leave 96
        of 256 compute units idle while the others stream at what one compute unit can take, or
        256 tiles of 10). Heights that divide N (the copy by tile wants whole tiles), from 16
        down to 8; the cost of a shape is what its busiest compute unit streams, its share of
        the weights and its reading of x, plus the meeting if K is split. Measured alone inside
        replayed graphs, weights from memory, us at 8 rows (16 rows per workgroup, its best
        split of K / 10 rows, K whole): [2,560 x 9,728] 15.4 / 12.8, [2,560 x 4,096] 7.7 / 7.4,
        [5,120 x 8,192] 20.9 / 20.1, [5,120 x 25,600] 53.6 / 58.1 (there 16 rows in four parts of
        K stay); 8 rows per workgroup (320 or 640 workgroups) lose everywhere."""
        best, best_cost = (16, 1), None
        for h in range(16, 7, -1):
            if h != 16 and (N % h or M < 5):
                # (up to 4 rows whole tiles stay ahead inside a step, measured at 4B-sized layers:
                # 2.34 against 2.37 ms at one row, 2.51 against 2.53 at four; from 6 rows on the
                # lower tiles win: 2.76 against 2.83 ms at 8 rows, 3.55 against 3.62 at 16)
                continue
            tiles = -(-N // h)
            splits = self._addnorm_splits(tiles, K, M, h)
            rounds = -(-tiles * splits // 256)
            cost = rounds * (K / splits) * (h + 0.5 * min(M, 16)) / 16 + (3000 * 8 / max(M, 8) if splits > 1 else 0)
            if best_cost is None or cost < best_cost * 0.97:
                best, best_cost = (h, splits), cost
        return best

    @staticmethod
    def _addnorm_splits(tiles, K, M, h=16):
        """Workgroups that share one tile's K in ``linear_add_norm``: 1, 2 or 4, whichever gives
        the busiest of the GPU's 256 compute units the least to stream, with the meeting in
        memory priced at some 3,000 elements of K (less at more rows, where streaming is
        slower); every wave keeps at least 256 elements. Measured on an MI355X at the output and
        down projections of 4B-, 8B- and 32B-sized layers (tiles 160, 256, 320; K 4,096 to
        25,600): 160 tiles of K = 9,728 take 12.3 us whole and 13.8 us in four parts at one row,
        15.6 and 15.3 us at 8 rows, 19.8 and 17.8 us at 16; 320 tiles of K = 25,600 take 77 us
        whole and 56 us in four parts at 8 rows; 320 tiles of K = 8,192 take 24.4 us whole, 22.6 us
        in two parts and 21.2 us in four at 8 rows."""
        best, best_cost = 1, None
        for splits in (1, 2, 4):
            if splits > 1 and K // (splits * 8) < 256:
                continue
            rounds = -(-tiles * splits // 256)
            cost = rounds * (K / splits) * h / 16 + (3000 * 8 / max(M, 8) if splits > 1 else 0)
            if best_cost is None or cost < best_cost:
                best, best_cost = splits, cost
        return best

    # -- matrix products ------------------------------------------------------------------------
    def library_tuning(self, on: bool) -> None:
        """While on, the library's matrix products (bfloat16, more than 16 rows) time the
        library's solutions for every new shape they meet and keep the fastest; afterwards
        the kept choices stay in use, for this process, and shapes met later take the
        library's default. The library's record of its choices goes to a file of this
        process in the temporary folder, never to the working folder."""
        import os
        import tempfile
        import torch.cuda.tunable as tunable
        if on:
            tunable.set_filename(os.path.join(tempfile.gettempdir(), f"socrates_amd_products_{os.getpid()}.csv"))
            tunable.enable(True)
            tunable.set_max_tuning_duration(30)          # ms per solution
            tunable.set_max_tuning_iterations(20)
            # Only solutions that agree with the library's default to a rounding of bfloat16 are
            # candidates: some of the faster ones round more often on the way (measured: logits
            # of a tiny model off by twice the usual error when one of them had been picked),
            # and which one is fastest varies from run to run.
            tunable.set_numerical_check_tolerances(True, 1e-3, 8e-3)
        tunable.tuning_enable(bool(on))
        self._tuning = bool(on)
        self.invalidate_graphs()                         # steps captured before replay the choices of their time
        if not on:
            self._cold = None                            # the buffer that cools the caches between timed calls

    def _faster(self, own, library) -> str:
        """Time the two ways of one product and name the faster. Weights come from memory in a
        decode step (each is read once per step, behind gigabytes of others), so a read of
        a buffer larger than the caches comes before every timed call (a write would leave the
        memory-side cache full of lines to write back, which the timed call then pays for)."""
        if getattr(self, "_cold", None) is None:
            self._cold = torch.zeros(160 << 20, dtype=torch.float32, device=self.device)     # 640 MB
        times = []
        for fn in (library, own):                        # the library first: its own tuning happens at its first call
            fn()
            total = 0.0
            for _ in range(6):
                self._cold.max()
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                fn()
                end.record()
                end.synchronize()
                total += start.elapsed_time(end)
            times.append(total)
        return "library" if times[0] < 0.97 * times[1] else "own"

    def linear(self, x, w, out_dtype=None, allow_partial=False, row_tiles=0, n_waves=0, k_splits=0):
        """x [M, K] times w [N, K] transposed. float32 operands (either) take the plain
        float32 kernel. bfloat16 pairs: up to 16 rows the skinny MFMA kernel (it streams
        the weights faster than the library does there); more rows the library product,
        or this package's tiled MFMA kernel if ``library_gemm`` is off. ``allow_partial``: the consumer
        (the residual-add + norm kernel) accepts float32 split-K partial sums [S, M, N]; the
        skinny kernel then spreads a narrow output over more workgroups, and a product of 17 to
        ``parts_rows`` rows is swept with K split over workgroups instead of going to the library."""
        if isinstance(x, NormOwed):
            return self._linear_owed(x, w, out_dtype or self.dtype, n_waves)
        if isinstance(x, RowsByTile):
            # 17 to 64 rows by tile (from ``add_rmsnorm``): the product with K outermost reads them so
            if (x.data.shape[1] > 16 and w.dim() == 2 and w.dtype == torch.bfloat16 and x.shape[1] == w.shape[1]
                    and not allow_partial and self.library_gemm and not (row_tiles or n_waves or k_splits)):
                (M, K), N = x.shape, w.shape[0]
                odt = out_dtype or self.dtype
                plan = self._stream_plan(M, N, K)
                if plan is not None:
                    self._want(w, "weight")
                    key, xt = (M, N, K, odt, False), x
                    choice = self.product_choice.get(key)
                    if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                        xr = x.by_rows()
                        choice = self.product_choice[key] = self._faster(
                            lambda: self._k_outermost(plan, xt, w, torch.empty((M, N), dtype=odt, device=self.device)),
                            lambda: torch.mm(xr, w.t()) if odt == torch.bfloat16 else torch.mm(xr, w.t(), out_dtype=odt))
                    if choice != "library" and (choice == "own" or self._stream_default(M, N, K, plan)):
                        return self._k_outermost(plan, x, w, torch.empty((M, N), dtype=odt, device=self.device))
            if (x.data.shape[1] > 16 and w.dim() == 2 and w.dtype == torch.bfloat16 and x.shape[1] == w.shape[1]
                    and allow_partial and self.library_gemm and not (row_tiles or n_waves or k_splits or self._tuning)):
                # 17 to 64 rows by tile (from the decode attention or the gate / up product) into a
                # projection that ends a branch: the sweep over parts of K reads them so
                (M, K), N = x.shape, w.shape[0]
                plan = self._parts_plan(M, N, K)
                if plan is not None and self.product_choice.get((M, N, K, out_dtype or self.dtype, True)) != "library":
                    self._want(w, "weight")
                    return self._sweep_parts(plan, x, w)
            x = x.by_rows()
        self._want(x, "x")
        self._want(w, "weight")
        if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(w.shape)}")
        (M, K), N = x.shape, w.shape[0]
        out_dtype = out_dtype or self.dtype
        if x.dtype not in _DTYPE_CODE or w.dtype not in _DTYPE_CODE or out_dtype not in _DTYPE_CODE:
            raise KernelError(f"linear: dtypes {x.dtype}, {w.dtype}, {out_dtype} are not supported")
        if M == 0:
            return torch.empty((M, N), dtype=out_dtype, device=self.device)
        both_bf16 = x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
        skinny_rows = 16 if self.library_gemm else 64
        own = both_bf16 and K % 8 == 0 and K >= 8 and M <= skinny_rows
        if own and self.library_gemm and not (row_tiles or n_waves or k_splits):
            # Up to 16 rows the skinny kernel is the rule; where a tuning pass has timed both
            # for this shape and the library won (its kernels do not pay for the rows of x as
            # the skinny kernel does), the library it is. Partial sums welcome: one float32 sum.
            key = (M, N, K, out_dtype, bool(allow_partial))
            choice = self.product_choice.get(key)
            lib_dtype = torch.float32 if allow_partial else out_dtype
            by_library = (lambda: torch.mm(x, w.t()) if lib_dtype == torch.bfloat16
                          else torch.mm(x, w.t(), out_dtype=lib_dtype))
            if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                choice = self.product_choice[key] = self._faster(
                    lambda: self.linear(x, w, out_dtype, allow_partial, -1), by_library)
            if choice == "library":
                self.forms["library"] += 1
                out = by_library()
                return out.unsqueeze(0) if allow_partial else out
        explicit = row_tiles > 0 or n_waves or k_splits
        if both_bf16 and allow_partial and self.library_gemm and not (row_tiles or explicit):
            # 17 to 64 rows into the residual sum: K split over sweeping workgroups, unless a
            # tuning pass has timed both for this shape and the library won
            plan = self._parts_plan(M, N, K)
            if plan is not None:
                key = (M, N, K, out_dtype, True)
                choice = self.product_choice.get(key)
                if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                    choice = self.product_choice[key] = self._faster(
                        lambda: self._sweep_parts(plan, x, w), lambda: torch.mm(x, w.t()))
                if choice != "library":
                    return self._sweep_parts(plan, x, w)
        if both_bf16 and not allow_partial and self.library_gemm and not (row_tiles or explicit):
            # 17 to 64 rows, whole sums: K outermost, unless a tuning pass has timed both and the library won
            plan = self._stream_plan(M, N, K)
            if plan is not None:
                key = (M, N, K, out_dtype, False)
                choice = self.product_choice.get(key)
                lib_dtype = out_dtype
                if choice is None and self._tuning and not torch.cuda.is_current_stream_capturing():
                    choice = self.product_choice[key] = self._faster(
                        lambda: self._k_outermost(plan, x, w, torch.empty((M, N), dtype=out_dtype, device=self.device)),
                        lambda: torch.mm(x, w.t()) if lib_dtype == torch.bfloat16 else torch.mm(x, w.t(), out_dtype=lib_dtype))
                if choice != "library" and (choice == "own" or self._stream_default(M, N, K, plan, by_tile=False)):
                    return self._k_outermost(plan, x, w, torch.empty((M, N), dtype=out_dtype, device=self.device))
        row_tiles = max(row_tiles, 0)                     # -1: the skinny kernel, whatever the table says
        if own and not explicit and not allow_partial:
            plan = self._sweep_plan(M, N, K)
            if plan is not None:
                out = torch.empty((M, N), dtype=out_dtype, device=self.device)
                self._sweep(plan, x, w, out, 0)
                return out
        if own:
            if not (row_tiles and n_waves and k_splits):
                rw, nw, ks = c_int(0), c_int(0), c_int(0)
                self._gemm.soc_gemm_skinny_plan(c_int(M), c_int(N), c_int(K), c_int(1 if allow_partial else 0),
                                                ctypes.byref(rw), ctypes.byref(nw), ctypes.byref(ks))
                row_tiles, n_waves = row_tiles or rw.value, n_waves or nw.value
                k_splits = k_splits or ks.value
            if k_splits > 1:
                part = torch.empty((k_splits, M, N), dtype=torch.float32, device=self.device)
                out, c_ptr, p_ptr = part, None, _ptr(part)
            else:
                out = torch.empty((M, N), dtype=out_dtype, device=self.device)
                c_ptr, p_ptr = _ptr(out), None
            wt, tiled = self._by_tile(w) if M <= 16 else (w, 0)
            self.forms[f"skinny:{k_splits}"] += 1
            _check(self._gemm.soc_gemm_bf16_skinny(_ptr(x), _ptr(wt), c_ptr, p_ptr, c_int(M), c_int(N), c_int(K),
                                                   c_int(_DTYPE_CODE[out_dtype]), c_int(row_tiles),
                                                   c_int(n_waves), c_int(k_splits), c_int(tiled), self._stream()),
                   f"linear [{M}x{K}] x [{N}x{K}]^T")
            return out
        if both_bf16 and self.library_gemm:
            self.forms["library"] += 1
            if out_dtype == torch.bfloat16:
                return torch.mm(x, w.t())
            return torch.mm(x, w.t(), out_dtype=out_dtype)
        out = torch.empty((M, N), dtype=out_dtype, device=self.device)
        args = (_ptr(x), _ptr(w), _ptr(out), c_int(M), c_int(N), c_int(K))
        if both_bf16 and K % 8 == 0 and K >= 8:
            err = self._gemm.soc_gemm_bf16_mfma(*args, c_int(_DTYPE_CODE[out_dtype]), self._stream())
        else:
            err = self._gemm.soc_gemm_generic(*args, c_int(_DTYPE_CODE[x.dtype]), c_int(_DTYPE_CODE[w.dtype]),
                                              c_int(_DTYPE_CODE[out_dtype]), self._stream())
        _check(err, f"linear [{M}x{K}] x [{N}x{K}]^T")
        return out

    def _linear_owed(self, owed, w, out_dtype, n_waves=0):
        """x' [M <= 16, K] of a NormOwed times w [N, K] transposed, the norm's factor applied
        to the sums: one skinny product, bfloat16 out."""
        x = owed.x
        self._want(x, "x", torch.bfloat16)
        self._want(w, "weight", torch.bfloat16)
        if w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(w.shape)}")
        (M, K), N = x.shape, w.shape[0]
        if out_dtype != torch.bfloat16 or not 0 < M <= 16 or K % 8:
            raise KernelError("rows owed a norm go to bfloat16 products of at most 16 rows")
        out = torch.empty((M, N), dtype=torch.bfloat16, device=self.device)
        plan = self._sweep_plan(M, N, K) if not n_waves else None
        if plan is not None:
            self._sweep(plan, x, w, out, 0, self._owed_args(owed, M, K))
            return out
        if not n_waves:
            n_waves = 8
            while n_waves > 1 and K // n_waves < 128:
                n_waves //= 2
        ssq, tiles, dim, eps = self._owed_args(owed, M, K)
        wt, tiled = self._by_tile(w)
        _check(self._gemm.soc_gemm_bf16_skinny_norm(
            _ptr(x), _ptr(wt), _ptr(out), c_int(M), c_int(N), c_int(K), c_int(n_waves), ssq, c_int(tiles),
            c_int(dim), c_float(eps), None, None, None, None, c_int(1), None, None, c_int(tiled), c_int(16),
            self._stream()),
            f"linear (norm owed) [{M}x{K}] x [{N}x{K}]^T")
        return out

    # -- attention pieces ----------------------------------------------------------------------
    def _qk(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps, inv_freq, rotary_dim, positions, token_rows,
            slot, split_out):
        N = qkv.shape[0]
        self._want(qkv, "qkv", self.dtype, (N, (Hq + 2 * Hkv) * D))
        if (q_gain is None) != (k_gain is None):
            raise KernelError("q and k gains come together")
        if q_gain is not None:
            self._want(q_gain, "q gain", torch.float32, (D,))
            self._want(k_gain, "k gain", torch.float32, (D,))
        if inv_freq is not None:
            if rotary_dim % 2 or not 2 <= rotary_dim <= D:
                raise KernelError(f"rotary_dim {rotary_dim} does not fit head size {D}")
            self._want(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
            self._want(positions, "positions", torch.int32, (N,))
        q = torch.empty((N, Hq, D), dtype=self.dtype, device=self.device)
        k = v = None
        kp = vp = table = None
        width = bs = 0
        if slot is not None and Hkv:
            self._check_slot(slot, Hkv, D)
            self._want(positions, "positions", torch.int32, (N,))
            self._want(token_rows, "token_rows", torch.int32, (N,))
            kp, vp, table, width, bs = slot.k, slot.v, slot.block_table, slot.block_table.shape[1], slot.block_size
        elif split_out and Hkv:
            k = torch.empty((N, Hkv, D), dtype=self.dtype, device=self.device)
            v = torch.empty((N, Hkv, D), dtype=self.dtype, device=self.device)
        elif Hkv:
            raise KernelError("keys and values need either a cache slot or split outputs")
        if inv_freq is None and positions is None:
            positions = torch.zeros((N,), dtype=torch.int32, device=self.device)
        _check(self._ew.soc_qk_norm_rope(
            _ptr(qkv), _ptr(q), _ptr(k), _ptr(v), _ptr(kp), _ptr(vp), _ptr(table), c_int(width),
            _ptr(token_rows), _ptr(positions), _ptr(q_gain), _ptr(k_gain), _ptr(inv_freq), c_int(N),
            c_int(Hq), c_int(Hkv), c_int(D), c_int(rotary_dim), c_int(bs), c_float(eps),
            c_int(self.code), self._stream()), "qk_norm_rope")
        return q, k, v

    def _check_slot(self, slot, Hkv, D):
        self._want(slot.k, "k pool", self.dtype)
        self._want(slot.v, "v pool", self.dtype, slot.k.shape)
        self._want(slot.block_table, "block table", torch.int32)
        if slot.k.dim() != 4 or tuple(slot.k.shape[1:]) != (Hkv, slot.block_size, D):
            raise KernelError(f"cache pool {tuple(slot.k.shape)} does not fit {Hkv} kv heads, "
                              f"block size {slot.block_size}, head size {D}")

    def qk_norm_rope_write(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps, inv_freq, rotary_dim,
                           positions, token_rows, slot):
        """Norm and rotate q and k, store k and v into the pages of ``slot`` (None: queries
        only, ``Hkv`` 0). Returns q [N, Hq, D]."""
        return self._qk(qkv, Hq, Hkv, D, q_gain, k_gain, eps, inv_freq, rotary_dim, positions,
                        token_rows, slot, False)[0]

    def qk_norm_split(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps):
        """Norm q and k only; returns q, k, v as separate tensors."""
        return self._qk(qkv, Hq, Hkv, D, q_gain, k_gain, eps, None, 0, None, None, None, True)

    def rope(self, x, positions, inv_freq, rotary_dim):
        N, H, D = x.shape
        self._want(x, "x", self.dtype)
        self._want(positions, "positions", torch.int32, (N,))
        if rotary_dim % 2 or not 2 <= rotary_dim <= D:
            raise KernelError(f"rotary_dim {rotary_dim} does not fit head size {D}")
        self._want(inv_freq, "inv_freq", torch.float32, (rotary_dim // 2,))
        _check(self._ew.soc_rope(_ptr(x), _ptr(positions), _ptr(inv_freq), c_int(N), c_int(H), c_int(D),
                                 c_int(rotary_dim), c_int(self.code), self._stream()), "rope")

    def kv_write(self, k, v, positions, token_rows, slot):
        N, Hkv, D = k.shape
        self._want(k, "k", self.dtype)
        self._want(v, "v", self.dtype, k.shape)
        self._want(positions, "positions", torch.int32, (N,))
        self._want(token_rows, "token_rows", torch.int32, (N,))
        self._check_slot(slot, Hkv, D)
        _check(self._ew.soc_kv_write(_ptr(k), _ptr(v), _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table),
                                     c_int(slot.block_table.shape[1]), _ptr(token_rows), _ptr(positions),
                                     c_int(N), c_int(Hkv), c_int(D), c_int(slot.block_size),
                                     c_int(self.code), self._stream()), "kv_write")

    def plan_splits(self, n_tokens, n_kv_heads, group, max_keys):
        """How the keys of one token are cut into splits so that the launch fills the GPU."""
        if self.attention_splits is not None:
            split_len, n_splits = self.attention_splits
            if min(split_len, 1 << 24) * n_splits < max_keys:
                raise KernelError(f"{n_splits} key splits of {split_len} keys do not cover the {max_keys} keys of the "
                                  "step's longest row")
            return self.attention_splits
        chunk = 1 if group == 1 else 2 if group == 2 else 4 if group <= 4 else 8
        base = n_tokens * n_kv_heads * ((group + chunk - 1) // chunk)
        if base >= 1024 or max_keys <= 256:
            return 1 << 30, 1
        n = min((max_keys + 127) // 128, (1024 + base - 1) // base)
        split_len = ((max_keys + n - 1) // n + 63) // 64 * 64
        return split_len, (max_keys + split_len - 1) // split_len

    SHORT_PORTION = 16      # sequences of a step with fewer tokens go with the decoded tokens

    @staticmethod
    def _portion_lengths(ctx):
        """Tokens of each sequence of the step, or None if the step does not say."""
        import numpy as np
        host = getattr(ctx, "host", None)
        if host is None or "seq_qstart" not in host:
            return None
        qstart = host["seq_qstart"].astype(np.int64)
        return qstart[1:] - qstart[:-1]

    def _row_blocks(self, ctx, n_tokens, tokens_per_block, which=None):
        """int32 [blocks, 2] on the device: (first token, tokens) of each run of at most
        ``tokens_per_block`` tokens of one sequence; None when every token is a run.
        ``which``: "short" or "long" takes the sequences with fewer than SHORT_PORTION
        tokens, or the others, only."""
        import numpy as np
        lens = self._portion_lengths(ctx)
        if which is None and (lens is None or tokens_per_block == 1 or ctx.max_q_len == 1):
            # every token alone (always right; what a decode step is anyway): no list
            return None, n_tokens
        host = ctx.host
        cache = host.setdefault("row_blocks", {})
        key = (tokens_per_block, which)
        if key not in cache:
            qstart = host["seq_qstart"].astype(np.int64)[:-1]
            if which is not None:
                keep = (lens < self.SHORT_PORTION) if which == "short" else (lens >= self.SHORT_PORTION)
                qstart, lens = qstart[keep], lens[keep]
            counts = (lens + tokens_per_block - 1) // tokens_per_block
            seq = np.repeat(np.arange(len(lens)), counts)
            j = np.arange(int(counts.sum())) - np.repeat(np.cumsum(counts) - counts, counts)
            first = qstart[seq] + j * tokens_per_block
            n = np.minimum(tokens_per_block, lens[seq] - j * tokens_per_block)
            blocks = np.stack([first, n], 1).astype(np.int32)
            upload = getattr(ctx, "upload", None)
            dev = upload(blocks) if upload is not None else torch.from_numpy(blocks).to(self.device)
            cache[key] = (dev, len(blocks))
        return cache[key]

    def plan_mfma(self, n_blocks, n_kv_heads, group, max_keys):
        """(split_len, n_splits) for the MFMA kernel; an override (``attention_splits``) is
        rounded to what the kernel takes and refused beyond its limit."""
        if self.attention_splits is not None:
            split_len, n_splits = self.attention_splits
            split_len = max(16, (min(split_len, 1 << 24) + 15) // 16 * 16)
            if split_len * n_splits < max_keys:
                raise KernelError(f"{n_splits} key splits of {split_len} keys do not cover the {max_keys} keys of the "
                                  "step's longest row")
            n_splits = max(1, min(n_splits, (max_keys + split_len - 1) // split_len))
            if n_splits > 1:
                n_splits = (n_splits + 3) // 4 * 4          # four splits share a workgroup
            if n_splits > MAX_KEY_SPLITS:
                raise KernelError(f"{n_splits} key splits asked for; the MFMA attention kernel takes at "
                                  f"most {MAX_KEY_SPLITS}")
            return split_len, n_splits
        return plan_key_splits(n_blocks, n_kv_heads, group, max_keys, self.split_target_waves, self.split_min_keys)

    def _wave_attention(self, lib, q, slot, ctx, out, scale, w, rt, gpl, which):
        """The per-wave MFMA kernel with key splits and merge, for all sequences of the step
        or for its short ones (``which``), on the current stream."""
        N, Hq, D = q.shape
        Hkv = slot.k.shape[1]
        G = Hq // Hkv
        tokens_per_block = max(1, (16 * rt) >> gpl)
        blocks, n_blocks = self._row_blocks(ctx, N, tokens_per_block, which)
        split_len, n_splits = self.plan_mfma(n_blocks, Hkv, G, ctx.max_ctx_len)
        if self.attention_splits is None and n_splits > 1:
            split_len = 0           # the kernel shares every row's own keys out evenly among the splits
        part_o = part_ml = None
        if n_splits > 4:
            # the workgroups of a task (four splits each) meet in memory
            tasks = n_blocks * Hkv * ((G + 15) // 16)
            if tasks > self._split_count.numel():
                raise KernelError(f"{tasks} (row block, kv head) pairs with key splits: more than the "
                                  f"{self._split_count.numel()} arrival counts held")
            part_rows = N if blocks is None else n_blocks * tokens_per_block
            part_o = torch.empty((part_rows, Hq, n_splits // 4, D), dtype=torch.float32, device=self.device)
            part_ml = torch.empty((part_rows, Hq, n_splits // 4, 2), dtype=torch.float32, device=self.device)
        _check(lib.soc_paged_attention_mfma(
            _ptr(q), _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table),
            c_int(slot.block_table.shape[1]), _ptr(ctx.token_rows), _ptr(ctx.positions), _ptr(blocks),
            c_int(n_blocks), _ptr(out), _ptr(part_o), _ptr(part_ml), _ptr(self._split_count), c_int(N),
            c_int(Hq), c_int(Hkv), c_int(slot.block_size), c_float(scale), c_int(w), c_int(split_len), c_int(n_splits),
            c_int(rt), c_int(gpl), c_int(0), self._stream()), "paged_attention (mfma)")

    def rope_table(self, inv_freq, first_pos, n_pos, out=None):
        """Cosines and sines of positions first_pos .. first_pos + n_pos - 1 with the rotation
        kernels' own arithmetic: float32 [n_pos, 2, len(inv_freq)] (into ``out`` if given)."""
        half = inv_freq.numel()
        self._want(inv_freq, "inv_freq", torch.float32, (half,))
        if out is None:
            out = torch.empty((n_pos, 2, half), dtype=torch.float32, device=self.device)
        self._want(out, "table", torch.float32, (n_pos, 2, half))
        _check(self._ew.soc_rope_table(_ptr(inv_freq), c_int(half), c_int(first_pos), c_int(n_pos), _ptr(out),
                                       self._stream()), "rope_table")
        return out

    def decode_attention(self, qkv, Hq, Hkv, D, q_gain, k_gain, eps, rope_table, slot, ctx, scale,
                         window=None, write=True, by_tile=False, terms=None):
        """A decode step's attention straight from the QKV product's rows: per-head norm,
        rotation, the write of the new key and value, and the attention over the pages in one
        kernel. ``qkv`` [N, (Hq + 2 Hkv) D] (with ``write``) or [N, Hq D]. Returns [N, Hq D],
        or None where this form does not apply (the caller then runs the kernels one after
        the other): bfloat16 steps in which every request brings one token, head sizes in
        steps of 32 without a rotation, in steps of 64 with one (``rope_table``, over the whole
        head: a lane's slices of a head then hold both partners of every rotated pair).
        ``by_tile``: the caller hands the result to ``linear_add_norm`` or ``linear`` only, so up
        to 16 rows may come as a ``RowsByTile``."""
        if terms is not None or not scale > 0:
            return None                 # scores with further terms, or an unusual scale: the plain kernel's
        if not (self.fuse_rope and self.dtype == torch.bfloat16 and self.attention_mfma
                and getattr(ctx, "max_q_len", 0) == 1 and D % 32 == 0 and 32 <= D <= 256
                and (rope_table is None or D % 64 == 0) and slot is not None):
            return None
        N = qkv.shape[0]
        heads = Hq + 2 * Hkv if write else Hq
        if N > 65535 or Hq % Hkv:
            return None
        self._want(qkv, "qkv", self.dtype, (N, heads * D))
        if (q_gain is None) != (k_gain is None):
            raise KernelError("q and k gains come together")
        if q_gain is not None:
            self._want(q_gain, "q gain", torch.float32, (D,))
            self._want(k_gain, "k gain", torch.float32, (D,))
        if rope_table is not None:
            # [positions, 2, D / 2] from ``rope_table``, a rotation over the whole head; every
            # position of the step must lie in it
            self._want(rope_table, "rope table", torch.float32, (rope_table.shape[0], 2, D // 2))
            if rope_table.shape[0] < ctx.max_ctx_len:
                raise KernelError(f"the rotation's table holds {rope_table.shape[0]} positions, the step "
                                  f"reaches {ctx.max_ctx_len}")
        self._check_slot(slot, Hkv, D)
        self._want(ctx.positions, "positions", torch.int32, (N,))
        self._want(ctx.token_rows, "token_rows", torch.int32, (N,))
        lib = self._attention_lib(D)
        G = Hq // Hkv
        gpl = max(0, (min(G, 16) - 1).bit_length())
        split_len, n_splits = self.plan_mfma(N, Hkv, G, ctx.max_ctx_len)
        if self.attention_splits is None and n_splits > 1:
            split_len = 0           # the kernel shares every row's own keys out evenly among the splits
        part_o = part_ml = None
        if n_splits > 4:
            tasks = N * Hkv * ((G + 15) // 16)
            if tasks > self._split_count.numel():
                return None
            part_o = torch.empty((N, Hq, n_splits // 4, D), dtype=torch.float32, device=self.device)
            part_ml = torch.empty((N, Hq, n_splits // 4, 2), dtype=torch.float32, device=self.device)
        tile_rows = (N + 15) // 16 * 16 if by_tile and self.rows_by_tile and N <= 64 and (Hq * D) % 32 == 0 else 0
        tiled = tile_rows > 0
        out = torch.empty((Hq * D // 32, tile_rows, 32) if tiled else (N, Hq * D), dtype=self.dtype, device=self.device)
        self.last_attention_kernel = ("fused", 1)
        self.forms[f"fused_attention:{n_splits}"] += 1
        _check(lib.soc_paged_attention_decode_fused(
            _ptr(qkv), c_int(heads), _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table),
            c_int(slot.block_table.shape[1]), _ptr(ctx.token_rows), _ptr(ctx.positions), _ptr(out), _ptr(part_o),
            _ptr(part_ml), _ptr(self._split_count), c_int(N), c_int(Hq), c_int(Hkv), c_int(slot.block_size),
            c_float(scale), c_int(int(window) if window else 0), c_int(split_len), c_int(n_splits), c_int(gpl),
            _ptr(q_gain), _ptr(k_gain), _ptr(rope_table), c_float(eps), c_int(1 if write else 0),
            c_int(tile_rows), self._stream()), "decode_attention")
        return RowsByTile(out, N, Hq * D) if tiled else out

    def paged_attention(self, q, slot, ctx, scale, window=None, terms=None):
        """q [N, Hq, D] against the pages of each token's row; returns [N, Hq * D]. ``terms``:
        what an architecture adds to plain softmax attention, a dict with any of ``softcap``
        (float: scores become softcap * tanh(scores / softcap)), ``sinks`` (float32 [Hq]: one
        more logit per head in the softmax's sum, with no value) and ``slopes`` (float32 [Hq]:
        slope * (key position - query position) added to the scaled scores). Such a layer,
        and one whose scale is not positive, goes to the kernel that computes scores on the
        vector units, in either dtype; the MFMA kernels take plain scores only."""
        N, Hq, D = q.shape
        self._want(q, "q", self.dtype)
        Hkv = slot.k.shape[1]
        self._check_slot(slot, Hkv, D)
        if Hq % Hkv:
            raise KernelError(f"{Hq} query heads do not divide into {Hkv} kv heads")
        self._want(ctx.positions, "positions", torch.int32, (N,))
        self._want(ctx.token_rows, "token_rows", torch.int32, (N,))
        lib = self._attention_lib(D)
        out = torch.empty((N, Hq * D), dtype=self.dtype, device=self.device)
        w = int(window) if window else 0
        G = Hq // Hkv
        softcap, sinks, slopes = 0.0, None, None
        if terms:
            if set(terms) - {"softcap", "sinks", "slopes"}:
                raise KernelError(f"attention: unknown score terms {sorted(set(terms) - {'softcap', 'sinks', 'slopes'})}")
            softcap = float(terms.get("softcap") or 0.0)
            sinks, slopes = terms.get("sinks"), terms.get("slopes")
            if softcap < 0:
                raise KernelError("attention: a soft cap is positive")
            for name, t in (("sinks", sinks), ("slopes", slopes)):
                if t is not None:
                    self._want(t, name, torch.float32, (Hq,))
        plain = softcap == 0.0 and sinks is None and slopes is None and scale > 0
        if self.dtype == torch.bfloat16 and self.attention_mfma and plain:
            gpl = max(0, (min(G, 16) - 1).bit_length())
            decode = getattr(ctx, "max_q_len", 1) == 1
            if N > 65535:
                raise KernelError("more than 65535 tokens in one attention call")
            # A step that mixes long portions with decoded tokens (or short ends of prompts):
            # the long ones go to the workgroup kernel, the short ones to the per-wave kernel,
            # whose key splits a single token behind a long context needs (in the workgroup
            # kernel it would hold four waves and walk its whole context alone).
            lens = self._portion_lengths(ctx)
            long_ = None if lens is None else lens >= self.SHORT_PORTION
            mixed = not decode and long_ is not None and bool(long_.any()) and not bool(long_.all())
            n_long = int(lens[long_].sum()) if mixed else N
            # Row tiles of the workgroup kernel. 1, 2: 16 or 32 rows per wave through the
            # 16 x 16 products; 32: 32 rows per wave through the 32 x 32 products (head sizes
            # in steps of 32); 64: the same with eight waves, each four on one half of a
            # block's keys. Chosen by the number of 32-row workgroups the long portions give
            # (measured at 8 kv heads of 4 x 128 and 4 x 64, in us for 16 / 2 x 16 / 32 rows /
            # 32 rows in two key halves; 512 slots of four waves on the GPU):
            #   256 tokens from 0 (64 workgroups): 11 / 14 / 13 / 14;  512 (128): 17 / 21 / 20 / 19
            #   1,024 from 0 (256): 32 / 36 / 34 / 29;  2,048 (512): 82 / 74 / 69 / 62
            #   3,072 from 0 (768): 163 / 112 / 107 / 123;  8,192 (2,048): 941 / 650 / 633 / 695
            #   1,024 behind 3,072 (256): 117 / 122 / 111 / 89;  2,048 behind 6,144 (512): 488 / 305 / 296 / 297
            # at head size 64 the eight-wave form stays ahead or level up to 8,192 tokens.
            th = self.prompt_form_thresholds
            wg_rt = 1
            if self.attention_row_tiles in (1, 2, 32, 64):
                wg_rt = self.attention_row_tiles
                if wg_rt >= 32 and D % 32:
                    wg_rt = 1
            elif D % 32 == 0:
                n32 = (n_long // (4 * max(1, 32 >> gpl))) * Hkv * ((G + 15) // 16)
                if n32 >= th["four_waves_of_32_rows"] and D > 64:
                    wg_rt = 32
                elif n32 >= th["eight_waves"]:
                    wg_rt = 64
            elif D <= 64 and (n_long // (4 * max(1, 32 >> gpl))) * Hkv * ((G + 15) // 16) >= th["two_tiles_of_16_rows"]:
                wg_rt = 2
            wg_tokens = 4 * max(1, (32 if wg_rt >= 32 else 16 * wg_rt) >> gpl)
            # Prompt portions go to the kernel whose four waves share the K and V tiles, if it
            # has a workgroup for every compute unit (it has no key splits; measured: 512
            # tokens behind 3.5 k of context, 256 workgroups, 107 us against 187 us); a
            # shorter portion behind a long context is better served by the per-wave kernel
            # with key splits (128 tokens behind 8 k: 95 us against 196 us). An override of
            # the row tiles (tests) forces the choice.
            enough = ((n_long // wg_tokens) * Hkv * ((G + 15) // 16) >= th["workgroup_kernel"]
                      or self.attention_row_tiles is not None)
            if (self.attention_workgroup and not decode and D <= 128 and self.attention_splits is None
                    and getattr(ctx, "max_q_len", 1) >= 16 and enough):
                rt = wg_rt
                self.last_attention_kernel = ("workgroup", rt)
                blocks, n_blocks = self._row_blocks(ctx, N, wg_tokens, "long" if mixed else None)
                _check(lib.soc_paged_attention_prefill(
                    _ptr(q), _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table),
                    c_int(slot.block_table.shape[1]), _ptr(ctx.token_rows), _ptr(ctx.positions), _ptr(blocks),
                    c_int(n_blocks), _ptr(out), c_int(N), c_int(Hq), c_int(Hkv), c_int(slot.block_size),
                    c_float(scale), c_int(w), c_int(rt), c_int(gpl), self._stream()),
                    "paged_attention (prefill)")
                if mixed:
                    # after the long ones, on the same stream: side by side on a second stream
                    # was measured and is slower (35.4 ms against 32.3 ms per mixed step at 8B sizes)
                    self._wave_attention(lib, q, slot, ctx, out, scale, w, 1, gpl, "short")
                return out
            rt = self.attention_row_tiles or 1
            rt = min(rt, 4 if D <= 64 else (2 if D <= 128 else 1))      # what the kernel is built with
            self.last_attention_kernel = ("wave", rt)
            self._wave_attention(lib, q, slot, ctx, out, scale, w, rt, gpl, None)
            return out
        max_keys = ctx.max_ctx_len if not w else min(w, ctx.max_ctx_len)
        split_len, n_splits = self.plan_splits(N, Hkv, G, max_keys)
        part_o = part_ml = None
        if n_splits > 1:
            part_o = torch.empty((N, Hq, n_splits, D), dtype=torch.float32, device=self.device)
            part_ml = torch.empty((N, Hq, n_splits, 2), dtype=torch.float32, device=self.device)
        step = 65535
        for lo in range(0, N, step):
            n = min(step, N - lo)
            _check(lib.soc_paged_attention_tokens(
                _ptr(q[lo:lo + n]), _ptr(slot.k), _ptr(slot.v), _ptr(slot.block_table),
                c_int(slot.block_table.shape[1]), _ptr(ctx.token_rows[lo:lo + n]),
                _ptr(ctx.positions[lo:lo + n]), _ptr(out[lo:lo + n]),
                _ptr(part_o[lo:lo + n]) if part_o is not None else None,
                _ptr(part_ml[lo:lo + n]) if part_ml is not None else None,
                c_int(n), c_int(Hq), c_int(Hkv), c_int(slot.block_size), c_float(scale), c_int(w),
                c_int(split_len), c_int(n_splits), c_int(self.code), c_float(softcap), _ptr(sinks), _ptr(slopes),
                self._stream()), "paged_attention")
        return out

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
