"""What the kernel set's modules share: the error type, the checked call, the entry points'
signatures, and the two carriers that products hand to each other in place of plain rows."""

from __future__ import annotations

from ctypes import c_float, c_int, c_longlong, c_void_p

import torch

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
    "soc_settle_owed": [P, P, I, I, P, I, I, F, P],
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
