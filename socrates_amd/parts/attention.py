"""Grouped-query attention over paged keys and values.

Formulas (model/qwen/qwen_kv_paged.py:147-175): q, k, v projections without bias,
heads packed by index; per-head RMSNorm of q and k, then the position encoding;
k and v go to the cache at the token's position; a query at position p in head h
scores the keys 0..p (or the last ``window`` of them) of kv head h // G with
``scale * <q, k>``, softmax in float32, and the weighted values are concatenated
by head and projected by o_proj. The reference attends within the prompt only
(qwen_kv_paged.py:167-173); here every query reads the pages, so a prompt may be
cut anywhere.
"""

from __future__ import annotations

import torch

from ..config.specs import AttentionSpec
from .registry import PagedKV, TensorDecl, build_part, register_part


class PagedAttention:
    @staticmethod
    def tensors(spec: AttentionSpec):
        q, kv, D = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim, spec.head_dim
        t = {"q_proj.weight": TensorDecl((q, spec.hidden)),
             "k_proj.weight": TensorDecl((kv, spec.hidden)),
             "v_proj.weight": TensorDecl((kv, spec.hidden)),
             "o_proj.weight": TensorDecl((spec.hidden, q))}
        if spec.qk_norm is not None:
            t["q_norm.weight"] = TensorDecl((D,), "vector")
            t["k_norm.weight"] = TensorDecl((D,), "vector")
        if spec.sinks:
            t["sinks"] = TensorDecl((spec.n_heads,), "vector")
        return t

    @staticmethod
    def cache_need(spec: AttentionSpec):
        return PagedKV(spec.n_kv_heads, spec.head_dim, spec.window)

    def __init__(self, spec: AttentionSpec, tensors, ops):
        self.spec, self.ops = spec, ops
        if spec.qk_norm is not None and spec.qk_norm.dim != spec.head_dim:
            raise ValueError("qk_norm runs over head_dim")
        # One operand for the three projections: rows [q heads | k heads | v heads].
        self.w_qkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"],
                                tensors["v_proj.weight"]], dim=0).contiguous()
        self.w_o = tensors["o_proj.weight"]
        self.q_gain = tensors.get("q_norm.weight")
        self.k_gain = tensors.get("k_norm.weight")
        self.eps = spec.qk_norm.eps if spec.qk_norm is not None else 0.0
        self.position = (build_part(spec.position, {}, ops)
                         if spec.position is not None else None)
        self.capturable = getattr(self.position, "capturable", True)
        # terms beyond plain softmax attention, for the kernel set (None: plain)
        terms = {}
        if spec.softcap is not None:
            terms["softcap"] = float(spec.softcap)
        if spec.sinks:
            terms["sinks"] = tensors["sinks"]
        if spec.distance_slopes is not None:
            terms["slopes"] = torch.tensor(spec.distance_slopes, dtype=torch.float32, device=ops.device)
        self.terms = terms or None
        self._free_layout = {"by_tile": True} if getattr(ops, "rows_by_tile", None) is not None else {}

    def reserve(self, n_positions):
        """Before the first step: what the position encoding keeps by position is made for
        the cache's longest row."""
        if hasattr(self.position, "reserve"):
            self.position.reserve(n_positions)

    takes_projection = True     # the block may supply the last product
    takes_norm_owed = True      # x goes to one product only

    def forward(self, x, ctx, slot, write=True, project=None):
        s, ops = self.spec, self.ops
        Hq, Hkv, D = s.n_heads, s.n_kv_heads, s.head_dim
        if write:
            qkv = ops.linear(x, self.w_qkv)
        else:
            # Reading another step's cache: only the queries are needed.
            qkv = ops.linear(x, self.w_qkv[: Hq * D])
            Hkv = 0
        rot = self.position.rotary() if hasattr(self.position, "rotary") else None
        o = None
        if ((self.position is None or rot is not None) and hasattr(ops, "decode_attention")
                and ctx.max_q_len == 1 and self.terms is None):
            # a decode step: norm, position encoding, cache write and attention in one kernel
            table = self.position.table(ctx.max_ctx_len) if hasattr(self.position, "table") else None
            if self.position is None or table is not None:
                # (o goes to a product and nowhere else: the kernel set may lay it out as it likes)
                o = ops.decode_attention(qkv, Hq, s.n_kv_heads, D, self.q_gain, self.k_gain, self.eps, table,
                                         slot, ctx, s.scale, s.window, write, **self._free_layout)
        if o is not None:
            pass
        elif self.position is None or rot is not None:
            inv_freq, rotary_dim = rot if rot is not None else (None, 0)
            q = ops.qk_norm_rope_write(
                qkv, Hq, Hkv, D, self.q_gain, self.k_gain, self.eps, inv_freq, rotary_dim,
                ctx.positions, ctx.token_rows, slot if write else None)
        else:
            # A position encoding without a fused form: norm, encode, then store.
            q, k, v = ops.qk_norm_split(qkv, Hq, Hkv, D, self.q_gain, self.k_gain, self.eps)
            self.position.apply(q, k, ctx.positions)
            if write:
                ops.kv_write(k, v, ctx.positions, ctx.token_rows, slot)
        if o is None:
            o = (ops.paged_attention(q, slot, ctx, s.scale, s.window) if self.terms is None
                 else ops.paged_attention(q, slot, ctx, s.scale, s.window, terms=self.terms))
        if project is not None:
            return project(o, self.w_o)
        # the block's next norm adds this output to the residual: partial sums are welcome
        return ops.linear(o, self.w_o, allow_partial=True)


register_part(AttentionSpec, PagedAttention)
