"""Attention over the paged cache and what prepares it: per-head norm, rotation and page write,
the choice among the attention kernels for a step, key splits and row blocks. A mixin of
``HipKernels``."""

from __future__ import annotations

from ctypes import c_float, c_int

import torch

from .common import KernelError, RowsByTile, _check, _ptr
from .planning import MAX_KEY_SPLITS, plan_key_splits


class Attention:
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
