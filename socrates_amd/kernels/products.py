"""Matrix products of the kernel set: the forms a product can take (a workgroup per weight
tile, a sweep over tiles with x in registers, parts of K over sweeping workgroups, K outermost,
the library), the epilogues folded into them (activation, residual sum, norm) and the rule or
the measurement that chooses among them. A mixin of ``HipKernels``."""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int

import torch

from .common import _DTYPE_CODE, KernelError, NormOwed, RowsByTile, _check, _ptr


class Products:
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

    def settle(self, owed):
        """The normed rows themselves, bfloat16 [M, dim], of rows still owed their norm's factor."""
        x = owed.x
        M, dim = x.shape
        self._want(x, "x", torch.bfloat16)
        self._want(owed.ssq, "sums of squares", torch.float32)
        out = torch.empty_like(x)
        _check(self._ew.soc_settle_owed(_ptr(x), _ptr(owed.ssq), c_int(owed.tiles), c_int(owed.ssq.shape[1]), _ptr(out),
                                        c_int(M), c_int(dim), c_float(owed.eps), self._stream()), "settle")
        return out

    def _linear_owed(self, owed, w, out_dtype, n_waves=0):
        """x' [M <= 16, K] of a NormOwed times w [N, K] transposed, the norm's factor applied
        to the sums: one skinny product, bfloat16 out. Where that product does not apply (a
        float32 weight or result) the rows are settled and go the ordinary way."""
        x = owed.x
        self._want(x, "x", torch.bfloat16)
        if w.dim() != 2 or x.shape[1] != w.shape[1]:
            raise KernelError(f"linear: x {tuple(x.shape)} does not fit weight {tuple(w.shape)}")
        (M, K), N = x.shape, w.shape[0]
        if w.dtype != torch.bfloat16 or out_dtype != torch.bfloat16 or not 0 < M <= 16 or K % 8:
            # (a weight kept in float32 because the file stores it so, a float32 result: the
            # product that takes those cannot apply the factor to its sums; the rows are settled first)
            return self.linear(self.settle(owed), w, out_dtype)
        self._want(w, "weight", torch.bfloat16)
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
