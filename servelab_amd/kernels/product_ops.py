"""Matrix products: the layouts a weight is kept in, and the routes a product takes by its rows
(few-rows kernels over the tiled copy, the LDS-staged kernel, tiles over the row-major copy, the
library for the bfloat16 table's large steps; float32 kernels for the float32 table)."""
import contextlib
import ctypes
import os
import tempfile
from typing import Optional

import torch

from .values import (Deferred, KernelError, LinearWeight, PartialSums, ScaledRows, TiledRows,
                     _c_float, _p)


class ProductOps:
    def _pair_tiles(self, M, N, K, th=16) -> bool:
        """Whether a few-rows product gives its workgroups two tiles of W (16
        rows each) instead of one.  Two tiles share one pass over x; these
        kernels are bound by what the busiest CU has to pull through its L1
        (45-50 GB/s a CU at most on MI355X, W and the re-read x alike) unless HBM
        is slower still, so the choice goes by the workgroups the busiest CU
        gets times the bytes of one.  Up to 8 rows x is small enough that the
        two forms measured within a few per cent of each other on the 7B, 32B
        and 72B shapes (pairs lose 7 % where K = 8192), so one tile stays; at 16
        rows pairs gain 15-25 % on the large matrices."""
        tiles = -(-N // th)
        if tiles < 2 or M <= 8:
            return False
        w, x = th * K, min(M, 16) * K                     # bytes / 2 of a tile of W and of x
        one = -(-tiles // self._num_cus) * (w + x)
        two = -(-(-(-tiles // 2)) // self._num_cus) * (2 * w + x)
        return two < 0.97 * one

    def _skinny(self, x, weight, bias, y, M, N, K, out_f32=False, gated=False, scaled=None,
                resid=None, next_gain=None, out_parts=None, rope=None, y_tiled=False):
        """One call of the few-rows kernel (at most 16 rows) in any of its forms."""
        parts = scaled.parts if scaled is not None else None
        x_tiled = scaled.tiled if scaled is not None else 0
        if isinstance(x, TiledRows):
            x_tiled, x = x.shape[0], x.data
        # (the product that adds to the stream reads the copy in lower tiles, where the matrix has one)
        wt, th = self._producer_copy(weight, M) if resid is not None else (weight.tiled, 16)
        pair = self._pair_tiles(M, N, K, th)
        self._call("gemm", "sl_gemm_skinny", _p(x), _p(wt), _p(bias), _p(y), M, N, K,
                   int(out_f32), int(gated), _p(parts), parts.shape[0] if parts is not None else 0,
                   _c_float(scaled.eps if scaled is not None else 0.0),
                   _p(scaled.rows) if scaled is not None else None, _p(resid), _p(next_gain),
                   _p(out_parts), ctypes.byref(rope) if rope is not None else None,
                   int(pair), int(x_tiled), int(y_tiled), th, int(M <= 8 and not pair and self.PAIR_X_LOADS))

    # --------------------------------------------------------------- linear
    def plan_weights(self, total_bytes: int) -> str:
        """Choose the layout for a model whose matrices take ``total_bytes``
        (called before the matrices are loaded)."""
        if self.act_dtype == torch.bfloat16:
            total = torch.cuda.get_device_properties(self.device).total_memory
            self.weight_layout = "dual" if 2 * total_bytes <= self.DUAL_MEMORY_SHARE * total else "tiled"
            # "tiled": as many matrices as fit below ROWS_COPIES_MEMORY_SHARE keep their row-major copy as
            # well, in the order in which they are loaded; the products of many rows of the others go
            # through the scratch buffer
            self._rows_budget = 0 if self.weight_layout == "dual" else \
                max(0, int(self.ROWS_COPIES_MEMORY_SHARE * total) - total_bytes)
            # a third copy of the matrices that add to the stream (about a third of all), in lower tiles
            self.lower_tiles = self.weight_layout == "dual" and 2.35 * total_bytes <= self.LOWER_TILES_MEMORY_SHARE * total
        return self.weight_layout

    def layout_summary(self) -> str:
        """The layout in words, for records: "dual", "rows", or "tiled" with how many of the
        matrices kept a row-major copy as well."""
        if self.weight_layout != "tiled" or not self._matrices_with_rows:
            return self.weight_layout
        return f"tiled, {self._matrices_with_rows} of {self._matrices} matrices also row-major"

    def producer_tile_height(self, N, rows=8):
        """(rows per tile, rows of x from which it pays) for the few-rows product of a matrix of N rows that
        adds to the residual stream.  At 8 rows and more such a product takes as long as its busiest CU needs
        to pull its tiles of W and its re-read of x, so the tiles should go round the CUs evenly: of 16, 14,
        12, 10 and 8 rows the height is taken whose busiest CU pulls least; 16 unless another saves
        LOWER_TILES_MIN_GAIN of it.  Measured on MI355X (us at 1 / 4 / 8 / 16 rows, tiles of 16 against the
        choice): 3584 x 18944, 14 rows (256 tiles on 256 CUs instead of 224): 23.8 / 25.7 / 29.4 / 38.6 against
        25.8 / 26.2 / 28.0 / 33.8; 5120 x 27648, 10 rows (512 tiles instead of 320, two on a quarter of the
        CUs): 57.6 / 61.2 / 68.9 against 54.1 / 52.6 / 56.1; 2048 x 11008, 8 rows (256 tiles instead of 128):
        12.3 / 13.5 / 15.5 against 12.1 / 12.6 / 13.7.  Where the busiest CU pulls less W (fewer rounds, or
        idle CUs put to work at half the tile) the lower tiles win from one row on; where only the re-read
        of x per tile of W shrinks (3584), from 8 rows on: below, HBM is the limit, and it streams tiles of
        1 KB a k-step a little faster.  (Timed with x in plain rows; with x laid out by k-step, as the engine
        hands it over, the 3584 case gains nothing end to end, which is why the default minimum gain leaves
        it at 16 rows.)"""
        def busiest(th, x):
            return -(-(-(-N // th)) // self._num_cus) * (th + x)
        # (a tile is one sum of squares a row for the products that read the stream next: the kernel that keeps
        # x in registers adds up 256 of them, 512 for rows of more than 4,096 values, as the others do)
        most = 256 if N <= 4096 else 512
        heights = [th for th in (16, 14, 12, 10, 8) if th == 16 or -(-N // th) <= most]
        best = min(heights, key=lambda th: (busiest(th, rows), -th))
        if busiest(best, rows) > (1 - self.LOWER_TILES_MIN_GAIN) * busiest(16, rows):
            return 16, 1
        return best, (1 if busiest(best, 0) <= 0.8 * busiest(16, 0) else 8)

    def _producer_copy(self, weight, M):
        """(tiled copy, its tile height) that the product adding ``M`` rows to the stream reads."""
        if weight.lower is not None and M >= weight.lower_from:
            return weight.lower, weight.th
        return weight.tiled, 16

    def prepare_weight(self, w, keep_rows=False, residual_delta=False, _th=None):
        """Called once per matrix at load: returns what ``linear`` takes.
        ``keep_rows``: the caller holds the row-major tensor anyway (a tied
        embedding table), so keeping it costs nothing.  ``residual_delta``: the
        matrix's products are only ever added to the residual stream."""
        N, K = w.shape
        self._check(w, self.act_dtype, None, "weight")
        if self.act_dtype != torch.bfloat16:
            return LinearWeight(w)
        if K % 32 or self.weight_layout == "rows":
            self.graph_rows_limit = min(self.graph_rows_limit, self.ROWS_KERNEL_MAX_M)
            return LinearWeight(w)
        tiled = torch.empty(-(-N // 16) * 16 * K, dtype=torch.bfloat16, device=self.device)
        self._call("gemm", "sl_tile_weight", _p(w), _p(tiled), N, K, 16)
        self._matrices += 1
        if self.weight_layout == "tiled" and not keep_rows and 2 * N * K > self._rows_budget:
            weight = LinearWeight(None, tiled, (N, K))
        else:
            if self.weight_layout == "tiled" and not keep_rows:
                self._rows_budget -= 2 * N * K
            self._matrices_with_rows += 1
            weight = LinearWeight(w, tiled)
        if residual_delta and self.fuse_norms and self.lower_tiles:
            th, lower_from = (_th, 1) if _th is not None else self.producer_tile_height(N)
            if th != 16:
                weight.lower = torch.empty(-(-N // th) * th * K, dtype=torch.bfloat16, device=self.device)
                weight.th, weight.lower_from = th, lower_from
                self._call("gemm", "sl_tile_weight", _p(w), _p(weight.lower), N, K, th)
        self.graph_rows_limit = min(self.graph_rows_limit, self._few_rows_limit(weight))
        return weight

    def rows_of(self, weight):
        """The row-major matrix of a weight; for a tiled-only weight it is
        written into the scratch buffer (valid until the next call)."""
        if weight.w is not None:
            return weight.w
        N, K = weight.shape
        if self._untiled is None or self._untiled.numel() < N * K:
            self._untiled = None
            self._untiled = torch.empty(N * K, dtype=torch.bfloat16, device=self.device)
        out = self._untiled[:N * K].view(N, K)
        self._call("gemm", "sl_untile_weight", _p(weight.tiled), _p(out), N, K, 16)
        return out


    def linear(self, x, weight, bias, out_f32=False, defer=False):
        """y = x W^T (+ bias); ``weight`` is a LinearWeight or a plain [N, K] tensor.
        ``defer``: y will only be added to the residual stream, so the product
        may be left to the norm that adds it: up to 16 rows a ``Deferred`` comes
        back (the norm's kernel runs the product), at 17..64 rows ``PartialSums``
        of a product whose K was split (the norm adds them up).

        bfloat16, by rows of x: 1..16 the few-rows kernel over the tiled weight,
        17..64 the wide or the LDS-staged kernel (by the size of W; the latter
        up to 128 rows), more the library, or that many rows at a time through
        those kernels when the result is wanted in float32.  float32: the wavefront-per-column kernel up to 16 rows, the
        tiled FMA kernel above; never a library product."""
        if not isinstance(weight, LinearWeight):
            weight = LinearWeight(weight)
        if isinstance(x, ScaledRows):
            return self._linear_scaled(x, weight, bias, out_f32, False)
        M, K = x.shape
        N = weight.shape[0]
        if isinstance(x, TiledRows) and not (defer and self.fuse_norms and not out_f32 and N <= 8192):
            # (rows by k-step are read by the few-rows kernel only, which is where they come from)
            if weight.shape != (N, K):
                raise KernelError(f"weight has shape {list(weight.shape)}, x has {K} columns")
            y = self._new((M, N), torch.float32 if out_f32 else None)
            self._skinny(x, weight, bias, y, M, N, K, out_f32)
            return y
        if (defer and self.fuse_norms and not out_f32 and 0 < M <= self._fused_rows(N)
                and weight.tiled is not None and weight.shape == (N, K) and N <= 8192):
            return Deferred(x, weight, bias)
        self._check(x, self.act_dtype, None, "x")
        if weight.shape != (N, K):
            raise KernelError(f"weight has shape {list(weight.shape)}, x has {K} columns")
        if weight.w is not None:
            self._check(weight.w, self.act_dtype, (N, K), "weight")
        if bias is not None:
            self._check(bias, torch.float32, (N,), "bias")
        if self.act_dtype == torch.float32:
            if K % 4 == 0 and M <= self.ROWS_KERNEL_MAX_M:
                return self.linear_rows(x, weight.w, bias, out_f32)
            if K % 16 == 0 and M >= self.F32_MFMA_MIN_M:
                return self.linear_f32_mfma(x, weight.w, bias)
            return self.linear_tiled(x, weight.w, bias, out_f32)
        limit = self._few_rows_limit(weight)
        plan = self._block_plan(M, N, K, weight)
        if plan:
            # (deferred: the norm adds the partial sums)
            return self.linear_block(x, weight, bias, out_f32, plan[0],
                                     partial=defer and self.fuse_norms and not out_f32, square=plan[1])
        if (defer and self.fuse_norms and not out_f32 and self._wide_from(N) <= M <= limit
                and K % 32 == 0 and N % 4 == 0 and self._takes_mid(M, N, K)):
            return self.linear_mid(x, weight, bias, partial=True,     # the norm adds the partial sums
                                   target=self.MID_DEFERRED_WORKGROUPS)
        if M <= limit:
            return self.linear_skinny(x, weight, bias, out_f32)
        if out_f32 and limit:
            # float32 results of many rows (the head for more requests than the few-rows kernels take,
            # logits of every position).  With a row-major copy of W: the library's product with its
            # float32 sums kept, one pass over W (7B shape, the head for 144 requests: 150 us; the
            # few-rows kernels stream W once per `limit` rows, 128 + 16 rows in 236 + 178 us).  Without:
            # those, several times faster than the plain tiled kernel below.
            if weight.w is not None:
                sums = self.library_sums(x, weight.w, torch.float32)
                return sums if bias is None else sums.add_(bias)
            return torch.cat([self.linear_skinny(x[i:i + limit], weight, bias, True)
                              for i in range(0, M, limit)])
        w = self.rows_of(weight)
        if M <= self.ROWS_KERNEL_MAX_M and K % 8 == 0:
            return self.linear_rows(x, w, bias, out_f32)
        if out_f32:
            if M <= 4 * self.ROWS_KERNEL_MAX_M and K % 8 == 0:
                return self.linear_rows(x, w, bias, out_f32)
            return self.linear_tiled(x, w, bias, out_f32)
        return self.linear_library(x, w, bias)

    def linear_wide(self, x, weight, bias, out_f32=False, gated=False):
        M, K = x.shape
        N = weight.shape[0]
        if weight.tiled is None:
            raise KernelError("linear_wide needs the tiled copy of the weight")
        y = self._new((M, N // 2 if gated else N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_wide", _p(x), _p(weight.tiled), _p(bias), _p(y), M, N, K,
                   int(out_f32), int(gated))
        return y

    def _takes_mid(self, M, N, K) -> bool:
        return N * K >= (self.MID_MIN_ELEMENTS if M <= 32 else self.MID_MIN_ELEMENTS_MANY)

    MID_MAX_M = 128               # the LDS-staged kernel takes up to this many rows

    def _few_rows_limit(self, weight) -> int:
        """Up to how many rows of x a product with this weight stays with the
        kernels that stream the tiled copy (more rows: the library): none
        without a tiled copy, SKINNY_MAX_M, or MID_MAX_M where the LDS-staged
        kernel takes the matrix."""
        if weight.tiled is None or self.act_dtype != torch.bfloat16:
            return 0
        N, K = weight.shape
        if K % 32 == 0 and N * K >= self.MID_MIN_ELEMENTS_MANY:
            return self.MID_MAX_M
        return self.SKINNY_MAX_M

    def linear_mid(self, x, weight, bias, out_f32=False, gated=False, ks=None, partial=False,
                   target=None):
        """17..128 rows with x staged through LDS; K split over workgroups when
        N alone gives too few of them.  ``partial``: a split product comes back
        as ``PartialSums`` for its reader to add up."""
        M, K = x.shape
        N = weight.shape[0]
        if weight.tiled is None:
            raise KernelError("linear_mid needs the tiled copy of the weight")
        wgs = -(-(-(-N // 16)) // 8)
        if ks is None:
            if target is None:
                target = self.MID_PARTIAL_WORKGROUPS if partial else self.MID_TARGET_WORKGROUPS
            ks = 1 if gated else max(1, min(16, K // 32 // 4, -(-target // wgs)))
        part = self._new((ks, M, N), torch.float32) if ks > 1 else None
        if partial and ks > 1:
            self._call("gemm", "sl_gemm_mid", _p(x), _p(weight.tiled), None, None, M, N, K,
                       0, 0, int(ks), self.MID_WIDE_WORKGROUPS, self._num_cus, _p(part))
            return PartialSums(part, bias)
        y = self._new((M, N // 2 if gated else N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_mid", _p(x), _p(weight.tiled), _p(bias), _p(y), M, N, K,
                   int(out_f32), int(gated), int(ks), self.MID_WIDE_WORKGROUPS, self._num_cus, _p(part))
        return y

    def _block_plan(self, M, N, K, weight):
        """How the block kernel takes a product of M rows: (shares of K, square tiles), or None
        when the product is not one of its own: bfloat16, a row-major copy of the weight, K in
        chunks of 64, a matrix of few rows (its tiles alone would leave most CUs idle, which is
        what the split repairs) but of BLOCK_MIN_ELEMENTS elements at least (smaller ones stay
        with the kernels they were measured on).  Tiles of 256 x 128 for BLOCK_MIN_M to BLOCK_MAX_M
        rows of x; tiles of 256 x 256 for matrices with long rows (K of BLOCK_SQUARE_MIN_K and
        more: the down projection) from 257 to BLOCK_SQUARE_MAX_M rows, if their tiles and shares
        fill three quarters of the CUs.  As many shares as give every CU a workgroup, 16 at most,
        of at least 3 chunks each (7B shape, down projection at 256 rows: 70 / 44 / 41 us with 4 / 8
        / 9 shares; q/k/v: 21 / 17 / 26 us with 4 / 7 / 8, the last being more workgroups than CUs;
        down at 527 rows: 84 us in square tiles, 101 us in 256 x 128, 130 us in the library's tuned
        kernel; at 1,024 rows 111 us in 4 shares, 144 us in 6)."""
        w = weight.w if isinstance(weight, LinearWeight) else weight
        if (self.act_dtype != torch.bfloat16 or not self.use_block_products or w is None
                or K % 64 or N % 4 or N > self.BLOCK_MAX_N or N * K < self.BLOCK_MIN_ELEMENTS):
            return None
        if K >= self.BLOCK_SQUARE_MIN_K and 256 < M <= self.BLOCK_SQUARE_MAX_M:
            tiles = -(-N // 256) * -(-M // 256)
            shares = min(16, K // 64 // 3, self._num_cus // tiles)
            if shares >= 1 and 4 * tiles * shares >= 3 * self._num_cus:
                return shares, True
        if not self.BLOCK_MIN_M <= M <= self.BLOCK_MAX_M:
            return None
        tiles = -(-N // 128) * -(-M // 256)
        return max(1, min(16, K // 64 // 3, self._num_cus // tiles)), False

    def linear_block(self, x, weight, bias, out_f32=False, ks=1, partial=False, square=False):
        """A few hundred rows over the row-major copy of the weight: workgroups
        own a tile of 256 rows of x by 128 rows of W (``square``: by 256) over
        one of ``ks`` shares of K.  ``partial``: the product comes back as
        ``PartialSums`` for its reader to add up."""
        M, K = x.shape
        N = weight.shape[0]
        w = weight.w if isinstance(weight, LinearWeight) else weight
        if w is None:
            raise KernelError("linear_block needs the row-major copy of the weight")
        self._check(x, self.act_dtype, (M, K), "x")
        self._check(w, self.act_dtype, (N, K), "weight")
        part = self._new((ks, M, N), torch.float32) if ks > 1 or partial else None
        if partial:
            if ks > 1:
                self._call("gemm", "sl_gemm_block", _p(x), _p(w), None, None, M, N, K, 0, int(ks), int(square),
                           _p(part))
            else:
                self._call("gemm", "sl_gemm_block", _p(x), _p(w), None, _p(part), M, N, K, 1, 1, int(square), None)
            return PartialSums(part, bias)
        y = self._new((M, N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_block", _p(x), _p(w), _p(bias), _p(y), M, N, K, int(out_f32),
                   int(ks), int(square), _p(part))
        return y

    def linear_skinny(self, x, weight, bias, out_f32=False):
        M, K = x.shape
        N = weight.shape[0]
        if weight.tiled is None:
            raise KernelError("linear_skinny needs the tiled copy of the weight")
        if M >= self._wide_from(min(N, K)):       # (the stream is what a projection reads or what it writes)
            if self._takes_mid(M, N, K):
                return self.linear_mid(x, weight, bias, out_f32)
            return self.linear_wide(x, weight, bias, out_f32)
        y = self._new((M, N), torch.float32 if out_f32 else None)
        self._skinny(x, weight, bias, y, M, N, K, out_f32)
        return y

    def _linear_scaled(self, xs, weight, bias, out_f32, gated, y_tiled=False):
        """The consumer of un-normalised rows: one few-rows product that scales
        its result rows by rsqrt(mean x^2 + eps)."""
        M, K = xs.shape
        N = weight.shape[0]
        if weight.tiled is None or weight.shape != (N, K) or M > self.FUSED_NORM_MAX_M:
            raise KernelError("un-normalised rows need a tiled weight and at most 16 rows")
        if bias is not None:
            self._check(bias, torch.float32, (N,), "bias")
        y = self._new((M, N // 2 if gated else N), torch.float32 if out_f32 else None)
        if self._takes_resident(N, K, xs.parts.shape[0]):
            self._call("gemm", "sl_gemm_resident", _p(xs.x), _p(weight.tiled), _p(bias), _p(y), M, N, K,
                       int(out_f32), int(gated), _p(xs.parts), xs.parts.shape[0], _c_float(xs.eps),
                       _p(xs.rows), int(xs.tiled), int(y_tiled))
        else:
            self._skinny(xs.x, weight, bias, y, M, N, K, out_f32, gated, scaled=xs, y_tiled=y_tiled)
        return TiledRows(y, (M, N // 2)) if y_tiled else y

    def _takes_resident(self, N, K, parts) -> bool:
        """Whether a consumer product runs on the workgroups that stay and walk the tiles
        (x in registers, row scales computed once): matrices with several tiles per CU whose
        row length the kernel is built for (the library says which: ``sl_gemm_resident_parts``,
        the most sums of squares a row its kernel for K adds up, 0 for no kernel).  Every other
        width takes the workgroup-per-tile kernel, which gives the same result bit for bit."""
        if -(-N // 16) < self.RESIDENT_MIN_ROUNDS * self._num_cus:
            return False
        most = self._resident_k.get(K)
        if most is None:
            most = self._resident_k[K] = int(self._lib["gemm"].sl_gemm_resident_parts(K))
        return 0 < parts <= most

    GATE_BLOCK = 8                # gate and up rows alternate in blocks of 8 (half an MFMA tile)

    def gated_linear(self, x, weight, block, _tiled_out=False):
        """silu(x Wg^T) * (x Wu^T) for a weight whose rows hold gate and up
        interleaved in blocks of ``block`` rows (``block`` = I: plain [Wg; Wu]).
        Few rows and a tiled weight with blocks of 8: one fused kernel."""
        if not isinstance(weight, LinearWeight):
            weight = LinearWeight(weight)
        if isinstance(x, ScaledRows):
            if block != self.GATE_BLOCK or weight.shape[0] % 16:
                raise KernelError("un-normalised rows need gate and up in blocks of 8")
            return self._linear_scaled(x, weight, None, False, True, y_tiled=_tiled_out)
        M, K = x.shape
        N = weight.shape[0]
        if (_tiled_out and M < self._wide_from(K) and M <= self._few_rows_limit(weight)
                and block == self.GATE_BLOCK and N % 16 == 0):
            self._check(x, self.act_dtype, None, "x")
            y = self._new((M, N // 2))
            self._skinny(x, weight, None, y, M, N, K, gated=True, y_tiled=True)
            return TiledRows(y, (M, N // 2))
        if M <= self._few_rows_limit(weight) and block == self.GATE_BLOCK and N % 16 == 0:
            self._check(x, self.act_dtype, None, "x")
            if M >= self._wide_from(K):
                if self._takes_mid(M, N, K):
                    return self.linear_mid(x, weight, None, gated=True)
                return self.linear_wide(x, weight, None, gated=True)
            y = self._new((M, N // 2))
            self._skinny(x, weight, None, y, M, N, K, gated=True)
            return y
        return self.silu_mul(self.linear(x, weight, None), block)

    def gated_mlp(self, x, w_gate_up, block, w_down, defer=False):
        """down(silu(gate x) * (up x)): ``gated_linear`` followed by ``linear``.  With few rows the
        kernel table keeps what lies between them in the layout its second kernel reads best
        (rows by k-step: the eight rows of a decode step then cost the down product half as many
        cache lines per load of x)."""
        if not isinstance(w_gate_up, LinearWeight):
            w_gate_up = LinearWeight(w_gate_up)
        if not isinstance(w_down, LinearWeight):
            w_down = LinearWeight(w_down)
        M = x.shape[0]
        inner = w_gate_up.shape[0] // 2
        tiled = (self.act_dtype == torch.bfloat16 and self.tile_few_rows and 1 < M <= self._fused_rows(w_down.shape[0])
                 and block == self.GATE_BLOCK and inner % 32 == 0 and w_gate_up.tiled is not None
                 and w_down.tiled is not None and w_down.shape[1] == inner and w_gate_up.shape[0] % 16 == 0)
        h = self.gated_linear(x, w_gate_up, block, _tiled_out=tiled)
        return self.linear(h, w_down, None, defer=defer)

    def linear_rows(self, x, w, bias, out_f32=False):
        M, K = x.shape
        N = w.shape[0]
        y = self._new((M, N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_rows", _p(x), _p(w), _p(bias), _p(y), M, N, K, int(out_f32),
                   int(self.ROWS_THROUGH_LDS))
        return y

    def linear_tiled(self, x, w, bias, out_f32=False):
        M, K = x.shape
        N = w.shape[0]
        y = self._new((M, N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_tiled", _p(x), _p(w), _p(bias), _p(y), M, N, K, int(out_f32))
        return y

    # (library products of fewer than LIBRARY_PADDED_MAX_M rows run on a multiple of LIBRARY_ROW_STEP
    # rows: few distinct shapes, each of which can be tuned)

    def library_rows(self, M: int) -> int:
        """The number of rows a library product of M rows of x runs with."""
        if M >= self.LIBRARY_PADDED_MAX_M:
            return M
        return -(-M // self.LIBRARY_ROW_STEP) * self.LIBRARY_ROW_STEP

    F32_MFMA_MIN_M = 17           # float32 products of this many rows or more run on the matrix cores

    def linear_f32_mfma(self, x, w, bias):
        """Float32 product by float32 matrix instructions (float32 inputs and sums,
        no reduced-precision mode); K % 16 == 0."""
        if self.act_dtype != torch.float32:
            raise KernelError("linear_f32_mfma is for the float32 table only")
        M, K = x.shape
        N = w.shape[0]
        y = self._new((M, N), torch.float32)
        self._call("gemm", "sl_gemm_f32_mfma", _p(x), _p(w), _p(bias), _p(y), M, N, K)
        return y

    def library_sums(self, x, w, out_dtype=None):
        """x w^T by the library, in bfloat16 or (``out_dtype`` float32) with the
        float32 sums kept.  Fewer than LIBRARY_PADDED_MAX_M rows are padded to a
        multiple of LIBRARY_ROW_STEP; the rows beyond M hold whatever the buffer
        held: a row of a product depends on its own row of x only (the library
        splits no K across rows), and they are cut off."""
        if self.act_dtype != torch.bfloat16:
            raise KernelError("the library GEMM is for the bfloat16 table only")
        M = x.shape[0]
        rows = self.library_rows(M)
        if rows != M:
            padded = self._new((rows, x.shape[1]))
            padded[:M].copy_(x)
            x = padded
        if out_dtype is None:
            return torch.mm(x, w.t())[:M]
        return torch.mm(x, w.t(), out_dtype=out_dtype)[:M]

    def linear_library(self, x, w, bias):
        """Many rows: the library's product.  A bias is added to the float32
        sums before the one rounding to bfloat16, as the few-rows kernels do, so
        that a row gives the same values whichever path its step takes."""
        if bias is None:
            return self.library_sums(x, w)
        return self.library_sums(x, w, torch.float32).add_(bias).to(torch.bfloat16)

    @contextlib.contextmanager
    def library_tuning(self, max_ms: int = 30, results_file: Optional[str] = None):
        """Inside the block, every new shape of a library product is timed over
        the library's own candidate kernels (PyTorch's TunableOp, at most
        ``max_ms`` a candidate) and the fastest is kept for that exact shape;
        afterwards tuned shapes keep their choice and every other shape takes
        the library's default.  The choices are also written to
        ``results_file`` (default: a file in the temporary folder), which a
        later process reads instead of timing again.  The library's pick for
        the 7B shape's prompt products measured 26 % slower than the tuned one
        on MI355X."""
        tunable = getattr(torch.cuda, "tunable", None)
        if tunable is None:                      # a PyTorch without TunableOp: the library's defaults stay
            yield
            return
        if results_file is None:
            results_file = os.path.join(tempfile.gettempdir(),
                                        f"servelab_amd_tunableop_{os.getuid()}.csv")
        tunable.set_filename(results_file)
        tunable.set_max_tuning_duration(int(max_ms))
        tunable.enable(True)
        tunable.tuning_enable(True)
        try:
            yield
        finally:
            tunable.tuning_enable(False)           # the choices made stay in use; nothing new is timed
