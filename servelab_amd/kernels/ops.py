"""The kernel table: every device computation of the engine, as calls into the
hand-written HIP libraries (ctypes, C ABI, the caller's current stream).

There is no fallback: without a GPU, without hipcc-built libraries, or for a
size a kernel refuses, a call raises.  Shapes, dtypes and contiguity are
checked here on the host before any launch, because a kernel that reads out of
bounds can take the GPU down.

Large bfloat16 matrix products (more rows than the hand-written few-rows
kernel takes) go to the library GEMM behind ``torch.addmm`` — where the
reference calls ``F.linear`` (servelab/parallel/layers.py:164-180).  The
float32 table never does: its products are the hand-written float32 kernels
(FMA, and float32 matrix instructions for many rows).
"""
import contextlib
import ctypes
import os
import tempfile
from typing import Optional

import torch

from . import build
from .tuning import Tuning

_c_int, _c_float, _c_void_p = ctypes.c_int, ctypes.c_float, ctypes.c_void_p


class KernelError(RuntimeError):
    pass


def _p(t: Optional[torch.Tensor]):
    return None if t is None else _c_void_p(t.data_ptr())


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


class _RopeStore(ctypes.Structure):
    """``RopeStore`` of gemm.hip."""
    _fields_ = [("cosv", _c_void_p), ("sinv", _c_void_p), ("slots", _c_void_p), ("kc", _c_void_p),
                ("vc", _c_void_p), ("nh", _c_int), ("nkv", _c_int), ("D", _c_int), ("page", _c_int),
                ("rot", _c_int), ("qscale", _c_float)]


class RotationPlan:
    """How the kernels of this table want the q and k channels of a head laid
    out for a position encoding, decided once at load (``plan_rotation``):
    ``order`` is the permutation the mixer applies to the rows of its q and k
    matrices and biases (new channel i is old channel ``order[i]``; None: as
    they are), ``rot_dim`` how many leading channels are rotated, ``blocked``
    whether the rotated channels lie in blocks of 8 followed by their 8
    partners (what the fused q/k/v kernel rotates) or as first and second half."""
    __slots__ = ("order", "rot_dim", "blocked")

    def __init__(self, order, rot_dim, blocked):
        self.order, self.rot_dim, self.blocked = order, int(rot_dim), bool(blocked)


class LinearWeight:
    """A weight matrix [N, K] as the products read it: row-major (``w``) for
    products with many rows, tiled (``tiled``, bfloat16 only) for the few-rows
    kernels that decode steps use.  Both, or one of them.  ``lower``: a further
    tiled copy in tiles of ``th`` < 16 rows, for the few-rows product that adds
    to the residual stream (see ``HipOps.producer_tile_height``)."""
    __slots__ = ("w", "tiled", "shape", "lower", "th", "lower_from")

    def __init__(self, w, tiled=None, shape=None):
        self.w, self.tiled = w, tiled
        self.shape = tuple(w.shape) if w is not None else tuple(shape)
        self.lower, self.th, self.lower_from = None, 16, 1          # lower_from: rows from which ``lower`` is read


class Deferred:
    """A product whose result is only ever added to the residual stream; the
    norm that takes it as its delta runs it, fused with the add and the norm
    (``HipOps.add_rmsnorm(..., fuse=True)``) or plainly (``materialize``)."""
    __slots__ = ("x", "weight", "bias")

    def __init__(self, x, weight, bias):
        self.x, self.weight, self.bias = x, weight, bias


class TiledRows:
    """Few rows of activations [M, K] laid out by k-step (element (m, k) at
    (k // 32) * (M * 32) + m * 32 + k % 32): what a gated product writes for the
    product that reads it (``HipOps.gated_mlp``).  Never leaves the kernel table."""
    __slots__ = ("data", "shape")

    def __init__(self, data, shape):
        self.data, self.shape = data, tuple(shape)

    def rows(self):
        M, K = self.shape
        return self.data.view(K // 32, M, 32).permute(1, 0, 2).reshape(M, K)


class PartialSums:
    """A product whose K was split over workgroups, left as float partial sums
    ``parts`` [ks, T, N] with the bias not yet added, for a reader that adds
    them up on its way (``rope_store``, ``add_rmsnorm``); ``HipOps.materialize``
    makes the plain tensor."""
    __slots__ = ("parts", "bias")

    def __init__(self, parts, bias):
        self.parts, self.bias = parts, bias


class ScaledRows:
    """Rows [T, H] that are normalised but for the factor rsqrt(mean x^2 + eps):
    ``x`` holds stream * gain in the activation dtype, ``parts`` [nparts, 16] the
    sums of squares of the stream by row.  Only ``linear`` and ``gated_linear``
    read them: they scale their result rows instead.  ``rows`` optionally
    selects which rows take part."""
    __slots__ = ("x", "parts", "eps", "rows", "tiled")

    def __init__(self, x, parts, eps, rows=None, tiled=0):
        self.x, self.parts, self.eps, self.rows = x, parts, eps, rows
        self.tiled = tiled          # x is laid out by k-step (see TiledRows) with this many rows; 0: plain rows

    @property
    def shape(self):
        return (self.rows.shape[0] if self.rows is not None else self.x.shape[0], self.x.shape[1])

    def plain_x(self):
        """``x`` as plain rows (a copy when it is laid out by k-step)."""
        if not self.tiled:
            return self.x
        T, K = self.x.shape
        return self.x.reshape(K // 32, T, 32).permute(1, 0, 2).reshape(T, K)


class HipOps:
    ROWS_KERNEL_MAX_M = 16        # the wavefront-per-column GEMM is used up to this many rows
    SKINNY_MAX_M = 64             # the matrix-core few-rows GEMM takes up to this many rows

    # Decode reads every weight once per step and is bound by how fast it
    # streams; the tiled layout streams faster (see gemm.hip).  Layouts:
    #   "dual"   row-major and tiled (twice the memory): library GEMM for many
    #            rows, few-rows kernels for decode;
    #   "tiled"  tiled only: a product with many rows first writes the matrix
    #            row-major into a scratch buffer (one extra pass over the matrix
    #            per product, only while prompts are being processed);
    #   "rows"   row-major only: decode uses the slower row-major kernels.
    # ``plan_weights(total_bytes)`` picks "dual" while two copies stay below
    # DUAL_MEMORY_SHARE of the device's memory, else "tiled".
    #
    # The numbers that choose between kernels (DUAL_MEMORY_SHARE, WIDE_MIN_M, MID_*, TARGET_WAVES,
    # SHARED_ATTENTION_*, ...) are the fields of ``tuning.Tuning``, set on the table at construction.

    def __init__(self, act_dtype: torch.dtype, device="cuda:0", tuning: Optional[Tuning] = None):
        if act_dtype not in (torch.bfloat16, torch.float32):
            raise KernelError(f"kernels exist for bfloat16 and float32, not {act_dtype}")
        if not torch.cuda.is_available():
            raise KernelError("servelab_amd needs a GPU: the HIP kernels have no CPU fallback")
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        self.tuning = tuning if tuning is not None else Tuning()
        self.tuning.apply(self)
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        # the current stream's handle without the wrapper objects torch.cuda.current_stream() builds
        # (a launch is a few microseconds of host time, and this was one of them)
        self._raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        self.dtype_name = "float32" if act_dtype == torch.float32 else "bfloat16"
        units = [build.unit(stem, self.dtype_name) for stem in build.DEFAULT_STEMS]
        build.ensure(units)
        self._lib = {stem: build.load(build.unit(stem, self.dtype_name))
                     for stem in build.DEFAULT_STEMS}
        self._fn = {}
        self.use_mfma_attention = True
        self.use_block_products = act_dtype == torch.bfloat16  # products in tiles over the row-major copy (gemm_block)
        self._num_cus = max(1, torch.cuda.get_device_properties(self.device).multi_processor_count)
        self._resident_k = {}
        self.fuse_norms = act_dtype == torch.bfloat16
        self.fuse_rope = act_dtype == torch.bfloat16
        self.tile_few_rows = act_dtype == torch.bfloat16      # gated_mlp keeps few rows tiled by k-step
        self.weight_layout = "dual" if act_dtype == torch.bfloat16 else "rows"
        self.lower_tiles = act_dtype == torch.bfloat16        # see plan_weights
        self._untiled = None          # scratch for "tiled": the row-major form of one matrix
        # Up to this many rows no product of a prepared weight goes to the library
        # (whose kernels may record memsets, which HIP graphs replay wrongly here):
        # decode steps of at most this many requests can be captured.
        self.graph_rows_limit = self.MID_MAX_M if act_dtype == torch.bfloat16 else self.SKINNY_MAX_M

    # ------------------------------------------------------------ plumbing
    def _call(self, stem, name, *args):
        fn = self._fn.get(name)
        if fn is None:
            fn = getattr(self._lib[stem], name)
            fn.restype = ctypes.c_char_p
            self._fn[name] = fn
        stream = self._raw_stream(self._device_index) if self._raw_stream is not None else \
            torch.cuda.current_stream(self.device).cuda_stream
        err = fn(*args, _c_void_p(stream))
        if err is not None:
            raise KernelError(f"{name}: {err.decode()}")

    def _check(self, t, dtype, shape=None, name="tensor"):
        if t.is_cuda and t.dtype is dtype and t.is_contiguous() and (shape is None or t.shape == shape):
            return                                        # (a torch.Size equals a tuple of the same numbers)
        if t.device.type != "cuda":
            raise KernelError(f"{name} is on {t.device}, not on the GPU")
        if t.dtype != dtype:
            raise KernelError(f"{name} has dtype {t.dtype}, expected {dtype}")
        if not t.is_contiguous():
            raise KernelError(f"{name} is not contiguous")
        if shape is not None and tuple(t.shape) != tuple(shape):
            raise KernelError(f"{name} has shape {list(t.shape)}, expected {list(shape)}")

    def _new(self, shape, dtype=None):
        return torch.empty(shape, dtype=dtype or self.act_dtype, device=self.device)

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

    # ------------------------------------------------------------ embedding
    def embed(self, ids, table):
        T = ids.shape[0]
        V, H = table.shape
        self._check(ids, torch.int32, (T,), "ids")
        self._check(table, self.act_dtype, None, "embedding table")
        out = self._new((T, H), torch.float32)
        self._call("elementwise", "sl_embed", _p(ids), _p(table), _p(out), T, H, V)
        return out

    # ---------------------------------------------------------------- norms
    def add_rmsnorm(self, resid, delta, weight, eps, fuse=False):
        """resid += delta (in place, float32); returns the normed rows.  A
        ``Deferred`` delta is run here; with ``fuse`` (the reader takes
        ``ScaledRows``) the product, the add and the norm are one kernel."""
        T, H = resid.shape
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        if isinstance(delta, Deferred):
            if fuse:
                return self._produce_scaled_rows(resid, delta, weight, eps)
            delta = self.materialize(delta)
        out = self._new((T, H))
        self._call("norm", "sl_add_rmsnorm", _p(resid), *self._delta_args(delta, T, H), None,
                   _p(weight), _p(out), T, H, _c_float(eps))
        return out

    def _delta_args(self, delta, T, H):
        """(delta, parts, nparts, T, bias) of the norm kernels for any kind of delta."""
        if isinstance(delta, PartialSums):
            ks = delta.parts.shape[0]
            self._check(delta.parts, torch.float32, (ks, T, H), "partial sums")
            if delta.bias is not None:
                self._check(delta.bias, torch.float32, (H,), "bias")
            return None, _p(delta.parts), ks, T, _p(delta.bias)
        if delta is not None:
            self._check(delta, self.act_dtype, (T, H), "delta")
        return _p(delta), None, 0, T, None

    def rows_add_rmsnorm(self, resid, delta, rows, weight, eps, fuse=False):
        """The normed rows ``rows`` of resid + delta.  The stream is left as it
        is, except that a fused ``Deferred`` delta is added into it."""
        T, H = resid.shape
        R = rows.shape[0]
        self._check(resid, torch.float32, None, "residual stream")
        self._check(weight, torch.float32, (H,), "norm weight")
        self._check(rows, torch.int32, (R,), "rows")
        if isinstance(delta, Deferred):
            if fuse and R <= 16:
                scaled = self._produce_scaled_rows(resid, delta, weight, eps)
                scaled.rows = rows
                return scaled
            delta = self.materialize(delta)
        out = self._new((R, H))
        self._call("norm", "sl_add_rmsnorm", _p(resid), *self._delta_args(delta, T, H), _p(rows),
                   _p(weight), _p(out), R, H, _c_float(eps))
        return out

    def materialize(self, value):
        """The plain tensor of a ``Deferred`` product (anything else is returned as it is)."""
        if isinstance(value, Deferred):
            return self.linear(value.x, value.weight, value.bias)
        if isinstance(value, PartialSums):
            ks, M, N = value.parts.shape
            y = self._new((M, N))
            self._call("gemm", "sl_splitk_reduce", _p(value.parts), _p(value.bias), _p(y), M, N, ks, 0)
            return y
        return value

    def _produce_scaled_rows(self, resid, d, gain, eps):
        x, weight = d.x, d.weight
        M, K = x.shape
        N = weight.shape[0]
        if tuple(resid.shape) != (M, N):
            raise KernelError(f"a delta of shape {[M, N]} does not fit the stream {list(resid.shape)}")
        self._check(x.data if isinstance(x, TiledRows) else x, self.act_dtype, None, "x")
        if d.bias is not None:
            self._check(d.bias, torch.float32, (N,), "bias")
        out = self._new((M, N))
        th = self._producer_copy(weight, M)[1]
        parts = self._new((-(-N // th), 16), torch.float32)
        tiled = M if self.tile_few_rows and M > 1 and N % 32 == 0 else 0     # for the products that read the rows
        self._skinny(x, weight, d.bias, out, M, N, K, resid=resid, next_gain=gain, out_parts=parts,
                     y_tiled=bool(tiled))
        return ScaledRows(out, parts, eps, tiled=tiled)

    # --------------------------------------------------------------- linear
    def plan_weights(self, total_bytes: int) -> str:
        """Choose the layout for a model whose matrices take ``total_bytes``
        (called before the matrices are loaded)."""
        if self.act_dtype == torch.bfloat16:
            total = torch.cuda.get_device_properties(self.device).total_memory
            self.weight_layout = "dual" if 2 * total_bytes <= self.DUAL_MEMORY_SHARE * total else "tiled"
            # a third copy of the matrices that add to the stream (about a third of all), in lower tiles
            self.lower_tiles = self.weight_layout == "dual" and 2.35 * total_bytes <= self.LOWER_TILES_MEMORY_SHARE * total
        return self.weight_layout

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
        if self.weight_layout == "tiled" and not keep_rows:
            weight = LinearWeight(None, tiled, (N, K))
        else:
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

    FUSED_NORM_MAX_M = 16         # the fused add + norm lives in the kernel for up to 16 rows

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
        if (defer and self.fuse_norms and not out_f32 and 0 < M <= self.FUSED_NORM_MAX_M
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
        shares = self._block_shares(M, N, K, weight)
        if shares:
            # (deferred: the norm adds the partial sums)
            return self.linear_block(x, weight, bias, out_f32, shares,
                                     partial=defer and self.fuse_norms and not out_f32)
        if (defer and self.fuse_norms and not out_f32 and self.WIDE_MIN_M <= M <= limit
                and K % 32 == 0 and N % 4 == 0 and self._takes_mid(M, N, K)):
            return self.linear_mid(x, weight, bias, partial=True,     # the norm adds the partial sums
                                   target=self.MID_DEFERRED_WORKGROUPS)
        if M <= limit:
            return self.linear_skinny(x, weight, bias, out_f32)
        if out_f32 and limit:
            # float32 results of many rows (logits of every position): W is
            # streamed once per `limit` rows by the few-rows kernels, several
            # times faster than the plain tiled kernel below
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

    def _block_shares(self, M, N, K, weight) -> int:
        """Over how many workgroups the block kernel splits K for a product of
        M rows, or 0 when the product is not one of its own: bfloat16, a
        row-major copy of the weight, K in chunks of 64, a matrix of few rows
        (its tiles alone would leave most CUs idle, which is what the split
        repairs) but of MID_MIN_ELEMENTS_MANY elements at least (smaller ones
        stay with the kernels they were measured on), and BLOCK_MIN_M to
        BLOCK_MAX_M rows of x.  As many shares as give every CU a workgroup,
        16 at most, of at least 3 chunks each (7B shape, down projection at 256
        rows: 70 / 44 / 41 us with 4 / 8 / 9 shares; q/k/v: 21 / 17 / 26 us
        with 4 / 7 / 8, the last being more workgroups than CUs)."""
        w = weight.w if isinstance(weight, LinearWeight) else weight
        if (self.act_dtype != torch.bfloat16 or not self.use_block_products or w is None
                or K % 64 or N % 4 or N > self.BLOCK_MAX_N or N * K < self.MID_MIN_ELEMENTS_MANY
                or not self.BLOCK_MIN_M <= M <= self.BLOCK_MAX_M):
            return 0
        tiles = -(-N // 128) * -(-M // 256)
        return max(1, min(16, K // 64 // 3, self._num_cus // tiles))

    def linear_block(self, x, weight, bias, out_f32=False, ks=1, partial=False):
        """A few hundred rows over the row-major copy of the weight: workgroups
        own a tile of 256 rows of x by 128 rows of W over one of ``ks`` shares
        of K.  ``partial``: the product comes back as ``PartialSums`` for its
        reader to add up."""
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
                self._call("gemm", "sl_gemm_block", _p(x), _p(w), None, None, M, N, K, 0, int(ks), _p(part))
            else:
                self._call("gemm", "sl_gemm_block", _p(x), _p(w), None, _p(part), M, N, K, 1, 1, None)
            return PartialSums(part, bias)
        y = self._new((M, N), torch.float32 if out_f32 else None)
        self._call("gemm", "sl_gemm_block", _p(x), _p(w), _p(bias), _p(y), M, N, K, int(out_f32),
                   int(ks), _p(part))
        return y

    def linear_skinny(self, x, weight, bias, out_f32=False):
        M, K = x.shape
        N = weight.shape[0]
        if weight.tiled is None:
            raise KernelError("linear_skinny needs the tiled copy of the weight")
        if M >= self.WIDE_MIN_M:
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
        if (_tiled_out and M < self.WIDE_MIN_M and M <= self._few_rows_limit(weight)
                and block == self.GATE_BLOCK and N % 16 == 0):
            self._check(x, self.act_dtype, None, "x")
            y = self._new((M, N // 2))
            self._skinny(x, weight, None, y, M, N, K, gated=True, y_tiled=True)
            return TiledRows(y, (M, N // 2))
        if M <= self._few_rows_limit(weight) and block == self.GATE_BLOCK and N % 16 == 0:
            self._check(x, self.act_dtype, None, "x")
            if M >= self.WIDE_MIN_M:
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
        tiled = (self.act_dtype == torch.bfloat16 and self.tile_few_rows and 1 < M <= self.FUSED_NORM_MAX_M
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

    def silu_mul(self, gate_up, block=None):
        T, two_i = gate_up.shape
        if two_i % 2:
            raise KernelError("silu_mul: the row must hold gate and up of equal width")
        inter = two_i // 2
        block = inter if block is None else int(block)
        if block < 1 or inter % block:
            raise KernelError(f"silu_mul: block {block} does not divide the width {inter}")
        self._check(gate_up, self.act_dtype, None, "gate_up")
        out = self._new((T, inter))
        self._call("elementwise", "sl_silu_mul", _p(gate_up), _p(out), T, inter, block)
        return out

    # ----------------------------------------------------------------- rope
    def rope_tables(self, positions, inv_freq):
        T, half = positions.shape[0], inv_freq.shape[0]
        self._check(positions, torch.int32, (T,), "positions")
        self._check(inv_freq, torch.float32, (half,), "inv_freq")
        cos = self._new((T, half), torch.float32)
        sin = self._new((T, half), torch.float32)
        self._call("elementwise", "sl_rope_tables", _p(positions), _p(inv_freq), _p(cos), _p(sin),
                   T, half)
        return cos, sin

    def _check_pages(self, k_cache, v_cache, nkv, D, page_size):
        pages = k_cache.shape[0]
        self._check(k_cache, self.act_dtype, (pages, nkv, page_size, D), "K pages")
        self._check(v_cache, self.act_dtype, (pages, nkv, D, page_size), "V pages")
        return pages

    def rope_store(self, qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                   pairs8=False, split=None, rot_dim=None, q_scale=1.0):
        """Rotate q and k of ``qkv`` in place (``cos`` None: no rotation) and write
        k and v to their cache rows (``k_cache`` None: no write).  The first
        ``rot_dim`` channels of a head are rotated (default: all), pair j being
        (j, j + rot_dim / 2); ``pairs8``: they come in blocks of 8 channels and
        their 8 partners (the order ``qkv_rope_store`` uses) instead.
        ``split``: the product arrives as ``PartialSums``; ``qkv`` is then only
        written (its q columns).  ``q_scale`` multiplies the q heads after the
        rotation, before their rounding."""
        T = qkv.shape[0]
        rot = D if rot_dim is None else int(rot_dim)
        if rot % 2 or not 0 <= rot <= D or (pairs8 and rot % 16) or (cos is not None and rot == 0):
            raise KernelError(f"rope_store: cannot rotate {rot} of {D} channels"
                              + (" in blocks of 8 pairs" if pairs8 else ""))
        self._check(qkv, self.act_dtype, (T, (nh + 2 * nkv) * D), "qkv")
        parts = bias = None
        if split is not None:
            parts, bias = split.parts, split.bias
            self._check(parts, torch.float32, (parts.shape[0], T, (nh + 2 * nkv) * D), "partial sums")
            if bias is not None:
                self._check(bias, torch.float32, ((nh + 2 * nkv) * D,), "bias")
        if cos is not None:
            self._check(cos, torch.float32, (T, rot // 2), "cos")
            self._check(sin, torch.float32, (T, rot // 2), "sin")
        if k_cache is not None:
            self._check_pages(k_cache, v_cache, nkv, D, page_size)
            self._check(slots, torch.int32, (T,), "slots")
        self._call("elementwise", "sl_rope_store", _p(qkv), _p(cos), _p(sin), _p(slots),
                   _p(k_cache), _p(v_cache), T, nh, nkv, D, rot, page_size, int(pairs8),
                   _p(parts), parts.shape[0] if parts is not None else 0, _p(bias), _c_float(q_scale))

    def qkv_rope_store(self, x, weight, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache,
                       page_size, rot_dim=None, q_scale=1.0):
        """q/k/v product, rotation and cache write.  The rows of ``weight`` (and
        ``bias``) hold every q and k head in the blocked pair order (``pairs8``
        above).  Returns the [T, (nh + 2 nkv) D] buffer whose q columns the
        attention reads.  For at most 16 rows and a tiled weight all of it is
        one kernel; k and v columns of the buffer are then not written."""
        if not isinstance(weight, LinearWeight):
            weight = LinearWeight(weight)
        M, K = x.shape
        N = weight.shape[0]
        rot = D if rot_dim is None else int(rot_dim)
        if N != (nh + 2 * nkv) * D or D % 16 or rot % 16 or not 0 <= rot <= D:
            raise KernelError("qkv_rope_store: weight rows must be (nh + 2 nkv) * D with D % 16 == 0, "
                              "the rotated width a multiple of 16")
        fused = (self.act_dtype == torch.bfloat16 and self.fuse_rope and 0 < M <= 16
                 and weight.tiled is not None and weight.shape == (N, K))
        if not fused:
            shares = 0 if isinstance(x, ScaledRows) else self._block_shares(M, N, K, weight)
            if shares:
                # K split over workgroups of the block kernel; the rotation kernel adds the partial sums up
                self._check(x, self.act_dtype, (M, K), "x")
                product = self.linear_block(x, weight, bias, ks=shares, partial=True)
                qkv = self._new((M, N))
                self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                True, split=product, rot_dim=rot, q_scale=q_scale)
                return qkv
            if (self.WIDE_MIN_M <= M <= self._few_rows_limit(weight) and K % 32 == 0
                    and not isinstance(x, ScaledRows)):
                # K split over workgroups; the rotation kernel adds the partial sums up
                product = self.linear_mid(x, weight, bias, partial=True)
                if isinstance(product, PartialSums):
                    qkv = self._new((M, N))
                    self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                    True, split=product, rot_dim=rot, q_scale=q_scale)
                    return qkv
                qkv = product
            elif (self.act_dtype == torch.bfloat16 and not isinstance(x, ScaledRows)
                    and M > self._few_rows_limit(weight)):
                # many rows: the library keeps the float32 sums, and the rotation kernel adds the
                # float32 bias, rotates and rounds once, exactly as the fused few-rows kernel does
                self._check(x, self.act_dtype, (M, K), "x")
                sums = self.library_sums(x, self.rows_of(weight), torch.float32)
                qkv = self._new((M, N))
                self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                                True, split=PartialSums(sums.unsqueeze(0), bias), rot_dim=rot,
                                q_scale=q_scale)
                return qkv
            else:
                qkv = self.linear(x, weight, bias)
            self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size, True,
                            rot_dim=rot, q_scale=q_scale)
            return qkv
        scaled = x if isinstance(x, ScaledRows) else None
        if scaled is None:
            self._check(x, self.act_dtype, None, "x")
        if bias is not None:
            self._check(bias, torch.float32, (N,), "bias")
        if cos is not None:
            self._check(cos, torch.float32, (M, rot // 2), "cos")
            self._check(sin, torch.float32, (M, rot // 2), "sin")
        if k_cache is not None:
            self._check_pages(k_cache, v_cache, nkv, D, page_size)
            self._check(slots, torch.int32, (M,), "slots")
        rope = _RopeStore(_ptr(cos), _ptr(sin), _ptr(slots if k_cache is not None else None),
                          _ptr(k_cache), _ptr(v_cache), nh, nkv, D, page_size, rot, q_scale)
        qkv = self._new((M, N))
        self._skinny(scaled.x if scaled is not None else x, weight, bias, qkv, M, N, K,
                     scaled=scaled, rope=rope)
        return qkv

    # --------------------------------------------- position encodings of a mixer
    def plan_rotation(self, head_dim, layout) -> RotationPlan:
        """The channel order of q and k heads for a position encoding whose
        ``layout`` is None (nothing is rotated) or says ``rot_dim`` (the leading
        channels that are rotated) and ``pairing``: "half" pairs channel j with
        j + rot_dim / 2, "interleaved" 2j with 2j + 1.  Scores do not depend on
        the order of the channels as long as q and the cached k agree, so an
        interleaved pairing is turned into halves by the order alone, and the
        rotated channels are laid out in blocks of 8 and their 8 partners where
        the fused q/k/v kernel can take them (head size and rotated width
        multiples of 16)."""
        D = int(head_dim)
        rot = 0 if layout is None else int(layout.rot_dim)
        pairing = "half" if layout is None else layout.pairing
        if rot % 2 or not 0 <= rot <= D:
            raise KernelError(f"a rotation of {rot} of {D} channels has no kernel: the width must be even")
        if pairing not in ("half", "interleaved"):
            raise KernelError(f"pairing '{pairing}' has no kernel (half or interleaved)")
        order = list(range(D))
        if pairing == "interleaved":
            order[:rot] = list(range(0, rot, 2)) + list(range(1, rot, 2))
        blocked = D % 16 == 0 and rot % 16 == 0
        if blocked and rot:
            halves = order[:rot]
            order[:rot] = [halves[(i % 16 >= 8) * (rot // 2) + 8 * (i // 16) + i % 8] for i in range(rot)]
        plain = order == list(range(D))
        return RotationPlan(None if plain else torch.tensor(order, dtype=torch.long), rot, blocked)

    LOG2E = 1.4426950408889634

    def split_attention_scale(self, scale: float):
        """(factor for q at its producer, scale left for ``paged_attention``).
        The matrix-core attention kernels want their scores in units of log 2:
        q then leaves ``project_qkv`` multiplied by scale * log2(e) (before its
        one rounding) and the attention call gets ln 2, whose product with
        log2(e) is 1, so no multiply-add per score is left.  The float32 table
        keeps the scale where the reference has it."""
        if self.act_dtype != torch.bfloat16 or not self.use_mfma_attention:
            return 1.0, float(scale)
        return float(scale) * self.LOG2E, 1.0 / self.LOG2E

    def project_qkv(self, x, weight, bias, nh, nkv, D, plan, tables, slots, k_cache, v_cache,
                    page_size, q_scale=1.0):
        """What a mixer calls: the q/k/v product of ``x`` (rows of ``weight`` in
        the order of ``plan``), the position encoding's work on q and k for this
        step's ``tables`` (whatever the encoding's ``tables()`` returned: None,
        or an object with ``cos`` and ``sin`` [T, rot_dim / 2]) and the write of
        k and v into the cache.  Returns [T, (nh + 2 nkv) D] whose q columns the
        attention reads, multiplied by ``q_scale`` (see ``split_attention_scale``)."""
        cos = sin = None
        if tables is not None:
            cos, sin = getattr(tables, "cos", None), getattr(tables, "sin", None)
            if cos is None or sin is None:
                raise KernelError(f"position tables of type {type(tables).__name__} have no kernel: "
                                  "this table rotates channel pairs by cos and sin and nothing else")
            if plan.rot_dim == 0:
                raise KernelError("the position encoding gives tables but its layout rotates nothing")
        if plan.blocked:
            return self.qkv_rope_store(x, weight, bias, nh, nkv, D, cos, sin, slots, k_cache, v_cache,
                                       page_size, rot_dim=plan.rot_dim, q_scale=q_scale)
        qkv = self.linear(x, weight, bias)
        self.rope_store(qkv, nh, nkv, D, cos, sin, slots, k_cache, v_cache, page_size,
                        rot_dim=plan.rot_dim, q_scale=q_scale)
        return qkv

    # ------------------------------------------------------------ attention
    def attend_and_project(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                           batch, scale, window, w_out, bias=None, defer=False):
        """``paged_attention`` followed by ``linear`` with the output projection.  For a step of a few
        single tokens the kernel table keeps what lies between them laid out by k-step, as
        ``gated_mlp`` does (at 16 rows the projection reads as many bytes of x as of W)."""
        if not isinstance(w_out, LinearWeight):
            w_out = LinearWeight(w_out)
        T = qkv.shape[0]
        tiled = (self.tile_few_rows and 1 < T <= self.FUSED_NORM_MAX_M and batch.max_q_len == 1
                 and batch.num_prefill_seqs == 0 and batch.num_seqs == T and w_out.tiled is not None
                 and w_out.shape[1] == nh * D
                 and self._mfma_attention_fits(D, nh // nkv, block_tables.shape[1], page_size, batch))
        attn = self.paged_attention(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                    batch, scale, window, _tiled_out=tiled)
        return self.linear(attn, w_out, bias, defer=defer)

    def paged_attention(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                        batch, scale, window, _tiled_out=False):
        T = qkv.shape[0]
        S, max_pages = block_tables.shape
        self._check(qkv, self.act_dtype, (T, (nh + 2 * nkv) * D), "qkv")
        self._check_pages(k_cache, v_cache, nkv, D, page_size)
        self._check(block_tables, torch.int32, None, "block tables")
        self._check(batch.tok_seq, torch.int32, (T,), "tok_seq")
        self._check(batch.positions, torch.int32, (T,), "positions")
        if S != batch.num_seqs:
            raise KernelError(f"block tables hold {S} sequences, the batch {batch.num_seqs}")
        if batch.max_ctx_len > max_pages * page_size:
            raise KernelError("block table is shorter than the context")
        out = self._new((T, nh * D))
        if self._mfma_attention_fits(D, nh // nkv, max_pages, page_size, batch):
            self._attention_mfma(qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables,
                                 batch, scale, window, out, out_rows=T if _tiled_out else 0)
            return TiledRows(out, (T, nh * D)) if _tiled_out else out
        stride = (nh + 2 * nkv) * D
        first = 0                         # tokens before this one are done
        n_pre, n_pre_tok = batch.num_prefill_seqs, batch.num_prefill_tokens
        if n_pre and D % 16 == 0 and batch.max_q_len > 1:
            # prompt portions (they come first in the batch): workgroups that stage each block of keys
            # once for 16 columns, instead of a wavefront per (token, head) that reads its own
            self._check(batch.cu_q, torch.int32, (batch.num_seqs + 1,), "cu_q")
            self._call("attention", "sl_attention_general_tiles", _p(qkv), stride, _p(k_cache),
                       _p(v_cache), _p(block_tables), max_pages, _p(batch.cu_q), _p(batch.positions),
                       n_pre, batch.max_q_len, nh, nkv, D, page_size, _c_float(scale),
                       int(window or 0), _p(out))
            first = n_pre_tok
        rest = T - first
        if rest == 0:
            return out
        # few tokens (a decode step): the keys of every (token, head) are shared out over several
        # wavefronts; the count depends on the number of tokens only, so that a captured step and an
        # eager one add up in the same order
        single = first > 0 or batch.max_q_len == 1
        group = nh // nkv                 # a wavefront takes up to 8 heads of a group together
        per_token = nkv * -(-group // 8) if group > 1 else nh
        nsplit = max(1, min(64, self.GENERAL_ATTENTION_WAVES // (rest * per_token))) if single else 1
        part_o = part_ml = None
        if nsplit > 1:
            part_o = self._new((rest, nh, nsplit, D), torch.float32)
            part_ml = self._new((rest, nh, nsplit, 2), torch.float32)
        self._call("attention", "sl_attention_general", _p(qkv[first:]), stride, _p(k_cache),
                   _p(v_cache), _p(block_tables), max_pages, _p(batch.tok_seq[first:]),
                   _p(batch.positions[first:]), rest, nh, nkv, D, page_size, _c_float(scale),
                   int(window or 0), _p(out[first:]), nsplit, _p(part_o), _p(part_ml))
        return out

    def _mfma_attention_fits(self, D, group, max_pages, page_size, batch):
        """The matrix-core kernels take bfloat16, head sizes that are multiples
        of 32, and block tables that cover the context rounded up to a whole
        32-key block; everything else goes to the general kernel."""
        if self.act_dtype != torch.bfloat16 or not self.use_mfma_attention:
            return False
        if D % 32 or D > 256 or group > 64:
            return False
        return max_pages * page_size >= -(-batch.max_ctx_len // 32) * 32

    def _attention_lib(self, D):
        key = ("attention_mfma", D)
        lib = self._lib.get(key)
        if lib is None:
            lib = build.load(build.unit("attention_mfma", "bfloat16", SL_HEAD_DIM=D))
            self._lib[key] = lib
        return key

    def _decode_shares(self, units, most) -> int:
        """Into how many shares the keys of each of ``units`` (request, kv head) pairs are cut, ``most`` at
        most.  A share is a wavefront, and a wavefront streams its keys at the pace of its round trips to
        memory, so the launch takes what its busiest CU holds: TARGET_WAVES wavefronts (two a CU) are best,
        and a launch slightly above a whole number of wavefronts per CU is the worst (7B shape, contexts of
        4,096: 14 requests in 10 shares, 560 wavefronts: 30.6 us a layer; in 9, 504 wavefronts: about 22 us;
        24 requests 576 against 480 wavefronts: 4.73 against 4.40 ms a step; 48 requests 384 / 576 / 768
        wavefronts: 5.62 / 5.77 / 5.49 ms).  Taken: the count whose wavefronts fill their rounds over the CUs
        best, less a fifth of its relative distance from the target; no more than half again the target."""
        cus, target = self._num_cus, self.TARGET_WAVES
        best, best_score = 1, None
        for shares in range(1, max(1, min(most, (3 * target // 2) // units)) + 1):
            waves = units * shares
            score = waves / (-(-waves // cus) * cus) - 0.2 * abs(waves - target) / target
            if best_score is None or score > best_score + 1e-9:
                best, best_score = shares, score
        return best

    def _pair_prompt_tiles(self, tiles, prompts_and_heads) -> bool:
        """Whether the workgroups of a whole prompt's attention take a late tile of the causal triangle and
        its early mirror (equal work for all, half as many workgroups) or a tile each, long ones first.
        Equal workgroups fill the chip in rounds of two per CU, and the last round may be nearly empty;
        tiles of their own leave the balance to the order in which workgroups start, at the price of
        twice the prologues.  7B shape, one prompt, pairs against a tile each: 4,096 tokens (448 pairs, one
        round) 175 against 223 us, 5,120 (560) 335 against 270, 7,168 (784) 546 against 461, 8,192 (896) 615
        against 572, 10,240 (1,120) 972 against 880, 14,336 (1,568) 1,842 against 1,618, 16,384 (1,792: three
        and a half rounds) 2,040 either way."""
        if not self.PAIR_PROMPT_TILES:
            return False
        pairs = -(-tiles // 2) * prompts_and_heads
        slots = 2 * self._num_cus
        rounds = -(-pairs // slots)
        return rounds == 1 or pairs >= self.UNPAIRED_BELOW_FILL * rounds * slots

    def _attention_mfma(self, qkv, nh, nkv, D, k_cache, v_cache, page_size, block_tables, batch,
                        scale, window, out, out_rows=0):
        lib = self._attention_lib(D)
        self._check(batch.cu_q, torch.int32, (batch.num_seqs + 1,), "cu_q")
        max_pages = block_tables.shape[1]
        n_pre, n_pre_tok = batch.num_prefill_seqs, batch.num_prefill_tokens
        n_dec = batch.num_seqs - n_pre
        if n_dec and n_pre_tok + n_dec != batch.num_tokens:
            raise KernelError("single-token sequences must come last in the batch")
        common = (_p(qkv), (nh + 2 * nkv) * D, _p(k_cache), _p(v_cache), _p(block_tables),
                  max_pages, _p(batch.cu_q), _p(batch.positions))
        tail = (nh, nkv, D, page_size, _c_float(scale), int(window or 0))
        name = f"sl_attention_mfma@{D}"
        if name not in self._fn:
            fn = self._lib[lib].sl_attention_mfma
            fn.restype = ctypes.c_char_p
            self._fn[name] = fn
        if n_pre:
            waves = -(-batch.max_q_len * (nh // nkv) // 32) * nkv * n_pre
            shared = (waves >= self.SHARED_ATTENTION_MIN_WAVES and
                      batch.max_ctx_len >= self.SHARED_ATTENTION_MIN_CONTEXT and
                      bool(self._lib[lib].sl_attention_mfma_shares_keys()))
            # tiles of a causal triangle differ in length and are paired; those of a portion
            # that starts deeper in its context than it is long do not
            triangle = batch.max_ctx_len < 2 * batch.max_q_len
            pair = triangle and self._pair_prompt_tiles(-(-batch.max_q_len * (nh // nkv) // 128), nkv * n_pre)
            # few unpaired tiles over a long context: each is cut into shares of its keys
            nsplit, part_o, part_ml = 1, None, None
            if shared and not triangle:
                nsplit = max(1, min(self.PROMPT_SPLIT_MAX, batch.max_ctx_len // 32 // self.PROMPT_SPLIT_MIN_BLOCKS,
                                    -(-self.PROMPT_SPLIT_WORKGROUPS // -(-waves // 4)),
                                    self.PROMPT_SPLIT_BYTES // (n_pre_tok * nh * D * 4)))
            if nsplit > 1:
                part_o = self._new((n_pre_tok, nh, nsplit, D), torch.float32)
                part_ml = self._new((n_pre_tok, nh, nsplit, 2), torch.float32)
            self._call(lib, name, *common, 0, n_pre, batch.max_q_len, *tail, nsplit,
                       0 if shared else 1 << 30, int(pair), _p(out), _p(part_o), _p(part_ml), 0,
                       n_pre_tok if nsplit > 1 else 0, self.NARROW_ATTENTION_WORKGROUPS, 0)
        if n_dec:
            blocks = -(-batch.max_ctx_len // 32)
            if window:
                blocks = min(blocks, -(-int(window) // 32) + 1)
            # (a few requests with long contexts: up to 256 shares, so that the launch still has TARGET_WAVES
            # wavefronts; 7B shape, one request at 32,000 tokens: 64 shares leave one wavefront per CU)
            most = int(self._lib[lib].sl_attention_mfma_max_splits())
            nsplit = self._decode_shares(n_dec * nkv, min(most, blocks // 2))
            part_o = part_ml = None
            if nsplit > 1:
                part_o = self._new((n_dec, nh, nsplit, D), torch.float32)
                part_ml = self._new((n_dec, nh, nsplit, 2), torch.float32)
            self._call(lib, name, *common, n_pre, n_dec, 1, *tail, nsplit, 0, 0, _p(out),
                       _p(part_o), _p(part_ml), n_pre_tok, n_dec if nsplit > 1 else 0, 0, int(out_rows))

    # ------------------------------------------------------------- sampling
    SAMPLE_SLICE = 2048           # logits per workgroup of the two-stage argmax and draw (at most 64 slices)
    CUT_SLICE = 4096              # logits per workgroup when cuts are searched (at most CUT_MAX_SLICES slices:
    CUT_MAX_SLICES = 16           # every workgroup adds up the tables of all slices of its row)

    def _sample_workspace(self, R, chunks, cuts):
        fn = self._fn.get("sl_sample_workspace")
        if fn is None:
            fn = self._lib["sampling"].sl_sample_workspace
            fn.restype = ctypes.c_size_t
            fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
            self._fn["sl_sample_workspace"] = fn
        return self._new((fn(R, chunks, int(cuts)) // 8,), torch.int64)

    def argmax(self, logits):
        R, V = logits.shape
        self._check(logits, torch.float32, None, "logits")
        out = self._new((R,), torch.int32)
        chunks = max(1, min(64, V // self.SAMPLE_SLICE))
        work = self._sample_workspace(R, chunks, False)
        self._call("sampling", "sl_argmax", _p(logits), R, V, chunks, _p(work), _p(out))
        return out

    def sample(self, logits, temperature, top_k, top_p, seeds, draws):
        """One token per row; rows with temperature 0 take the argmax.  ``top_k``
        and ``top_p`` both None: no row is cut, which takes the two-stage draw.
        With cuts, rows of CUT_SLICE * 2 logits or more are searched by several
        workgroups a row, shorter ones by one."""
        R, V = logits.shape
        self._check(logits, torch.float32, None, "logits")
        self._check(temperature, torch.float32, (R,), "temperature")
        self._check(seeds, torch.int64, (R,), "seeds")
        self._check(draws, torch.int64, (R,), "draws")
        if (top_k is None) != (top_p is None):
            raise KernelError("sample: top_k and top_p go together")
        out = self._new((R,), torch.int32)
        if top_k is None:
            chunks = max(1, min(64, V // self.SAMPLE_SLICE))
            work = self._sample_workspace(R, chunks, False)
        else:
            self._check(top_k, torch.int32, (R,), "top_k")
            self._check(top_p, torch.float32, (R,), "top_p")
            chunks = max(1, min(self.CUT_MAX_SLICES, V // self.CUT_SLICE))
            work = self._sample_workspace(R, chunks, True) if chunks >= 2 else None
        self._call("sampling", "sl_sample", _p(logits), R, V, _p(temperature), _p(top_k),
                   _p(top_p), _p(seeds), _p(draws), chunks, _p(work), _p(out))
        return out

    def sample_static(self, logits, temperature=None, top_k=None, top_p=None, seeds=None, draws=None):
        """``sample`` (or ``argmax`` when ``temperature`` is None) through the
        library's entry point that allocates nothing: its scratch is a static
        device array of 8 MiB inside the library, shared by all calls on this
        GPU, so calls must not overlap on two streams.  Only the result tensor
        is allocated here; sizes whose scratch would not fit are refused."""
        R, V = logits.shape
        self._check(logits, torch.float32, None, "logits")
        if temperature is not None:
            self._check(temperature, torch.float32, (R,), "temperature")
            self._check(seeds, torch.int64, (R,), "seeds")
            self._check(draws, torch.int64, (R,), "draws")
        if (top_k is None) != (top_p is None) or (top_k is not None and temperature is None):
            raise KernelError("sample_static: top_k and top_p go together and need temperatures")
        if top_k is not None:
            self._check(top_k, torch.int32, (R,), "top_k")
            self._check(top_p, torch.float32, (R,), "top_p")
        out = self._new((R,), torch.int32)
        self._call("sampling", "sl_sample_static", _p(logits), R, V, _p(temperature), _p(top_k),
                   _p(top_p), _p(seeds), _p(draws), _p(out))
        return out

