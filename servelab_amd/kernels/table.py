"""The base of the kernel table: the loaded libraries of one activation dtype on one device, the
call into a library on the caller's current stream, and the host-side checks every call makes
before it launches (a kernel that reads out of bounds can take the GPU down)."""
import ctypes
from typing import Optional

import torch

from . import build
from .tuning import Tuning
from .values import KernelError, _c_void_p


class KernelTable:
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
    # The numbers that choose between kernels (DUAL_MEMORY_SHARE, WIDE_MIN_M, MID_*, FEW_*, MANY_*,
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
        self._rows_budget = 0         # bytes of row-major copies a "tiled" model may still keep (plan_weights)
        self._matrices = self._matrices_with_rows = 0
        # Up to this many rows no product of a prepared weight goes to the library
        # (whose kernels may record memsets, which HIP graphs replay wrongly here):
        # decode steps of at most this many requests can be captured.
        self.graph_rows_limit = self.MID_MAX_M if act_dtype == torch.bfloat16 else self.SKINNY_MAX_M

    # ------------------------------------------------------------ plumbing
    def _fused_rows(self, width) -> int:
        """Up to how many rows a step over a residual stream of ``width`` values takes the fused
        few-rows kernels (``Tuning.fused_rows_by_width``)."""
        for upto, rows in self.FUSED_ROWS_BY_WIDTH:
            if width <= upto:
                return min(int(rows), self.FUSED_NORM_MAX_M)
        return 0

    def _wide_from(self, width) -> int:
        """From how many rows on the products of a step over a stream of ``width`` values take
        the kernels in which tiles of W share their reads of x."""
        return min(self.WIDE_MIN_M, self._fused_rows(width) + 1)

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
