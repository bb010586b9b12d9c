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
from .attention_ops import AttentionOps
from .norm_ops import NormOps
from .product_ops import ProductOps
from .sampling_ops import SamplingOps
from .table import KernelTable
from .values import (Deferred, KernelError, LinearWeight, PartialSums, RotationPlan,  # noqa: F401
                     ScaledRows, TiledRows, _RopeStore, _c_float, _p, _ptr)


class HipOps(NormOps, ProductOps, AttentionOps, SamplingOps, KernelTable):
    """The whole table: the base (libraries, calls, checks) and one group of calls per domain.
    ``norm_ops``: embedding, add + norm, silu-multiply; ``product_ops``: weights and products;
    ``attention_ops``: rotation, cache write, attention; ``sampling_ops``: argmax and draws."""
