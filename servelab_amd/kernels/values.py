"""What travels between the calls of the kernel table: weights in the layouts the kernels read,
products that are handed on unfinished (deferred to the norm that adds them, partial sums of a
split K, rows that are not yet normalised, rows laid out by k-step), the plan of a rotation, and
the error every refused size raises."""
import ctypes
from typing import Optional

import torch

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
