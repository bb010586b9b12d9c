"""Embedding gather, residual add + RMSNorm (with the products the norm runs or adds up itself),
and the silu-multiply of a gate/up product."""
import torch

from .values import Deferred, KernelError, PartialSums, ScaledRows, TiledRows, _c_float, _p


class NormOps:
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
            if fuse and R <= self._fused_rows(H):
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
