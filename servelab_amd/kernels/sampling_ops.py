"""Argmax and seeded draws from float32 logits."""
import ctypes

import torch

from .values import KernelError, _p


class SamplingOps:
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
