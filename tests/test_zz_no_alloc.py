"""The sampling entry point that allocates nothing (``sl_sample_static``, over a
static device scratch array inside the library), called through ctypes: its
tokens equal those of ``sl_sample`` with a workspace, on two calls in a row of
which the second has the smaller input, for greedy rows, plain draws and rows
with top-k / top-p cuts; greedy rows are the argmax and drawn rows the plain
Gumbel-max draw of tests/emulated_ops.py; sizes beyond the static array are
refused."""
import ctypes

import pytest
import torch

from emulated_ops import perturbed_scores
from servelab_amd.kernels import build

pytestmark = pytest.mark.gpu

_c = ctypes.c_void_p


def _library():
    lib = ctypes.CDLL(build.ensure([build.unit("sampling", "bfloat16")])[build.unit("sampling", "bfloat16")])
    lib.sl_sample.restype = ctypes.c_char_p
    lib.sl_sample_static.restype = ctypes.c_char_p
    lib.sl_sample_workspace.restype = ctypes.c_size_t
    lib.sl_sample_workspace.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
    return lib


def _ptr(t):
    return None if t is None else _c(t.data_ptr())


def _inputs(R, V, mode, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    logits = torch.randn(R, V, generator=gen, device="cuda") * 3.0
    if mode == "greedy":
        return logits, None, None, None, None, None
    temperature = torch.full((R,), 0.8, device="cuda")
    temperature[::3] = 0.0                                    # greedy rows among the draws
    seeds = torch.arange(R, device="cuda", dtype=torch.int64) * 7919 + seed
    draws = torch.arange(R, device="cuda", dtype=torch.int64) % 5
    if mode == "draw":
        return logits, temperature, None, None, seeds, draws
    top_k = torch.full((R,), -1, device="cuda", dtype=torch.int32)
    top_k[1::2] = 40
    top_p = torch.full((R,), 1.0, device="cuda")
    top_p[0::2] = 0.9
    return logits, temperature, top_k, top_p, seeds, draws


def _with_workspace(lib, logits, temperature, top_k, top_p, seeds, draws):
    R, V = logits.shape
    cuts = top_k is not None
    chunks = max(1, min(16, V // 4096)) if cuts else max(1, min(64, V // 2048))
    work = torch.empty(lib.sl_sample_workspace(R, chunks, int(cuts)) // 8 + 1, dtype=torch.int64,
                       device="cuda")
    out = torch.full((R,), -1, dtype=torch.int32, device="cuda")
    err = lib.sl_sample(_ptr(logits), R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
                        _ptr(draws), chunks, _ptr(work), _ptr(out),
                        _c(torch.cuda.current_stream().cuda_stream))
    assert err is None, err
    return out


def _static(lib, logits, temperature, top_k, top_p, seeds, draws):
    """(error, tokens, bytes torch had handed out before and after the call)."""
    R, V = logits.shape
    out = torch.full((R,), -1, dtype=torch.int32, device="cuda")
    held = torch.cuda.memory_allocated()
    err = lib.sl_sample_static(_ptr(logits), R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p),
                               _ptr(seeds), _ptr(draws), _ptr(out),
                               _c(torch.cuda.current_stream().cuda_stream))
    assert torch.cuda.memory_allocated() == held              # (torch's own allocations, at least)
    return err, out


@pytest.mark.parametrize("mode", ["greedy", "draw", "cuts"])
def test_static_scratch_sampling_equals_sampling_with_a_workspace(mode):
    lib = _library()
    # two calls in a row on the same static array, the second smaller in rows and in width: what
    # the first left behind must not reach the second's result
    for R, V, seed in ((24, 152064, 1), (5, 33000, 2), (3, 1000, 3)):
        args = _inputs(R, V, mode, seed)
        want = _with_workspace(lib, *args)
        err, got = _static(lib, *args)
        assert err is None, err
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{mode} R={R} V={V}: {got.tolist()} vs {want.tolist()}"
        assert int(got.min()) >= 0 and int(got.max()) < V
        if mode == "draw":                                    # held to the plain draw, not only to sl_sample
            logits, temperature, _, _, seeds, draws = args
            for r, tok in enumerate(got.tolist()):
                if float(temperature[r]) == 0.0:
                    assert tok == int(logits[r].argmax())
                    continue
                scores = perturbed_scores(logits[r], float(temperature[r]), int(seeds[r]), int(draws[r]))
                assert scores[tok] >= scores.max() - 2e-3, f"R={R} V={V} row {r}"
    if mode == "greedy":
        logits = _inputs(3, 1000, "greedy", 3)[0]
        assert torch.equal(_static(lib, logits, None, None, None, None, None)[1].long(),
                           logits.argmax(-1))


def test_sizes_beyond_the_static_array_are_refused():
    lib = _library()
    args = _inputs(128, 152064, "cuts", 4)                    # 128 rows x 16 slices x 6 KB > 8 MiB
    err, out = _static(lib, *args)
    assert err is not None and b"8 MiB" in err
    torch.cuda.synchronize()
    assert int(out.max()) == -1                               # nothing ran
    err, _ = _static(lib, *_inputs(64, 152064, "cuts", 5))   # 64 rows fit
    assert err is None
    torch.cuda.synchronize()


def test_the_kernel_table_reaches_it():
    from servelab_amd.kernels import HipOps
    ops = HipOps(torch.bfloat16)
    args = _inputs(7, 40000, "cuts", 6)
    assert torch.equal(ops.sample_static(*args), ops.sample(*args))
    logits = args[0]
    assert torch.equal(ops.sample_static(logits), ops.argmax(logits))
