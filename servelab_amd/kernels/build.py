"""Compiles the HIP sources under ``csrc/`` into shared libraries for gfx950.

Each source is a unit of its own: ``hipcc -shared -fPIC`` turns it into one
``.so`` with a C ABI, loaded through ctypes.  A unit is compiled per activation
dtype (and per the sizes a source takes as macros, such as the head size of the
matrix-core attention kernels), so the first call for a model compiles what
that model needs and nothing else.  Libraries are kept beside the sources in
``csrc/_build/`` under a name that carries a hash of the source, the headers and
the flags, so a stale library is never loaded.
"""
import ctypes
import hashlib
import os
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from typing import Dict, Iterable, List, Optional, Tuple

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
BASE_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-std=c++17", "-shared", "-fPIC",
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

Unit = Tuple[str, Tuple[str, ...]]          # (source stem, defines)

_loaded: Dict[Unit, ctypes.CDLL] = {}


class BuildError(RuntimeError):
    pass


def unit(stem: str, dtype: str, **defines) -> Unit:
    """A unit: source ``stem``.hip for activation dtype 'bfloat16' | 'float32'."""
    if dtype not in ("bfloat16", "float32"):
        raise ValueError(f"kernels exist for bfloat16 and float32, not {dtype}")
    d = ["SL_F32=1"] if dtype == "float32" else []
    d += [f"{k}={v}" for k, v in sorted(defines.items())]
    return (stem, tuple(d))


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def build_dir() -> str:
    """``csrc/_build`` when it can be written, else a per-user temporary folder."""
    d = os.environ.get("SERVELAB_AMD_BUILD_DIR") or os.path.join(CSRC, "_build")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        open(probe, "w").close()
        os.remove(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"servelab_amd_build_{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _digest(u: Unit) -> str:
    h = hashlib.sha256()
    headers = sorted(n for n in os.listdir(CSRC) if n.endswith(".h"))
    for name in [u[0] + ".hip"] + headers:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(f.read())
    h.update(" ".join(BASE_FLAGS + list(u[1])).encode())
    return h.hexdigest()[:12]


def library_path(u: Unit, folder: Optional[str] = None) -> str:
    tag = "_".join(d.replace("=", "").replace("SL_", "").lower() for d in u[1]) or "bf16"
    return os.path.join(folder or build_dir(), f"{u[0]}_{tag}_{_digest(u)}.so")


def find_built(u: Unit) -> Optional[str]:
    """An up-to-date library of the unit, in the tree or the fallback folder."""
    for folder in (os.path.join(CSRC, "_build"),
                   os.path.join(tempfile.gettempdir(), f"servelab_amd_build_{os.getuid()}")):
        p = library_path(u, folder)
        if os.path.exists(p):
            return p
    return None


def compile_unit(u: Unit, out: str) -> str:
    tmp = f"{out}.{os.getpid()}.tmp"
    cmd = [hipcc()] + BASE_FLAGS + ["-D" + d for d in u[1]] + \
        ["-o", tmp, os.path.join(CSRC, u[0] + ".hip")]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())      # hipcc wants a home for its cache
    try:
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                             env=env)
    except FileNotFoundError:
        raise BuildError(f"hipcc not found ({cmd[0]}): the HIP kernels cannot be built")
    if res.returncode != 0:
        raise BuildError(f"hipcc failed for {u}:\n{res.stdout}")
    os.replace(tmp, out)
    return out


def ensure(units: Iterable[Unit], force: bool = False, verbose: bool = True) -> Dict[Unit, str]:
    """Paths of the libraries of ``units``, compiling the missing ones in
    parallel and printing a line as each one is done."""
    units = list(dict.fromkeys(units))
    paths: Dict[Unit, str] = {}
    todo: List[Unit] = []
    for u in units:
        p = None if force else find_built(u)
        if p:
            paths[u] = p
        else:
            todo.append(u)
    if not todo:
        return paths
    folder = build_dir()
    t0 = time.time()
    if verbose:
        print(f"[servelab_amd] compiling {len(todo)} HIP units for {ARCH} into {folder}",
              file=sys.stderr, flush=True)
    workers = max(1, min(len(todo), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as pool:
        futures = {pool.submit(compile_unit, u, library_path(u, folder)): u for u in todo}
        pending = set(futures)
        while pending:
            done = {f for f in pending if f.done()}
            for f in done:
                u = futures[f]
                paths[u] = f.result()
                if verbose:
                    print(f"[servelab_amd]   built {os.path.basename(paths[u])} "
                          f"({time.time() - t0:.0f}s)", file=sys.stderr, flush=True)
            pending -= done
            if pending:
                time.sleep(0.2)
                if verbose and int(time.time() - t0) % 20 == 0 and time.time() - t0 > 19:
                    print(f"[servelab_amd]   still compiling {len(pending)} units "
                          f"({time.time() - t0:.0f}s)", file=sys.stderr, flush=True)
                    time.sleep(1.0)
    return paths


def prune(keep: Iterable[str], folder: Optional[str] = None) -> int:
    """Removes the libraries in the build folder that are not in ``keep``
    (those of older sources, which no digest names any more); returns how many."""
    folder = folder or build_dir()
    keep = {os.path.abspath(p) for p in keep}
    gone = 0
    for name in os.listdir(folder):
        path = os.path.abspath(os.path.join(folder, name))
        if name.endswith(".so") and path not in keep:
            try:
                os.remove(path)
                gone += 1
            except OSError:
                pass
    return gone


def load(u: Unit) -> ctypes.CDLL:
    """The loaded library of a unit (compiled first when none is built)."""
    if u not in _loaded:
        path = ensure([u])[u]
        _loaded[u] = ctypes.CDLL(path)
    return _loaded[u]


# every unit the package can ask for with the default set of head sizes
DEFAULT_STEMS = ("elementwise", "norm", "gemm", "attention", "sampling")


def all_units(head_dims=(32, 64, 96, 128, 192, 256)) -> List[Unit]:
    units = []
    for dtype in ("bfloat16", "float32"):
        for stem in DEFAULT_STEMS:
            units.append(unit(stem, dtype))
    for d in head_dims:
        if d % 32 == 0:
            units.append(unit("attention_mfma", "bfloat16", SL_HEAD_DIM=d))
    return units
