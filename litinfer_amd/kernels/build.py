"""Building and loading the HIP libraries.

Each file under csrc/ becomes one shared library, compiled by hipcc for gfx950
and loaded through ctypes; its entry points are plain `extern "C"` functions
that take device pointers and a stream.  A library's file name carries a hash
of its source, the shared headers and the flags, so a changed source is never
served by an old build.  Libraries are looked for, and built when absent, in
`litinfer_amd/_lib/` or, where the tree cannot be written, in a per-user
folder under the temporary directory.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path
from typing import Dict, List, Optional

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-result"]          # no fast-math: the 32-bit path needs exact expf/sinf/cosf

# The attention kernels multiply their matrix-core accumulators by the softmax's rescaling factors:
# with the accumulators in ordinary vector registers this needs no copies to and from the
# accumulation registers (and fewer registers in all).
MODULE_FLAGS = {"attention": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
                # the products' loads into LDS are inline assembly that sets M0 and says so in its clobber
                # list, which the compiler remarks upon for every instance
                "gemm": ["-Wno-inline-asm"]}

MODULES = ("elementwise", "gemm", "attention", "sampling", "host")     # what a model needs
# measuring kernels of the benchmark (a streaming read, a copy, a matrix-core loop): built with the
# rest by `build_all(everything=True)`, otherwise when the benchmark first asks for them
EXTRA_MODULES = ("probe",)
# "host" is plain C++ (the cache's bookkeeping and the layout of a step's batch): no device code
HOST_MODULES = ("host",)
HOST_FLAGS = ["-O2", "-std=c++17", "-shared", "-fPIC"]


def _source(module: str) -> Path:
    return CSRC / (f"{module}.cpp" if module in HOST_MODULES else f"{module}.hip")


def _flags(module: str) -> List[str]:
    return HOST_FLAGS if module in HOST_MODULES else FLAGS + MODULE_FLAGS.get(module, [])

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                           "the HIP kernels cannot be built")


def _headers() -> List[Path]:
    return sorted(CSRC.glob("*.h")) + sorted(CSRC.glob("*.hpp"))


def _digest(module: str) -> str:
    h = hashlib.sha256()
    for p in [_source(module), *([] if module in HOST_MODULES else _headers())]:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(_flags(module)).encode())
    return h.hexdigest()[:16]


def _lib_dirs() -> List[Path]:
    dirs = [Path(__file__).resolve().parent.parent / "_lib"]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(Path(tempfile.gettempdir()) / f"litinfer_amd-{uid}" / "_lib")
    return dirs


_dir_lock = threading.Lock()
_chosen_dir: Optional[Path] = None


def _writable_dir() -> Path:
    global _chosen_dir
    with _dir_lock:
        if _chosen_dir is not None:
            return _chosen_dir
        for d in _lib_dirs():
            try:
                d.mkdir(parents=True, exist_ok=True)
                probe = d / f".probe-{os.getpid()}-{threading.get_ident()}"
                probe.write_bytes(b"")
                probe.unlink()
                _chosen_dir = d
                return d
            except OSError:
                continue
    raise KernelBuildError("no writable folder for the built libraries: tried "
                           + ", ".join(str(d) for d in _lib_dirs()))


def lib_name(module: str) -> str:
    return f"li_{module}-{_digest(module)}.so"


def find_built(module: str) -> Optional[Path]:
    name = lib_name(module)
    for d in _lib_dirs():
        if (d / name).exists():
            return d / name
    return None


def compile_module(module: str, verbose: bool = True) -> Path:
    """Compile the module's source under csrc/ now, whether or not a build exists."""
    src = _source(module)
    if not src.exists():
        raise KernelBuildError(f"no source {src}")
    out_dir = _writable_dir()
    out = out_dir / lib_name(module)
    tmp = out_dir / f".{out.name}.{os.getpid()}.tmp"
    cmd = [_hipcc(), *_flags(module), f"-I{CSRC}", str(src), "-o", str(tmp)]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())     # hipcc wants a HOME it can look into
    t0 = time.time()
    if verbose:
        print(f"[litinfer_amd] compiling {src.name} for {ARCH} ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    while True:
        try:
            log, _ = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[litinfer_amd]   ... still compiling {src.name} "
                      f"({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed on {src.name}:\n{log}")
    os.replace(tmp, out)
    for old in out_dir.glob(f"li_{module}-*.so"):
        if old != out:
            old.unlink(missing_ok=True)
    if verbose:
        print(f"[litinfer_amd] built {out.name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def build_all(verbose: bool = True, force: bool = True, everything: bool = False) -> List[Path]:
    """Compile every module that a model needs (in parallel); with `everything`, the
    benchmark's measuring kernels too."""
    modules = MODULES + (EXTRA_MODULES if everything else ())
    outs: Dict[str, Path] = {}
    errs: List[BaseException] = []

    def work(m):
        try:
            outs[m] = compile_module(m, verbose) if force or find_built(m) is None else find_built(m)
        except BaseException as e:           # noqa: BLE001 - reported below
            errs.append(e)

    threads = [threading.Thread(target=work, args=(m,)) for m in modules]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errs:
        raise errs[0]
    return [outs[m] for m in modules]


def load(module: str) -> ctypes.CDLL:
    """The library of a module: the built one, or build it first if there is none."""
    with _lock:
        if module in _loaded:
            return _loaded[module]
        path = find_built(module) or compile_module(module)
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from e
        _loaded[module] = lib
        return lib
