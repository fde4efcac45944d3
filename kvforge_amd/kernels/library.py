"""Builds and loads the HIP kernel modules (one shared library per source file).

A module is compiled with ``hipcc --offload-arch=gfx950`` the first time something asks for it
and the source has changed since the library on disk was built (a stamp file holds the hash of
the sources and flags).  Libraries live in ``kvforge_amd/csrc/_build``; when that folder cannot
be written (a read-only checkout) they go to a per-user folder under the temporary directory.
There is no fallback path: a module that cannot be built or loaded raises ``KernelBuildError``.
"""

from __future__ import annotations

import concurrent.futures
import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
# packed fp32 instructions are switched off for all device code
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]
# Flags of single modules.  attn_mfma: its scores come out of the matrix cores, and before every
# max of such a value the compiler otherwise puts a copy that quiets signalling NaNs (eight more
# instructions per block of keys in a loop that is bound by its vector instructions: 8% of the
# prefill kernel's time).  Masked scores are -inf and no NaN is formed from them (an empty row's
# reference is replaced by zero before it is subtracted), so the kernel may assume there are none.
MODULE_FLAGS: dict[str, list[str]] = {"attn_mfma": ["-fno-honor-nans"]}
# Libraries a module is linked against (after its sources on the command line).
ROCM_LIB = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "lib")
MODULE_LINK: dict[str, list[str]] = {"gemm_library": [f"-L{ROCM_LIB}", f"-Wl,-rpath,{ROCM_LIB}", "-lhipblaslt"]}
HEADERS = ["common.h", "sampling_static.h"]
MODULES: dict[str, list[str]] = {
    "elementwise": ["elementwise.hip"],
    "gemm_generic": ["gemm_generic.hip"],
    "gemm_bf16": ["gemm_bf16.hip"],
    "attn_generic": ["attn_generic.hip"],
    "attn_mfma": ["attn_mfma.hip"],
    "sampling": ["sampling.hip"],
    "gemm_library": ["gemm_library.hip"],
}


class KernelBuildError(RuntimeError):
    pass


_loaded: dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def available_modules() -> list[str]:
    return [m for m, srcs in MODULES.items()
            if all(os.path.isfile(os.path.join(CSRC, s)) for s in srcs)]


def _build_dir() -> str:
    override = os.environ.get("KVFORGE_BUILD_DIR")
    candidates = [override] if override else []
    candidates.append(os.path.join(CSRC, "_build"))
    candidates.append(os.path.join(tempfile.gettempdir(), f"kvforge_amd_build_{os.getuid()}"))
    for d in candidates:
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".w{os.getpid()}.{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise KernelBuildError(f"no writable folder for kernel libraries among {candidates}")


def _source_hash(name: str) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + MODULE_FLAGS.get(name, [])).encode())
    for f in MODULES[name] + HEADERS:
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def _find_built(name: str, want_hash: str) -> str | None:
    """A library whose stamp matches the sources, in the in-tree folder or the fallback."""
    for d in (os.environ.get("KVFORGE_BUILD_DIR"), os.path.join(CSRC, "_build"),
              os.path.join(tempfile.gettempdir(), f"kvforge_amd_build_{os.getuid()}")):
        if not d:
            continue
        so, stamp = os.path.join(d, f"{name}.so"), os.path.join(d, f"{name}.stamp")
        try:
            with open(stamp) as f:
                if f.read().strip() == want_hash and os.path.isfile(so):
                    return so
        except OSError:
            continue
    return None


def _log(msg: str) -> None:
    sys.stderr.write(f"[kvforge_amd] {msg}\n")   # one write: lines of modules built side by side stay whole
    sys.stderr.flush()


def build_module(name: str, force: bool = False, verbose: bool = True) -> str:
    """Compile one module if needed; returns the path of its shared library."""
    if name not in MODULES:
        raise KernelBuildError(f"unknown kernel module {name!r}; known: {sorted(MODULES)}")
    for s in MODULES[name]:
        if not os.path.isfile(os.path.join(CSRC, s)):
            raise KernelBuildError(f"kernel source {s} of module {name!r} is missing in {CSRC}")
    want = _source_hash(name)
    if not force:
        found = _find_built(name, want)
        if found:
            return found
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.isfile(hipcc):
        raise KernelBuildError(
            f"kernel module {name!r} is not built and hipcc was not found; "
            "run `python -c 'import __graft_entry__ as g; g.build()'` where ROCm is installed")
    out_dir = _build_dir()
    so, stamp = os.path.join(out_dir, f"{name}.so"), os.path.join(out_dir, f"{name}.stamp")
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.{threading.get_ident()}.so")
    cmd = [hipcc, *FLAGS, *MODULE_FLAGS.get(name, []), f"-I{CSRC}", *[os.path.join(CSRC, s) for s in MODULES[name]], *MODULE_LINK.get(name, []), "-o", tmp]
    t0 = time.time()
    if verbose:
        _log(f"compiling kernel module {name} for {ARCH} ...")
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                            env=env, cwd=out_dir)
    done = threading.Event()

    def heartbeat() -> None:
        while not done.wait(15.0):
            _log(f"  still compiling {name} ({time.time() - t0:.0f} s)")

    hb = threading.Thread(target=heartbeat, daemon=True)
    if verbose:
        hb.start()
    output, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        lines = [ln for ln in output.splitlines() if "packed-fp32-ops" not in ln]
        raise KernelBuildError(f"hipcc failed for module {name!r}:\n" + "\n".join(lines[-60:]))
    os.replace(tmp, so)
    with open(stamp + ".tmp", "w") as f:
        f.write(want)
    os.replace(stamp + ".tmp", stamp)
    if verbose:
        _log(f"compiled {name} in {time.time() - t0:.1f} s -> {so}")
    return so


def build_modules(names: list[str] | None = None, force: bool = False,
                  verbose: bool = True) -> dict[str, str]:
    """Compile several modules side by side."""
    names = list(names) if names is not None else available_modules()
    workers = max(1, min(len(names), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 1, 8))
    with concurrent.futures.ThreadPoolExecutor(workers) as ex:
        futs = {n: ex.submit(build_module, n, force, verbose) for n in names}
        return {n: f.result() for n, f in futs.items()}


def load(name: str) -> ctypes.CDLL:
    """The loaded library of a module, built first when it has to be."""
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(name)
        if lib is None:
            path = build_module(name)
            try:
                lib = ctypes.CDLL(path)
            except OSError as e:
                raise KernelBuildError(f"cannot load kernel module {name!r} from {path}: {e}") from e
            _loaded[name] = lib
    return lib


def ensure(names: list[str]) -> None:
    """Build (side by side) and load the named modules."""
    missing = [n for n in names if n not in _loaded]
    if missing:
        build_modules(missing)
        for n in missing:
            load(n)
