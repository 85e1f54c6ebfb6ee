"""Compile the HIP sources under ``csrc/`` for gfx950 and load them with ctypes.

Every source file becomes one shared library, ``_lib/<name>.so`` beside this
package, so a run compiles only the kernels it calls.  A library is rebuilt
when its source (or ``common.h``) differs from the stamp written at its last
build; when ``hipcc`` is absent a stale or missing library is an error, never a
silent fallback.  If the package folder cannot be written, libraries go to a
per-user folder under the temporary directory.
"""

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(_PKG, "csrc")

SOURCES = ("embed", "norm", "gemm_f32", "gemm_bf16", "gemm_bf16_decode", "attention", "attention_decode", "attention_prefill", "sampling", "engine")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-shared",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]

_lock = threading.Lock()
_loaded = {}


class ExtensionError(RuntimeError):
    """A HIP library is missing, stale without a compiler, or failed to build."""


def _hipcc():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


def _lib_dir():
    d = os.path.join(_PKG, "_lib")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.unlink(probe)
        return d
    except OSError:
        d = os.path.join(tempfile.gettempdir(), f"mlx_lm_amd-lib-{os.getuid()}")
        os.makedirs(d, exist_ok=True)
        return d


def _readonly_lib_dir():
    return os.path.join(_PKG, "_lib")


def _source(name):
    """The path of the source called ``name``: one of ``csrc/``, or one registered with ``add_source``."""
    return _extra_sources.get(name) or os.path.join(CSRC, name + ".hip")


_extra_sources = {}


def add_source(path):
    """Make a ``.hip`` file outside ``csrc/`` known (a native part of a library of its own, which
    includes ``engine_parts.h``): ``load(name)`` then builds and loads it like the others, its
    library beside its source under ``_lib/``.  Returns the name (the file's, without ``.hip``)."""
    path = os.path.abspath(path)
    name = os.path.splitext(os.path.basename(path))[0]
    if name in SOURCES:
        raise ExtensionError(f"'{name}' is the name of one of the package's own sources")
    if not os.path.exists(path):
        raise ExtensionError(f"no such source: {path}")
    _extra_sources[name] = path
    return name


def _digest(name):
    h = hashlib.sha256()
    headers = sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))
    for f in [_source(name)] + [os.path.join(CSRC, h) for h in headers]:
        with open(f, "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def _is_current(so, name):
    stamp = so + ".stamp"
    if not (os.path.exists(so) and os.path.exists(stamp)):
        return False
    with open(stamp) as fh:
        return fh.read().strip() == _digest(name)


def compile_one(name, out_dir=None, verbose=True):
    """Compile ``csrc/<name>.hip`` into ``<out_dir>/<name>.so``; returns the path."""
    hipcc = _hipcc()
    if hipcc is None:
        raise ExtensionError(f"hipcc not found; cannot build the '{name}' kernels")
    out_dir = out_dir or _out_dir(name)
    so = os.path.join(out_dir, name + ".so")
    tmp = f"{so}.{os.getpid()}.tmp"
    cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, _source(name), "-o", tmp]
    t0 = time.time()
    if verbose:
        print(f"[mlx_lm_amd] compiling {name}.hip for gfx950 ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    # a line now and then while the compiler runs
    while True:
        try:
            out, err = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(
                    f"[mlx_lm_amd] still compiling {name}.hip ({time.time() - t0:.0f} s)",
                    file=sys.stderr,
                    flush=True,
                )
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.unlink(tmp)
        lines = [l for l in err.splitlines() if "not a recognized feature" not in l]
        raise ExtensionError(f"hipcc failed on {name}.hip:\n" + "\n".join(lines[-40:]))
    os.replace(tmp, so)
    with open(so + ".stamp", "w") as fh:
        fh.write(_digest(name))
    if verbose:
        print(f"[mlx_lm_amd] built {name}.so in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return so


def _out_dir(name):
    """Where the library of source ``name`` goes: the package's ``_lib/``, or for a source
    registered with ``add_source`` a ``_lib/`` beside it (the temporary folder if neither can be written)."""
    if name not in _extra_sources:
        return _lib_dir()
    d = os.path.join(os.path.dirname(_extra_sources[name]), "_lib")
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".w{os.getpid()}")
        with open(probe, "w"):
            pass
        os.unlink(probe)
        return d
    except OSError:
        return _lib_dir()


def build_all(verbose=True):
    """Compile every source, whether or not a built library is there."""
    d = _lib_dir()
    return [compile_one(n, d, verbose) for n in SOURCES] + [compile_one(n, None, verbose) for n in _extra_sources]


def load(name):
    """The ctypes library for ``csrc/<name>.hip``, built first if need be."""
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        if name not in SOURCES and name not in _extra_sources:
            raise ExtensionError(f"no kernel source named '{name}'")
        so = None
        dirs = (_readonly_lib_dir(), _lib_dir())
        if name in _extra_sources:
            dirs = (os.path.join(os.path.dirname(_extra_sources[name]), "_lib"),) + dirs
        for d in dirs:
            cand = os.path.join(d, name + ".so")
            if _is_current(cand, name):
                so = cand
                break
        if so is None:
            if _hipcc() is None:
                raise ExtensionError(
                    f"the '{name}' kernels are not built (or older than their source) and "
                    "hipcc is not available; run __graft_entry__.build() where hipcc is"
                )
            so = compile_one(name)
        try:
            lib = ctypes.CDLL(so)
        except OSError as e:
            raise ExtensionError(f"cannot load {so}: {e}") from e
        if hasattr(lib, "mlxlm_last_error"):  # (a part of a library of its own reports through the host's)
            lib.mlxlm_last_error.restype = ctypes.c_char_p
        _loaded[name] = lib
        return lib


def check(lib, code, what):
    if code != 0:
        raise RuntimeError(lib.mlxlm_last_error().decode() or f"{what} failed")
