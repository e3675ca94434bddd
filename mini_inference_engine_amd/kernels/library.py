"""Building and loading the HIP kernel libraries.

Each ``csrc/<module>.hip`` becomes one shared library with a plain C interface
(raw device pointers and a stream), built by hipcc for gfx950 and loaded through
ctypes.  A library's file name carries a digest of its source, the shared header
and the flags, so a changed source is never served by a stale build.  Libraries
are built into ``csrc/_build`` (or a per-user folder under the temporary
directory when the tree is read-only); a module that is not built yet is built
at its first use, with a progress line now and then.  There is no other
implementation to fall back on: if a library can neither be found nor built,
loading raises.
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

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-fno-gpu-sanitize",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


class KernelModule:
    """One HIP source that becomes one shared library (per variant).  ``signatures``: entry point ->
    ctypes argument types (every entry point returns int: 0, or a negative code with a message readable
    through <name>_last_error()).  ``variants``: lists of -D defines built ahead of time; others compile at
    first use.  ``flags``: compiler flags beside FLAGS.  ``source``: the .hip file (by default csrc/<name>.hip);
    a module outside the package hashes its own file and this package's headers."""

    def __init__(self, name, signatures=None, variants=None, flags=None, source=None):
        self.name = name
        self.signatures = dict(signatures or {})
        self.variants = [tuple(v) for v in (variants or [()])]
        self.flags = list(flags or [])
        self.source = source or os.path.join(CSRC, name + ".hip")


MODULES: dict[str, KernelModule] = {}


def register_kernel_module(name: str, signatures=None, variants=None, flags=None, source=None) -> KernelModule:
    """Make a kernel source known to the loader, the build-everything step and the backend's
    declaration of argument types.  A part that brings a kernel of its own calls this (from outside the
    package too) and then reaches its entry points through ``HipBackend.lib(name)``."""
    MODULES[name] = KernelModule(name, signatures, variants, flags, source)
    return MODULES[name]


def kernel_module(name: str) -> KernelModule:
    if name not in MODULES:
        raise KernelLibraryError(f"kernel module {name!r} is not registered (known: {sorted(MODULES)})")
    return MODULES[name]


_loaded: dict = {}
_lock = threading.Lock()


class KernelLibraryError(RuntimeError):
    pass


def available_modules() -> list[str]:
    return [name for name, m in MODULES.items() if os.path.isfile(m.source)]


def _digest(name: str, defines: tuple) -> str:
    mod = kernel_module(name)
    h = hashlib.sha256()
    for path in [mod.source] + sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")):
        with open(path, "rb") as f:
            h.update(f.read())
    h.update(" ".join(FLAGS + mod.flags + [ARCH] + list(defines)).encode())
    return h.hexdigest()[:16]


def _tag(defines: tuple) -> str:
    return "".join("_" + d.replace("=", "").replace("-D", "") for d in defines)


def _build_dirs() -> list[str]:
    dirs = [os.path.join(CSRC, "_build")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"mini_inference_engine_amd_build_{uid}"))
    return dirs


def _trusted(d: str) -> bool:
    """Libraries are loaded into the process, so a folder outside the package counts only if it is this
    user's own and nobody else can write to it (the per-user folder under the temporary directory has a
    name anyone could have created first)."""
    if os.path.dirname(os.path.abspath(d)) == os.path.abspath(CSRC):
        return True
    try:
        st = os.stat(d)
    except OSError:
        return False
    return (not hasattr(os, "getuid") or st.st_uid == os.getuid()) and not (st.st_mode & 0o022)


def library_file(module: str, defines: tuple = ()) -> str:
    return f"{module}{_tag(defines)}-{_digest(module, defines)}.so"


def find_built(module: str, defines: tuple = ()) -> str | None:
    name = library_file(module, defines)
    for d in _build_dirs():
        p = os.path.join(d, name)
        if os.path.isfile(p) and _trusted(d):
            return p
    return None


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if c and os.path.isfile(c):
            return c
    raise KernelLibraryError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the kernels cannot be built")


def build(module: str, defines: tuple = (), verbose: bool = True) -> str:
    """Compile one module now (also when a built file is already there)."""
    mod = kernel_module(module)
    src = mod.source
    if not os.path.isfile(src):
        raise KernelLibraryError(f"no kernel source {src}")
    name = library_file(module, defines)
    out_dir = None
    for d in _build_dirs():
        try:
            os.makedirs(d, mode=0o700, exist_ok=True)
            if not _trusted(d):
                continue
            fd, probe = tempfile.mkstemp(dir=d, prefix=".w")
            os.close(fd)
            os.remove(probe)
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise KernelLibraryError(f"no writable folder to build kernels in (tried {_build_dirs()})")
    out = os.path.join(out_dir, name)
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.{threading.get_ident()}.tmp")
    cmd = [_hipcc(), f"--offload-arch={ARCH}", *FLAGS, *mod.flags, *defines, "-I", CSRC, src, "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)        # hipcc's helpers want some HOME; an empty one is fine
    t0 = time.time()
    if verbose:
        print(f"[mini_inference_engine_amd] compiling {module}.hip {' '.join(defines)} for {ARCH} ...",
              file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    lines = []

    def _drain():
        for ln in proc.stdout:
            lines.append(ln)

    th = threading.Thread(target=_drain, daemon=True)
    th.start()
    while proc.poll() is None:
        try:
            proc.wait(timeout=10)
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[mini_inference_engine_amd]   ... still compiling {module}.hip ({time.time() - t0:.0f} s)",
                      file=sys.stderr, flush=True)
    th.join()
    log = "".join(ln for ln in lines if "packed-fp32-ops" not in ln)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise KernelLibraryError(f"hipcc failed on {module}.hip:\n{log}")
    os.replace(tmp, out)
    # older builds of the same module and defines are of no use any more
    prefix = f"{module}{_tag(defines)}-"
    for fn in os.listdir(out_dir):
        if fn.startswith(prefix) and fn.endswith(".so") and fn != name:
            try:
                os.remove(os.path.join(out_dir, fn))
            except OSError:
                pass
    if verbose:
        print(f"[mini_inference_engine_amd]   built {name} in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    return out


def load(module: str, defines: tuple = ()) -> ctypes.CDLL:
    """The module's library, built first if no current build exists."""
    key = (module, tuple(defines))
    with _lock:
        if key in _loaded:
            return _loaded[key]
        path = find_built(module, tuple(defines)) or build(module, tuple(defines))
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from e
        err = getattr(lib, f"{module}_last_error")
        err.restype = ctypes.c_char_p
        lib._mie_error = err
        lib._mie_path = path
        for entry, argtypes in kernel_module(module).signatures.items():
            fn = getattr(lib, entry)
            fn.argtypes = list(argtypes)
            fn.restype = ctypes.c_int
        _loaded[key] = lib
        return lib


def build_all(verbose: bool = True, jobs: int = 4) -> list[str]:
    """Compile every module and variant the engine and its tests use."""
    from concurrent.futures import ThreadPoolExecutor
    work = []
    for m in available_modules():
        for defines in variants_of(m):
            work.append((m, defines))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        return list(ex.map(lambda w: build(w[0], w[1], verbose), work))


def variants_of(name: str) -> list[tuple]:
    """Compile-time variants of a module built ahead of time; plain modules have one (no defines)."""
    return list(kernel_module(name).variants)


def check(lib, code: int) -> None:
    if code != 0:
        raise RuntimeError(lib._mie_error().decode(errors="replace"))


from . import modules as _builtin_modules  # noqa: E402,F401  (registers the package's own kernel modules)
