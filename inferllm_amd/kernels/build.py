"""Compiling and loading the HIP kernel library (gfx950 only).

`library()` returns the loaded `ctypes.CDLL`.  It loads the built library beside
the sources when its stamp matches the sources' hash; otherwise it compiles
first (every `.hip` file with hipcc, then one link), printing a line per file so
a first call on a fresh checkout shows progress.  When the package folder cannot
be written to, the build goes to a per-user folder under the temporary
directory.  There is no fallback of any kind: a missing compiler or a failed
build raises `KernelLibraryError`.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from typing import List, Optional

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
LIB_NAME = "libinferllm_hip.so"
ARCH = "gfx950"
# -packed-fp32-ops off: the compiler must not form packed float32 instructions
HIPCC_FLAGS = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument"]


class KernelLibraryError(RuntimeError):
    pass


_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()


def sources() -> List[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers() -> List[str]:
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".h"))


def source_hash() -> str:
    h = hashlib.sha256()
    h.update(" ".join(HIPCC_FLAGS).encode())
    for f in sources() + _headers():
        h.update(f.encode())
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise KernelLibraryError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                             "the HIP kernels cannot be built, and there is no other path")


def _writable(d: str) -> bool:
    try:
        os.makedirs(d, exist_ok=True)
        probe = os.path.join(d, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def _out_dirs() -> List[str]:
    per_user = os.path.join(tempfile.gettempdir(), f"inferllm_amd_{os.getuid()}")
    return [CSRC, per_user]


def _stamp_path(d: str) -> str:
    return os.path.join(d, LIB_NAME + ".stamp")


def _built_in(d: str, want: Optional[str]) -> Optional[str]:
    lib = os.path.join(d, LIB_NAME)
    if not os.path.isfile(lib):
        return None
    if want is None:
        return lib
    try:
        with open(_stamp_path(d)) as f:
            return lib if f.read().strip() == want else None
    except OSError:
        return None


def build(verbose: bool = True, force: bool = True) -> str:
    """Compile every kernel source for gfx950 and link the library; returns its path."""
    want = source_hash()
    if not force:
        for d in _out_dirs():
            lib = _built_in(d, want)
            if lib:
                return lib
    hipcc = _hipcc()
    out_dir = next((d for d in _out_dirs() if _writable(d)), None)
    if out_dir is None:
        raise KernelLibraryError(f"no writable folder for the kernel library among {_out_dirs()}")
    obj_dir = os.path.join(out_dir, "_build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    say = (lambda m: print(f"[inferllm_amd] {m}", file=sys.stderr, flush=True)) if verbose else (lambda m: None)
    say(f"building {LIB_NAME} for {ARCH}: {len(srcs)} sources -> {out_dir}")
    t0 = time.time()

    def compile_one(src: str) -> str:
        obj = os.path.join(obj_dir, src[:-4] + ".o")
        cmd = [hipcc] + HIPCC_FLAGS + ["-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src}:\n{r.stdout}")
        say(f"  compiled {src} ({time.time() - t0:.0f} s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), os.cpu_count() or 1))
    with ThreadPoolExecutor(workers) as ex:
        objs = list(ex.map(compile_one, srcs))
    tmp = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    r = subprocess.run([hipcc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", tmp] + objs,
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise KernelLibraryError(f"linking {LIB_NAME} failed:\n{r.stdout}")
    os.replace(tmp, os.path.join(out_dir, LIB_NAME))
    with open(_stamp_path(out_dir), "w") as f:
        f.write(want + "\n")
    say(f"built in {time.time() - t0:.0f} s")
    return os.path.join(out_dir, LIB_NAME)


_C_TYPES = {"int": ctypes.c_int, "float": ctypes.c_float, "double": ctypes.c_double,
            "size_t": ctypes.c_size_t, "unsigned": ctypes.c_uint, "uint32_t": ctypes.c_uint32,
            "int32_t": ctypes.c_int32, "uint64_t": ctypes.c_uint64, "int64_t": ctypes.c_int64,
            "unsigned long long": ctypes.c_ulonglong, "long long": ctypes.c_longlong}


def _declare(lib: ctypes.CDLL) -> None:
    """Give every entry point of api.h its argument and result types, so that a call with the
    wrong number or kind of arguments raises here instead of reading garbage over there."""
    with open(os.path.join(CSRC, "api.h")) as f:
        text = re.sub(r"//[^\n]*", "", f.read())
    for ret, name, params in re.findall(r"\b(int|void)\s+(illm_\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        for prm in (p.strip() for p in params.split(",")):
            if not prm or prm == "void":
                continue
            if "*" in prm:
                types.append(ctypes.c_void_p)
                continue
            ctype = " ".join(w for w in prm.split()[:-1] if w != "const")
            if ctype not in _C_TYPES:
                raise KernelLibraryError(f"api.h: {name} has a parameter of type {ctype!r} that "
                                         "the loader does not know")
            types.append(_C_TYPES[ctype])
        try:
            fn = getattr(lib, name)
        except AttributeError:
            raise KernelLibraryError(f"{LIB_NAME} lacks {name}, which api.h declares: "
                                     "the library is not the one these sources build") from None
        fn.argtypes = types
        fn.restype = ctypes.c_int if ret == "int" else None


def library() -> ctypes.CDLL:
    """The loaded kernel library; built first if no current build exists."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = build(verbose=True, force=False)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from None
        _declare(lib)
        _lib = lib
        return _lib


def library_path() -> Optional[str]:
    return getattr(_lib, "_name", None) if _lib is not None else None
