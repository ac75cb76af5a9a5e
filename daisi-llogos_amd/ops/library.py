"""Builds and loads the HIP kernel library (gfx950) that every device op calls.

`build()` always compiles; `load()` uses the library that is there and compiles only
when none is, or when the one that is there was built from other sources.  There is no
fallback: without the library the ops raise.
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
from concurrent.futures import ThreadPoolExecutor

_CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
_PKG = os.path.dirname(_CSRC)
LIB_NAME = "libllogos_hip.so"
ARCH = "gfx950"

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    # packed 32-bit float instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]

_lock = threading.Lock()
_lib = None


class KernelLibraryError(RuntimeError):
    """The HIP kernel library is missing and could not be built, or failed to load."""


def _log(msg: str) -> None:
    print(f"[llogos] {msg}", file=sys.stderr, flush=True)


def sources() -> list:
    return sorted(f for f in os.listdir(_CSRC) if f.endswith(".hip"))


def _source_hash() -> str:
    h = hashlib.sha256()
    for name in sorted(os.listdir(_CSRC)):
        if name.endswith((".hip", ".h")):
            h.update(name.encode())
            with open(os.path.join(_CSRC, name), "rb") as fh:
                h.update(fh.read())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()


def _private(path: str) -> bool:
    """Whether a folder under the shared temporary directory is this user's alone (a library is
    never built into or loaded from a folder that another user could have written)."""
    try:
        st = os.stat(path)
    except OSError:
        return False
    return st.st_uid == os.getuid() and (st.st_mode & 0o077) == 0


def _writable(path: str) -> bool:
    try:
        os.makedirs(path, mode=0o700, exist_ok=True)
        if not path.startswith(_PKG) and not _private(path):
            return False
        probe = os.path.join(path, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def build_dirs() -> list:
    """Where a built library may live: in the tree, else a per-user folder under the
    temporary directory (for a tree the user cannot write to)."""
    dirs = [os.path.join(_PKG, "_build")]
    tmp = os.path.join(tempfile.gettempdir(), f"llogos_build_{os.getuid()}_{_source_hash()[:12]}")
    dirs.append(tmp)
    return dirs


def find_library() -> str | None:
    env = os.environ.get("LLOGOS_KERNEL_LIBRARY")
    if env:
        return env if os.path.isfile(env) else None
    stale = None
    for d in build_dirs():
        p = os.path.join(d, LIB_NAME)
        if os.path.isfile(p) and (d.startswith(_PKG) or _private(d)):
            if not is_stale(p):
                return p
            stale = stale or p          # one built from the present sources, in a later folder, goes first
    return stale


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelLibraryError("hipcc not found: the HIP kernel library cannot be built")


def _run_with_progress(cmd: list, what: str, env: dict) -> None:
    start = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, text=True)
    done = threading.Event()

    def ticker():
        while not done.wait(20.0):
            _log(f"still compiling {what} ({time.time() - start:.0f} s)")
    th = threading.Thread(target=ticker, daemon=True)
    th.start()
    out, _ = proc.communicate()
    done.set()
    if proc.returncode != 0:
        raise KernelLibraryError(f"hipcc failed on {what}:\n{out}")
    noise = ("packed-fp32-ops", "is not a recognized feature")
    for line in out.splitlines():
        if line.strip() and not any(n in line for n in noise):
            print(line, file=sys.stderr)


def build(verbose: bool = True) -> str:
    """Compile every .hip source for gfx950 and link the shared library.  Returns its path."""
    hipcc = _hipcc()
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise KernelLibraryError("no writable folder for the kernel library")
    env = dict(os.environ)
    # an empty or unwritable HOME must not stop the compiler from keeping its temporaries
    env.setdefault("TMPDIR", tempfile.gettempdir())
    srcs = sources()
    # every build has object files of its own: two processes that build at once (test workers that
    # both find a stale library) must not link each other's half-written objects
    obj_dir = tempfile.mkdtemp(prefix=f"obj.{os.getpid()}.", dir=out_dir)
    stamp = _source_hash()                               # of the sources as they are now, before they are compiled
    if verbose:
        _log(f"building {LIB_NAME} for {ARCH} from {len(srcs)} sources into {out_dir}")
    t0 = time.time()
    counter = {"n": 0}

    def compile_one(name: str) -> str:
        obj = os.path.join(obj_dir, name[:-4] + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", _CSRC, "-c", os.path.join(_CSRC, name), "-o", obj]
        _run_with_progress(cmd, name, env)
        with _lock:
            counter["n"] += 1
            if verbose:
                _log(f"compiled {name} ({counter['n']}/{len(srcs)}, {time.time() - t0:.0f} s)")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    tmp_lib = os.path.join(out_dir, f".{LIB_NAME}.{os.getpid()}")
    tmp_stamp = os.path.join(out_dir, f".sources.sha256.{os.getpid()}")
    lib_path = os.path.join(out_dir, LIB_NAME)
    try:
        with ThreadPoolExecutor(max_workers=workers) as pool:
            objs = list(pool.map(compile_one, srcs))
        _run_with_progress([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", tmp_lib, *objs], "link", env)
        with open(tmp_stamp, "w") as fh:
            fh.write(stamp)
        # A reader must never see a library under a stamp that is not its own: the old stamp is taken
        # away first (a library without a stamp counts as stale), then the library is put in place,
        # then its stamp; both are written beside their places and renamed, so neither is ever half there.
        try:
            os.remove(os.path.join(out_dir, "sources.sha256"))
        except OSError:
            pass
        os.replace(tmp_lib, lib_path)
        os.replace(tmp_stamp, os.path.join(out_dir, "sources.sha256"))
    finally:
        shutil.rmtree(obj_dir, ignore_errors=True)
        for leftover in (tmp_lib, tmp_stamp):
            try:
                os.remove(leftover)
            except OSError:
                pass
    if verbose:
        _log(f"built {lib_path} in {time.time() - t0:.0f} s")
    global _lib
    _lib = None
    return lib_path


_C_TYPES = {"int": ctypes.c_int, "float": ctypes.c_float, "double": ctypes.c_double, "long long": ctypes.c_longlong,
            "unsigned": ctypes.c_uint, "hipStream_t": ctypes.c_void_p}


def exported_signatures() -> dict:
    """name -> (result type, [argument types]) of every entry point, read from the sources'
    LLOGOS_EXPORT declarations (pointers of any kind are c_void_p).  An entry point whose
    declaration uses a type this does not know raises: a wrong guess would pass wrong bits."""
    import re
    found = {}
    for name in sources():
        with open(os.path.join(_CSRC, name)) as fh:
            text = fh.read()
        for m in re.finditer(r"LLOGOS_EXPORT\s+([\w\s\*]+?)\s*\b(\w+)\s*\(([^)]*)\)", text):
            ret, fn, args = m.groups()

            def ctype(decl: str, named: bool):
                decl = " ".join(decl.replace("*", " * ").split())
                if "*" in decl:
                    return ctypes.c_void_p
                words = [w for w in decl.split() if w != "const"]
                if named and len(words) > 1:
                    words = words[:-1]                       # the parameter's name
                key = " ".join(words)
                if key not in _C_TYPES:
                    raise KernelLibraryError(f"{name}: entry point {fn} uses the type '{key}', which has no ctypes counterpart here")
                return _C_TYPES[key]
            arg_list = [a for a in (x.strip() for x in args.split(",")) if a and a != "void"]
            found[fn] = (ctype(ret, False), [ctype(a, True) for a in arg_list])
    return found


def declare(lib: ctypes.CDLL) -> None:
    """Argument and result types for every entry point, so that a call with too few arguments,
    an integer that does not fit or a tensor where a number belongs raises instead of passing
    wrong bits to a kernel."""
    for fn, (ret, args) in exported_signatures().items():
        try:
            f = getattr(lib, fn)
        except AttributeError:
            raise KernelLibraryError(f"the library has no entry point {fn}, which the sources declare") from None
        f.restype, f.argtypes = ret, args


def is_stale(lib_path: str) -> bool:
    stamp = os.path.join(os.path.dirname(lib_path), "sources.sha256")
    try:
        with open(stamp) as fh:
            return fh.read().strip() != _source_hash()
    except OSError:
        return True


def load() -> ctypes.CDLL:
    """The loaded kernel library; built first if no built library exists."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
    path = find_library()
    if path is None:
        path = build()
    elif not os.environ.get("LLOGOS_KERNEL_LIBRARY") and is_stale(path):
        # Python's declarations of the entry points describe the present sources: a library built
        # from other sources would take wrong pointers and strides.  (A library named by
        # LLOGOS_KERNEL_LIBRARY is the user's word and is trusted.)
        _log(f"{path} was built from other sources than those in {_CSRC}: building again")
        try:
            path = build()
        except KernelLibraryError as e:
            raise KernelLibraryError(f"{path} is stale and cannot be rebuilt: {e}") from e
    try:
        lib = ctypes.CDLL(path)
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from e
    declare(lib)
    from ..cache.pages import PAGE_TOKENS, key_offset, value_offset
    if lib.llogos_page_tokens() != PAGE_TOKENS:
        raise KernelLibraryError(f"{path} was built for pages of {lib.llogos_page_tokens()} positions, "
                                 f"the cache uses {PAGE_TOKENS}")
    for token, d, hd in ((0, 0, 16), (5, 9, 16), (63, 127, 128), (37, 70, 96), (18, 33, 64), (44, 255, 256)):
        if (lib.llogos_page_key_offset(token, d, hd) != key_offset(token, d, hd)
                or lib.llogos_page_value_offset(token, d) != value_offset(token, d)):
            raise KernelLibraryError(f"{path} lays pages out otherwise than cache/pages.py does")
    with _lock:
        _lib = lib
    return lib
