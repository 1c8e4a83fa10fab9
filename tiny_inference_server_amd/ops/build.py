"""Compiles the HIP sources under csrc/ for gfx950 and loads the results with ctypes.

Every source file becomes one shared library of plain C entry points, so a first call in a fresh
checkout compiles only what it uses, in seconds, without torch headers. A library's file name carries a
hash of its source, the shared header and the compiler flags: an edited source is never served by a
stale library. Libraries are kept under csrc/_build/ when that is writable, else in a per-user
folder under the system's temporary directory.
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
from typing import Dict, Iterable, List, Optional

CSRC = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))

ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-shared", "-fPIC",
    # packed 32-bit float instructions stay off
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# library name -> source file; headers every library depends on
SOURCES: Dict[str, str] = {
    "rowwise": "rowwise.hip",
    "rope_cache": "rope_cache.hip",
    "attention_generic": "attention_generic.hip",
    "attention_mfma": "attention_mfma.hip",
    "gemm_plain": "gemm_plain.hip",
    "gemm_skinny": "gemm_skinny.hip",
    "gemm_library": "gemm_library.hip",
    "gemm_tiles": "gemm_tiles.hip",
    "sampling": "sampling.hip",
}
HEADERS = ["common.h", "attention_mfma.h"]
# what a library links beyond the HIP runtime
LINK: Dict[str, List[str]] = {"gemm_library": ["-lhipblaslt"]}

_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def available_sources() -> List[str]:
    """Every library that build() makes by default, variants spelled out."""
    out = []
    for n, f in SOURCES.items():
        if not os.path.isfile(os.path.join(CSRC, f)):
            continue
        if n in VARIANTS:
            out.extend(f"{n}@{v}" for v in VARIANTS[n][1])
        else:
            out.append(n)
    return out


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be built")


# libraries compiled once per value of a macro: name -> (macro, values that build() makes without being asked)
VARIANTS: Dict[str, tuple] = {
    "attention_mfma": ("TIS_HD", (32, 48, 64, 128, 256)),
}


def split_variant(name: str):
    """'attention_mfma@128' -> ('attention_mfma', ['-DTIS_HD=128'])."""
    if "@" not in name:
        if name in VARIANTS:
            raise BuildError(f"library {name!r} is built per {VARIANTS[name][0]}: ask for '{name}@<value>'")
        return name, []
    base, value = name.split("@", 1)
    if base not in VARIANTS:
        raise BuildError(f"library {base!r} has no variants")
    return base, [f"-D{VARIANTS[base][0]}={int(value)}"]


def _digest(name: str) -> str:
    base, defines = split_variant(name)
    h = hashlib.sha1()
    for f in [SOURCES[base]] + HEADERS:
        with open(os.path.join(CSRC, f), "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(FLAGS + defines + LINK.get(base, [])).encode())
    return h.hexdigest()[:12]


def _build_dirs() -> List[str]:
    dirs = []
    if os.environ.get("TIS_AMD_BUILD_DIR"):
        dirs.append(os.environ["TIS_AMD_BUILD_DIR"])
    dirs.append(os.path.join(CSRC, "_build"))
    dirs.append(os.path.join(tempfile.gettempdir(), f"tis_amd_build_{os.getuid()}"))
    return dirs


def _writable_dir() -> str:
    for d in _build_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe_{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the compiled kernels; tried " + ", ".join(_build_dirs()))


def library_file(name: str) -> Optional[str]:
    """Path of the up-to-date built library of `name`, or None if there is none."""
    fname = f"{name}.{_digest(name)}.so"
    for d in _build_dirs():
        p = os.path.join(d, fname)
        if os.path.isfile(p):
            return p
    return None


def _compile(name: str, out_dir: str) -> str:
    base, defines = split_variant(name)
    src = os.path.join(CSRC, SOURCES[base])
    out = os.path.join(out_dir, f"{name}.{_digest(name)}.so")
    tmp = f"{out}.tmp{os.getpid()}"
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env["HOME"], os.W_OK):
        env["HOME"] = out_dir   # the compiler may want a cache folder
    cmd = [_hipcc()] + FLAGS + defines + ["-I", CSRC, "-o", tmp, src] + LINK.get(base, [])
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        raise BuildError(f"hipcc failed on {SOURCES[base]} ({name}):\n{proc.stdout[-4000:]}")
    os.replace(tmp, out)
    # older builds of the same library are of no further use
    for f in os.listdir(out_dir):
        if f.startswith(name + ".") and f.endswith(".so") and os.path.join(out_dir, f) != out:
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    return out


def build(names: Optional[Iterable[str]] = None, force: bool = False, log=None) -> Dict[str, str]:
    """Compile the named libraries (default: all) that are missing, or all of them with `force`.

    Compilations run side by side; while they run a line is printed every few seconds.
    """
    log = log or (lambda s: print(s, file=sys.stderr, flush=True))
    names = list(names) if names is not None else available_sources()
    for n in names:
        if split_variant(n)[0] not in SOURCES:
            raise BuildError(f"unknown kernel library {n!r}; known: {', '.join(SOURCES)}")
    result: Dict[str, str] = {}
    todo = []
    for n in names:
        have = None if force else library_file(n)
        if have:
            result[n] = have
        else:
            todo.append(n)
    if not todo:
        return result
    out_dir = _writable_dir()
    log(f"[tis-amd] compiling {len(todo)} HIP kernel librar{'y' if len(todo) == 1 else 'ies'} for {ARCH}: "
        f"{', '.join(todo)} -> {out_dir}")
    errors: Dict[str, BaseException] = {}
    done: List[str] = []

    def work(n):
        try:
            result[n] = _compile(n, out_dir)
        except BaseException as e:  # reported below
            errors[n] = e
        done.append(n)

    threads = [threading.Thread(target=work, args=(n,), daemon=True) for n in todo]
    t0 = time.time()
    for t in threads:
        t.start()
    last = t0
    while any(t.is_alive() for t in threads):
        time.sleep(0.2)
        if time.time() - last > 5:
            last = time.time()
            log(f"[tis-amd] still compiling ({len(done)}/{len(todo)} done, {last - t0:.0f} s)")
    if errors:
        raise BuildError("\n".join(str(e) for e in errors.values()))
    log(f"[tis-amd] compiled {len(todo)} in {time.time() - t0:.1f} s")
    return result


def load(name: str) -> ctypes.CDLL:
    """The loaded library `name`; compiled first if no current build exists."""
    with _lock:
        lib = _loaded.get(name)
        if lib is not None:
            return lib
        path = library_file(name) or build([name])[name]
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise BuildError(f"cannot load {path}: {e}") from None
        _loaded[name] = lib
        return lib
