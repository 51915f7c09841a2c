"""Compiles the HIP sources under ``csrc/`` for gfx950 into one shared library and loads it.

``build()`` always compiles.  ``load()`` takes the library that is there and compiles only when there
is none, printing a line per file so that a first call in a fresh checkout shows progress.  The
library sits beside this file; when that folder cannot be written (a read-only checkout) it goes to a
folder under the system's temporary directory instead, named for the user and for the sources' contents, so
that a library built from other sources is never picked up there.  Beside the library lies a stamp with the
hash of the sources it was built from; when the stamp and the sources differ, ``load()`` says so on stderr and
builds again instead of loading it.
There is no fallback: without the library every op raises.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent.parent
CSRC = PKG / "csrc"
LIB_NAME = "libminiserve_gfx950.so"
ARCH = "gfx950"
# -packed-fp32-ops off: hipcc must not form packed float instructions from scalar code
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

_lib = None


class KernelLibraryError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"),
                 os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "bin", "hipcc")):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelLibraryError("hipcc not found (looked at $HIPCC, PATH and $ROCM_PATH/bin); the HIP kernels "
                             "cannot be built and there is no fallback")


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def source_hash() -> str:
    """A short hash of everything the library is compiled from."""
    h = hashlib.sha256()
    for f in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(f.name.encode())
        h.update(f.read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:12]


def _fallback_dir() -> Path:
    return Path(tempfile.gettempdir()) / f"llm_infrence_engine_amd-{os.getuid()}-{source_hash()}"


def _stamp_of(lib: Path) -> Path:
    return lib.with_suffix(".stamp")


def built_from(lib: Path) -> str:
    """The hash of the sources ``lib`` was built from, as its stamp says."""
    stamp = _stamp_of(lib)
    return stamp.read_text().strip() if stamp.is_file() else "unknown sources"


def library_path() -> Path | None:
    """The built library, or None."""
    for d in (PKG / "kernels", _fallback_dir()):
        p = d / LIB_NAME
        if p.is_file():
            return p
    return None


def sources() -> list:
    return sorted(CSRC.glob("*.hip"))


def build(verbose: bool = True) -> Path:
    """Compile every ``csrc/*.hip`` and link the library.  Returns its path."""
    hipcc = _hipcc()
    out_dir = PKG / "kernels"
    if not _writable(out_dir):
        out_dir = _fallback_dir()
        if not _writable(out_dir):
            raise KernelLibraryError(f"neither {PKG / 'kernels'} nor {out_dir} can be written")
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise KernelLibraryError(f"no HIP sources under {CSRC}")
    t0 = time.time()

    def say(msg):
        if verbose:
            print(f"[kernels {time.time() - t0:5.1f}s] {msg}", file=sys.stderr, flush=True)

    say(f"compiling {len(srcs)} HIP sources for {ARCH} with {hipcc}")

    def compile_one(src: Path):
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src.name}:\n{r.stdout}\n{r.stderr}")
        say(f"compiled {src.name}")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 4, 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", str(tmp), *map(str, objs)],
                       capture_output=True, text=True)
    if r.returncode != 0:
        raise KernelLibraryError(f"linking {LIB_NAME} failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, out_dir / LIB_NAME)
    _stamp_of(out_dir / LIB_NAME).write_text(source_hash() + "\n")
    say(f"linked {out_dir / LIB_NAME}")
    global _lib
    _lib = None
    return out_dir / LIB_NAME


def resource_usage() -> dict:
    """What every kernel of the library needs, from the compiler's own report: {kernel: {"vgprs", "agprs",
    "scratch" (bytes a lane: registers spilled to memory), "lds", "occupancy"}}.  Compiles the device code of
    every source again (no library is written)."""
    import re

    hipcc = _hipcc()

    def one(src: Path):
        cmd = [hipcc, *FLAGS, "-I", str(CSRC), "-c", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage",
               "-o", os.devnull, str(src)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {src.name}:\n{r.stdout}\n{r.stderr}")
        found, name = {}, None
        keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch", "LDS Size [bytes/block]": "lds",
                "Occupancy [waves/SIMD]": "occupancy"}
        for line in r.stderr.splitlines():
            m = re.search(r"remark:\s+(.*?): (\S+) \[-Rpass-analysis", line)
            if not m:
                continue
            what, value = m.group(1).strip(), m.group(2)
            if what == "Function Name":
                name = value
                found[name] = {}
            elif name and what in keys:
                found[name][keys[what]] = int(value)
        return found

    out = {}
    with ThreadPoolExecutor(max(1, min(len(sources()), os.cpu_count() or 4, 16))) as pool:
        for d in pool.map(one, sources()):
            out.update(d)
    return out


def load() -> ctypes.CDLL:
    """The loaded library; built first if it does not exist yet."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (its HIP runtime must be the one in the process before ours binds to it)

    path = library_path()
    if path is not None and built_from(path) != source_hash():
        # a library older than its sources is never loaded: numbers and test results would be those of other code
        print(f"[kernels] {path} was built from {built_from(path)}, the sources under {CSRC} are {source_hash()}: "
              f"building it again", file=sys.stderr, flush=True)
        path = None
    if path is None:
        path = build(verbose=True)
    try:
        _lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise KernelLibraryError(f"cannot load {path}: {e}") from e
    return _lib
