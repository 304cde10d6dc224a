"""Compile the HIP sources of this folder for gfx950 into one shared library, in-tree.

`build()` always compiles.  `ensure_built()` compiles only when no library matching the current sources is
there (a fresh checkout's first call), printing a line per file so that a waiting user sees progress.  The
library is plain C ABI (`api.h`), loaded with ctypes; nothing here depends on a Python extension toolchain,
a home directory or a network.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCES = ("elementwise.hip", "gemm.hip", "gemm_mfma.hip", "gemm_mid.hip", "gemm_decode.hip", "attention.hip", "sampling.hip")
HEADERS = ("common.h", "mfma_tiles.h", "api.h")
LIBRARY = "libakv_kernels.so"
ATTENTION_SOURCE = "attention_mfma.hip"        # compiled once per head size, into its own small library
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 192, 256)
ARCH = "gfx950"
# packed-fp32 instructions are switched off for all device code of this library
FLAGS = ("-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
         "-packed-fp32-ops", "-Wno-unused-command-line-argument")


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the HIP kernels cannot be "
                       "built, and the engine has no other way to compute")


def source_stamp(sources=None) -> str:
    digest = hashlib.sha256()
    for name in (SOURCES if sources is None else tuple(sources)) + HEADERS:
        with open(os.path.join(HERE, name), "rb") as handle:
            digest.update(name.encode() + b"\0" + handle.read())
    digest.update(" ".join(FLAGS).encode())
    return digest.hexdigest()


_BUILD_DIR: str | None = None
_BUILD_DIR_LOCK = threading.Lock()


def _build_dir() -> str:
    """`_build/` beside the sources; a per-user temporary folder when the tree cannot be written.  Decided once
    (several head sizes are compiled by threads of one process)."""
    global _BUILD_DIR
    with _BUILD_DIR_LOCK:
        if _BUILD_DIR is None:
            local = os.path.join(HERE, "_build")
            try:
                os.makedirs(local, exist_ok=True)
                probe = os.path.join(local, f".probe{os.getpid()}")
                with open(probe, "w"):
                    pass
                os.remove(probe)
                _BUILD_DIR = local
            except OSError:
                _BUILD_DIR = os.path.join(tempfile.gettempdir(), f"akv_build_{os.getuid()}_{source_stamp()[:12]}")
                os.makedirs(_BUILD_DIR, exist_ok=True)
        return _BUILD_DIR


def library_path() -> str | None:
    """The built library matching the current sources, or None."""
    stamp = source_stamp()
    for folder in (os.path.join(HERE, "_build"),
                   os.path.join(tempfile.gettempdir(), f"akv_build_{os.getuid()}_{stamp[:12]}")):
        lib, mark = os.path.join(folder, LIBRARY), os.path.join(folder, "stamp")
        if os.path.exists(lib) and os.path.exists(mark):
            with open(mark) as handle:
                if handle.read().strip() == stamp:
                    return lib
    return None


def _log(message: str) -> None:
    print(f"[akv build] {message}", file=sys.stderr, flush=True)


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = _build_dir()
    started = time.time()
    if verbose:
        _log(f"compiling {len(SOURCES)} HIP sources for {ARCH} into {out_dir}")

    def compile_one(name: str) -> str:
        obj = os.path.join(out_dir, name.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(HERE, name), "-o", obj]
        result = subprocess.run(cmd, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{result.stderr}")
        if verbose:
            _log(f"compiled {name} ({time.time() - started:.0f} s)")
        return obj

    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    lib = os.path.join(out_dir, LIBRARY)
    partial = lib + f".{os.getpid()}.tmp"
    result = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objects, "-o", partial],
                            capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"linking {LIBRARY} failed:\n{result.stderr}")
    os.replace(partial, lib)
    with open(os.path.join(out_dir, "stamp"), "w") as handle:
        handle.write(source_stamp())
    if verbose:
        _log(f"linked {lib} ({time.time() - started:.0f} s)")
    return lib


def ensure_built(verbose: bool = True) -> str:
    return library_path() or build(verbose)


# ---- the attention kernels, one library per head size ------------------------------------------------------------

def _attention_names(head_dim: int) -> tuple[str, str]:
    return f"libakv_attention_d{head_dim}.so", f"stamp_attention_d{head_dim}"


def attention_library_path(head_dim: int) -> str | None:
    stamp = source_stamp((ATTENTION_SOURCE,))
    lib_name, mark_name = _attention_names(head_dim)
    for folder in (os.path.join(HERE, "_build"),
                   os.path.join(tempfile.gettempdir(), f"akv_build_{os.getuid()}_{source_stamp()[:12]}")):
        lib, mark = os.path.join(folder, lib_name), os.path.join(folder, mark_name)
        if os.path.exists(lib) and os.path.exists(mark):
            with open(mark) as handle:
                if handle.read().strip() == stamp:
                    return lib
    return None


def build_attention(head_dim: int, verbose: bool = True) -> str:
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise ValueError(f"the attention kernels take head sizes that are multiples of 16 up to 256, not {head_dim}")
    hipcc = _hipcc()
    out_dir = _build_dir()
    started = time.time()
    lib_name, mark_name = _attention_names(head_dim)
    lib = os.path.join(out_dir, lib_name)
    partial = lib + f".{os.getpid()}.tmp"
    if verbose:
        _log(f"compiling {ATTENTION_SOURCE} for head size {head_dim}")
    cmd = [hipcc, *FLAGS, f"-DAKV_HEAD_DIM={head_dim}", "-shared", os.path.join(HERE, ATTENTION_SOURCE), "-o", partial]
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed on {ATTENTION_SOURCE} (head size {head_dim}):\n{result.stderr}")
    os.replace(partial, lib)
    with open(os.path.join(out_dir, mark_name), "w") as handle:
        handle.write(source_stamp((ATTENTION_SOURCE,)))
    if verbose:
        _log(f"built {lib} ({time.time() - started:.0f} s)")
    return lib


def ensure_attention(head_dim: int, verbose: bool = True) -> str:
    return attention_library_path(head_dim) or build_attention(head_dim, verbose)


def build_all(head_dims=DEFAULT_HEAD_DIMS, verbose: bool = True) -> list[str]:
    """The kernel library and the attention libraries of the usual head sizes."""
    paths = [build(verbose)]
    with ThreadPoolExecutor(max_workers=4) as pool:
        paths += list(pool.map(lambda d: build_attention(d, verbose), head_dims))
    return paths


if __name__ == "__main__":
    print("\n".join(build_all()))
