"""Compiling the HIP sources under `csrc/` into one shared library for gfx950.

`build()` always compiles; `ensure_built()` compiles only when no library
matching the current sources exists, which is what happens at the first call in
a fresh checkout.  The library lives in-tree (`kernels/_lib/`); if that folder
cannot be written, a per-user folder under the temporary directory is used.
"""

from __future__ import annotations

import concurrent.futures
import glob
import hashlib
import os
import subprocess
import sys
import tempfile
import time

ARCH = "gfx950"
_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
LIB_NAME = f"libpae_{ARCH}.so"
# Packed float32 instructions are switched off for every kernel: scalar float
# code must compile to scalar float instructions.  So is the contraction of a multiply and an add
# into one fused instruction at the compiler's discretion: the same expression must round the same
# way in every kernel it is compiled into (a step's layers run either as separate kernels or as
# phases of one, and give the same bits); where a fused multiply-add is wanted it is written (fmaf).
HIPCC_FLAGS = [f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise BuildError("hipcc not found")


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def source_hash() -> str:
    digest = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    for path in sources() + sorted(glob.glob(os.path.join(CSRC, "*.h"))):
        digest.update(os.path.basename(path).encode())
        with open(path, "rb") as handle:
            digest.update(handle.read())
    return digest.hexdigest()[:16]


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = os.path.join(folder, f".probe{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return True
    except OSError:
        return False


def lib_dir() -> str:
    in_tree = os.path.join(_HERE, "_lib")
    if _writable(in_tree):
        return in_tree
    fallback = os.path.join(tempfile.gettempdir(), f"pae_build_{os.getuid()}")
    if _writable(fallback):
        return fallback
    raise BuildError(f"neither {in_tree} nor {fallback} can be written")


def _say(verbose: bool, text: str) -> None:
    if verbose:
        print(f"[pae build] {text}", file=sys.stderr, flush=True)


def _compile_one(hipcc: str, src: str, obj: str) -> str:
    cmd = [hipcc, *HIPCC_FLAGS, "-I", CSRC, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    return src


def build(verbose: bool = True) -> str:
    """Compile every source and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = lib_dir()
    obj_dir = os.path.join(out_dir, "obj")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise BuildError(f"no .hip sources under {CSRC}")
    started = time.time()
    _say(verbose, f"compiling {len(srcs)} HIP sources for {ARCH} into {out_dir}")
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]
    workers = max(1, min(len(srcs), (os.cpu_count() or 2), 8))
    with concurrent.futures.ThreadPoolExecutor(workers) as pool:
        futures = [pool.submit(_compile_one, hipcc, s, o) for s, o in zip(srcs, objs)]
        for done in concurrent.futures.as_completed(futures):
            _say(verbose, f"  compiled {os.path.basename(done.result())} ({time.time() - started:.0f}s)")
    lib = os.path.join(out_dir, LIB_NAME)
    tmp = lib + f".tmp{os.getpid()}"
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, lib)
    with open(os.path.join(out_dir, "source_hash.txt"), "w") as handle:
        handle.write(source_hash())
    _say(verbose, f"linked {LIB_NAME} ({time.time() - started:.0f}s)")
    return lib


def ensure_built(verbose: bool = True) -> str:
    """Path of a library built from the current sources, compiling if there is none."""
    out_dir = lib_dir()
    lib = os.path.join(out_dir, LIB_NAME)
    stamp = os.path.join(out_dir, "source_hash.txt")
    if os.path.exists(lib) and os.path.exists(stamp):
        with open(stamp) as handle:
            if handle.read().strip() == source_hash():
                return lib
        _say(verbose, "sources changed since the library was built")
    return build(verbose)
