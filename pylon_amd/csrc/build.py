"""Compile the HIP sources beside this file into one shared library for gfx950.

``python -m pylon_amd.csrc.build`` (or :func:`build`) runs ``hipcc`` once per source,
in parallel, and links ``libpylon_hip.so``.  The library is kept in ``_build/`` beside
the sources; when that folder cannot be written (a read-only checkout) it goes to a
per-user folder under the system's temporary directory instead.  A stamp with the hash
of the sources lies beside the library, so a library built from other sources is not
mistaken for a current one.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import List, Optional

SOURCE_DIR = Path(__file__).resolve().parent
LIB_NAME = "libpylon_hip.so"
ARCH = "gfx950"
# Packed-fp32 code generation is switched off for every kernel of this library.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# Per source: the prefill attention keeps its accumulators in ordinary vector registers
# (the softmax rescales them every block; in accumulation registers each touch costs two
# extra moves, and the kernel needs fewer registers in total this way).
EXTRA_FLAGS = {
    "attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def sources() -> List[Path]:
    return sorted(SOURCE_DIR.glob("*.hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    for path in sorted(list(SOURCE_DIR.glob("*.hip")) + list(SOURCE_DIR.glob("*.h"))):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    digest.update(repr(sorted(EXTRA_FLAGS.items())).encode())
    return digest.hexdigest()[:16]


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dirs() -> List[Path]:
    """Where a built library may lie, in order of preference."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [
        SOURCE_DIR / "_build",
        Path(tempfile.gettempdir()) / f"pylon_amd_build_{uid}",
    ]


def find_library(*, require_current: bool = True) -> Optional[Path]:
    want = source_hash()
    for folder in build_dirs():
        lib = folder / LIB_NAME
        stamp = folder / (LIB_NAME + ".hash")
        if not lib.is_file():
            continue
        if not require_current:
            return lib
        if stamp.is_file() and stamp.read_text().strip() == want:
            return lib
    return None


def hipcc_path() -> str:
    found = shutil.which("hipcc")
    if found:
        return found
    for candidate in ("/opt/rocm/bin/hipcc",):
        if os.path.exists(candidate):
            return candidate
    raise RuntimeError("hipcc was not found; the HIP kernels cannot be compiled")


def _say(text: str, quiet: bool) -> None:
    if not quiet:
        print(f"[pylon_amd build] {text}", file=sys.stderr, flush=True)


def build(*, quiet: bool = False, jobs: Optional[int] = None) -> Path:
    """Compile every source and link the library; returns its path."""
    folder = next((d for d in build_dirs() if _writable(d)), None)
    if folder is None:
        raise RuntimeError("no writable folder for the compiled kernels")
    hipcc = hipcc_path()
    srcs = sources()
    jobs = jobs or min(len(srcs), max(1, min(16, os.cpu_count() or 1)))
    env = dict(os.environ)
    # hipcc keeps temporary files under TMPDIR and a cache under HOME; give it places
    # that exist even for a user without a home directory.
    env.setdefault("TMPDIR", tempfile.gettempdir())
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = str(folder)
    started = time.time()
    _say(f"compiling {len(srcs)} HIP sources for {ARCH} into {folder}", quiet)

    def compile_one(src: Path) -> Path:
        obj = folder / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, *EXTRA_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
        proc = subprocess.run(cmd, env=env, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{proc.stdout}\n{proc.stderr}")
        _say(f"compiled {src.name} ({time.time() - started:.0f} s)", quiet)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(compile_one, srcs))
    lib_tmp = folder / (LIB_NAME + f".tmp{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(lib_tmp), *map(str, objects)]
    proc = subprocess.run(cmd, env=env, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(lib_tmp, folder / LIB_NAME)
    (folder / (LIB_NAME + ".hash")).write_text(source_hash() + "\n")
    for obj in objects:
        try:
            obj.unlink()
        except OSError:
            pass
    _say(f"built {folder / LIB_NAME} in {time.time() - started:.0f} s", quiet)
    return folder / LIB_NAME


def ensure_built(*, quiet: bool = False) -> Path:
    """The current library, compiling it first if there is none."""
    lib = find_library()
    if lib is not None:
        return lib
    return build(quiet=quiet)


if __name__ == "__main__":
    print(build())
