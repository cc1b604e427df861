"""Builds the gfx950 kernel library from ``kvcore_amd/csrc`` with hipcc.

``build()`` always compiles; ``ensure_built()`` compiles only when no library that
matches the sources is there.  The library is written next to this file when that
folder is writable, else under the temporary folder, so that a read-only checkout
still works.  Progress lines go to stderr while the compiler runs.
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
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
LIB_NAME = "libkvcore_hip.so"
ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # float32 division and square root rounded correctly (the compiler's default, said aloud:
    # the seeded random fill relies on it to give the bits of its host twin)
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Wno-unused-command-line-argument",
]


def _sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def source_hash() -> str:
    h = hashlib.sha256()
    for path in sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h"))):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(" ".join(HIPCC_FLAGS).encode())
    return h.hexdigest()[:16]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError(
        "kvcore_amd: hipcc was not found, so the gfx950 kernel library cannot be built; "
        "this engine has no other compute path"
    )


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe_{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def candidate_dirs() -> list[Path]:
    """Where the library may live: in the tree first, then a per-user temporary folder."""
    in_tree = Path(__file__).resolve().parent
    tmp = Path(tempfile.gettempdir()) / f"kvcore_amd_{os.getuid()}_{source_hash()}"
    return [in_tree, tmp]


def find_library() -> Path | None:
    """A built library whose recorded source hash matches the sources, if any."""
    want = source_hash()
    for folder in candidate_dirs():
        lib = folder / LIB_NAME
        stamp = folder / (LIB_NAME + ".srchash")
        if lib.is_file() and stamp.is_file() and stamp.read_text().strip() == want:
            return lib
    return None


def build(verbose: bool = True) -> Path:
    """Compile every source for gfx950 and link the shared library.  Always compiles."""
    hipcc = _hipcc()
    out_dir = next((d for d in candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError("kvcore_amd: no writable folder for the kernel library")
    obj_dir = out_dir / "_build" if out_dir.name != "ops" else out_dir.parent.parent / "_build" / "ops"
    if not _writable(obj_dir):
        obj_dir = Path(tempfile.mkdtemp(prefix="kvcore_amd_obj_"))
    sources = _sources()
    if not sources:
        raise RuntimeError(f"kvcore_amd: no .hip sources under {CSRC}")

    def log(msg: str) -> None:
        if verbose:
            print(f"[kvcore_amd build] {msg}", file=sys.stderr, flush=True)

    log(f"compiling {len(sources)} sources for {ARCH} with {hipcc}")
    done = threading.Event()

    def heartbeat() -> None:
        start = time.time()
        while not done.wait(15.0):
            log(f"still compiling ({time.time() - start:.0f} s)")

    beat = threading.Thread(target=heartbeat, daemon=True)
    beat.start()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *HIPCC_FLAGS, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src.name}:\n{proc.stderr[-4000:]}")
        log(f"compiled {src.name}")
        return obj

    try:
        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            objects = list(pool.map(compile_one, sources))
        lib = out_dir / LIB_NAME
        tmp_lib = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
        cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objects), "-o", str(tmp_lib)]
        proc = subprocess.run(cmd, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc link failed:\n{proc.stderr[-4000:]}")
        os.replace(tmp_lib, lib)
        (out_dir / (LIB_NAME + ".srchash")).write_text(source_hash() + "\n")
    finally:
        done.set()
    log(f"built {lib}")
    return lib


def ensure_built(verbose: bool = True) -> Path:
    lib = find_library()
    if lib is not None:
        return lib
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
