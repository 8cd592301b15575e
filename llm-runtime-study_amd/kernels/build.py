"""Compiles the HIP sources under csrc/ into one shared library for gfx950.

The library is kept inside the package folder next to a file holding the hash of the
sources it was built from.  `ensure_built()` compiles only when no library matching
the sources exists, printing a line as each file starts and finishes, so that a first
call in a fresh checkout shows progress.  Files are compiled in parallel.  A checkout
that the user cannot write to gets its library in a folder of the user's own under the
temporary directory, named by the hash of the sources.
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

PACKAGE_DIR = Path(__file__).resolve().parent.parent
SOURCE_DIR = PACKAGE_DIR / "csrc"
LIBRARY = Path(__file__).resolve().parent / "liblrs_kernels.so"
HASH_FILE = LIBRARY.with_suffix(".so.hash")
ARCH = "gfx950"
# -packed-fp32-ops: keep the compiler from forming packed float32 instructions.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
FLAGS = [f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wno-unused-command-line-argument"] + DEVICE_FLAGS
# the vendor's matrix library, for bfloat16 products of many rows (csrc/library_gemm.hip)
ROCM_LIB = Path(os.environ.get("ROCM_PATH", "/opt/rocm")) / "lib"
LINK_FLAGS = [f"-L{ROCM_LIB}", "-lhipblaslt", f"-Wl,-rpath,{ROCM_LIB}"]


class BuildError(RuntimeError):
    """Raised when the kernel library cannot be compiled."""


def sources() -> list[Path]:
    return sorted(SOURCE_DIR.glob("*.hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    for path in sorted(SOURCE_DIR.glob("*.hip")) + sorted(SOURCE_DIR.glob("*.h")) + sorted(SOURCE_DIR.glob("*.inc")):
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    digest.update(" ".join(FLAGS + LINK_FLAGS).encode())
    return digest.hexdigest()


def is_current() -> bool:
    return LIBRARY.is_file() and HASH_FILE.is_file() and HASH_FILE.read_text().strip() == source_hash()


def _outside_the_checkout() -> Path:
    """Where the library goes when the checkout cannot be written to."""
    return Path(tempfile.gettempdir()) / f"lrs_kernels_{os.getuid()}_{source_hash()[:16]}"


def _writable(folder: Path) -> bool:
    return os.access(folder, os.W_OK | os.X_OK)


def _hipcc() -> str:
    found = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)
    if found is None:
        raise BuildError("hipcc was not found: the kernel library cannot be built")
    return found


def _say(message: str) -> None:
    print(f"[kernels] {message}", file=sys.stderr, flush=True)


def _compile_one(hipcc: str, src: Path, obj: Path) -> None:
    _say(f"compiling {src.name} ...")
    started = time.time()
    proc = subprocess.run([hipcc, *FLAGS, "-c", str(src), "-o", str(obj)], capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed on {src.name}:\n{proc.stderr}")
    _say(f"compiled {src.name} in {time.time() - started:.1f} s")


def build(force: bool = True) -> Path:
    """Compile every source and link the library; returns its path."""
    if not force and is_current():
        return LIBRARY
    library, hash_file, build_dir = LIBRARY, HASH_FILE, SOURCE_DIR / "_build"
    if not (_writable(LIBRARY.parent) and _writable(SOURCE_DIR)):
        folder = _outside_the_checkout()
        library, hash_file, build_dir = folder / LIBRARY.name, folder / HASH_FILE.name, folder / "_build"
        if not force and library.is_file() and hash_file.is_file() and hash_file.read_text().strip() == source_hash():
            return library
        folder.mkdir(mode=0o700, exist_ok=True)
        _say(f"{LIBRARY.parent} is not writable: building in {folder}")
    hipcc = _hipcc()
    build_dir.mkdir(exist_ok=True)
    srcs = sources()
    if not srcs:
        raise BuildError(f"no HIP sources under {SOURCE_DIR}")
    objects = [build_dir / (src.stem + ".o") for src in srcs]
    started = time.time()
    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        for future in [pool.submit(_compile_one, hipcc, s, o) for s, o in zip(srcs, objects)]:
            future.result()
    tmp = library.with_suffix(f".so.tmp{os.getpid()}")
    proc = subprocess.run(
        [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objects), *LINK_FLAGS, "-o", str(tmp)],
        capture_output=True, text=True,
    )
    if proc.returncode != 0:
        raise BuildError(f"linking the kernel library failed:\n{proc.stderr}")
    os.replace(tmp, library)
    hash_file.write_text(source_hash() + "\n")
    _say(f"built {library.name} in {time.time() - started:.1f} s")
    return library


def ensure_built() -> Path:
    """Return the library, compiling it first if none matches the sources."""
    return build(force=False)


if __name__ == "__main__":
    build(force=True)
