"""Compile the HIP sources under `csrc/` into one shared library with hipcc.

The library is built in-tree (`mini_infer_amd/_lib/libmini_infer_hip.so`) so it
travels with the source folder; if that folder cannot be written, a per-user
folder under the temporary directory is used.  A stamp file next to the library
holds a hash of the sources and flags, which tells a fresh library from a stale one.
"""

from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path

CSRC_DIR = Path(__file__).resolve().parent.parent / "csrc"
IN_TREE_DIR = Path(__file__).resolve().parent.parent / "_lib"
LIB_NAME = "libmini_infer_hip.so"
OFFLOAD_ARCH = "gfx950"

# -packed-fp32-ops is switched off on purpose: some packed float32 forms have
# given wrong results on this hardware.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _say(message: str) -> None:
    print(f"[mini_infer_amd build] {message}", file=sys.stderr, flush=True)


def find_hipcc() -> str | None:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    return None


def source_files() -> list[Path]:
    return sorted(CSRC_DIR.glob("*.hip"))


def source_hash() -> str:
    digest = hashlib.sha256()
    for path in sorted(CSRC_DIR.glob("*")):
        if path.suffix in (".hip", ".h"):
            digest.update(path.name.encode())
            digest.update(path.read_bytes())
    digest.update(" ".join(HIPCC_FLAGS).encode())
    return digest.hexdigest()


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}"
        probe.write_text("x")
        probe.unlink()
        return True
    except OSError:
        return False


def candidate_dirs() -> list[Path]:
    fallback = Path(tempfile.gettempdir()) / f"mini_infer_amd-{os.getuid()}" / "_lib"
    return [IN_TREE_DIR, fallback]


def find_built(require_fresh: bool = False) -> Path | None:
    """Path of a built library, or None.  With `require_fresh`, its stamp must match."""
    wanted = source_hash() if require_fresh else None
    for folder in candidate_dirs():
        lib = folder / LIB_NAME
        if not lib.exists():
            continue
        if wanted is None:
            return lib
        stamp = folder / (LIB_NAME + ".stamp")
        if stamp.exists() and stamp.read_text().strip() == wanted:
            return lib
    return None


def _compile_one(hipcc: str, src: Path, obj: Path) -> tuple[Path, float, str]:
    started = time.time()
    done = subprocess.run(
        [hipcc, *HIPCC_FLAGS, "-c", str(src), "-o", str(obj)],
        capture_output=True,
        text=True,
        cwd=str(CSRC_DIR),
    )
    noise = "is not a recognized feature for this target"
    log = "\n".join(line for line in done.stderr.splitlines() if noise not in line)
    if done.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{log}")
    return src, time.time() - started, log


def build(force: bool = False, verbose: bool = True) -> Path:
    """Compile every `.hip` source and link the library; returns its path."""
    if not force:
        fresh = find_built(require_fresh=True)
        if fresh is not None:
            return fresh
    hipcc = find_hipcc()
    if hipcc is None:
        raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin)")
    out_dir = next((d for d in candidate_dirs() if _writable(d)), None)
    if out_dir is None:
        raise RuntimeError(f"no writable folder for the library among {candidate_dirs()}")
    sources = source_files()
    if verbose:
        _say(f"compiling {len(sources)} HIP sources for {OFFLOAD_ARCH} into {out_dir}")
    obj_dir = out_dir / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    started = time.time()
    objects: list[Path] = []
    workers = max(1, min(len(sources), os.cpu_count() or 1, 8))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        jobs = {}
        for src in sources:
            obj = obj_dir / (src.stem + ".o")
            objects.append(obj)
            jobs[pool.submit(_compile_one, hipcc, src, obj)] = src
        pending = set(jobs)
        while pending:
            finished, pending = concurrent.futures.wait(pending, timeout=15)
            for job in finished:
                src, seconds, log = job.result()
                if verbose:
                    _say(f"  {src.name}: {seconds:.1f} s")
                    if log.strip():
                        _say(log)
            if pending and verbose:
                names = ", ".join(sorted(jobs[j].name for j in pending))
                _say(f"  still compiling after {time.time() - started:.0f} s: {names}")
    lib = out_dir / LIB_NAME
    tmp_lib = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    link = subprocess.run(
        [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-o", str(tmp_lib)]
        + [str(o) for o in objects],
        capture_output=True,
        text=True,
    )
    if link.returncode != 0:
        raise RuntimeError(f"linking {LIB_NAME} failed:\n{link.stderr}")
    os.replace(tmp_lib, lib)
    (out_dir / (LIB_NAME + ".stamp")).write_text(source_hash() + "\n")
    if verbose:
        _say(f"built {lib} in {time.time() - started:.1f} s")
    return lib


if __name__ == "__main__":
    build(force="--force" in sys.argv)
