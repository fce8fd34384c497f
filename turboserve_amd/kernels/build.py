"""Compile the HIP sources under ``csrc/`` for gfx950 into shared libraries.

The kernels are plain ``extern "C"`` entry points taking device pointers and a stream, so the
build is ``hipcc`` and nothing else: no torch headers, seconds per file.  Libraries are built
in-tree (``turboserve_amd/kernels/_lib``) when the tree is writable, otherwise under a per-user
folder in the temporary directory; a stamp with the hash of the sources says whether a built
library is current.

The sources are grouped into modules, one library each, so that a run only compiles what it
uses: ``core`` holds the kernels of every run (both dtypes, incl. the whole 32-bit path),
``attn_d<N>`` the matrix-core attention kernels of bfloat16 serving for head size N.
"""

from __future__ import annotations

import concurrent.futures
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
IN_TREE = Path(__file__).resolve().parent / "_lib"

ARCH = "gfx950"

#: module name -> sources (relative to csrc/)
MODULES: dict[str, tuple[str, ...]] = {
    "core": (
        "elementwise.hip",
        "attention_generic.hip",
        "gemm_plain.hip",
        "gemm_skinny.hip",
        "gemm_tiled.hip",
        "gemm_wide.hip",
        "sampling.hip",
        "probe.hip",
    ),
}

#: Head sizes whose matrix-core attention module ``build_all`` compiles ahead of time: the
#: common ones and those of the test configurations.  Any other multiple of 16 up to 256 is
#: compiled when a model with that head size is first loaded.
PREBUILT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 256)


def attention_module(head_dim: int) -> str:
    """Name of the bfloat16 matrix-core attention module for one head size."""
    return f"attn_d{int(head_dim)}"


def module_spec(module: str) -> tuple[tuple[str, ...], tuple[str, ...]]:
    """``(sources, extra compiler flags)`` of a module; ``attn_d<N>`` modules are one source
    compiled for head size N."""
    if module in MODULES:
        return MODULES[module], ()
    if module.startswith("attn_d") and module[6:].isdigit():
        head_dim = int(module[6:])
        if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
            raise BuildError(f"the matrix-core attention kernels take head sizes 16..256 in steps of 16, not {head_dim}")
        return ("attention_mfma.hip",), (f"-DTS_HEAD_DIM={head_dim}",)
    raise BuildError(f"unknown kernel module {module!r}")


def all_modules() -> list[str]:
    return [*MODULES, *(attention_module(d) for d in PREBUILT_HEAD_DIMS)]

HIPCC_FLAGS = (
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


class BuildError(RuntimeError):
    """hipcc is missing or a source did not compile."""


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).is_file():
            return candidate
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def source_hash(module: str) -> str:
    sources, extra = module_spec(module)
    digest = hashlib.sha256()
    digest.update(" ".join((*HIPCC_FLAGS, *extra)).encode())
    headers = sorted([*CSRC.glob("*.hpp"), *CSRC.glob("*.h")])
    for path in [*headers, *(CSRC / name for name in sources)]:
        digest.update(path.name.encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()


def _writable(directory: Path) -> bool:
    try:
        directory.mkdir(parents=True, exist_ok=True)
        probe = directory / f".probe-{os.getpid()}-{threading.get_ident()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dir() -> Path:
    """Where libraries are written: ``$TURBOSERVE_AMD_BUILD_DIR``, the tree, or a temp folder."""
    override = os.environ.get("TURBOSERVE_AMD_BUILD_DIR")
    if override:
        path = Path(override)
        path.mkdir(parents=True, exist_ok=True)
        return path
    if _writable(IN_TREE):
        return IN_TREE
    fallback = Path(tempfile.gettempdir()) / f"turboserve_amd-{os.getuid()}"
    fallback.mkdir(parents=True, exist_ok=True)
    return fallback


def library_path(module: str, directory: Path | None = None) -> Path:
    return (directory or build_dir()) / f"libts_{module}.so"


def is_current(module: str, directory: Path | None = None) -> bool:
    lib = library_path(module, directory)
    stamp = lib.with_suffix(".stamp")
    return lib.is_file() and stamp.is_file() and stamp.read_text().strip() == source_hash(module)


def _say(message: str) -> None:
    print(f"[turboserve_amd build] {message}", file=sys.stderr, flush=True)


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        noise = "is not a recognized feature for this target"
        errors = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
        raise BuildError(f"{' '.join(cmd)}\nfailed with exit status {proc.returncode}:\n{errors}")


def build_module(module: str, *, directory: Path | None = None, verbose: bool = True) -> Path:
    """Compile one module from scratch and return the library's path."""
    source_names, extra_flags = module_spec(module)
    hipcc = find_hipcc()
    out_dir = directory or build_dir()
    out_dir.mkdir(parents=True, exist_ok=True)
    obj_dir = out_dir / f"obj_{module}"
    obj_dir.mkdir(exist_ok=True)
    sources = [CSRC / name for name in source_names]
    started = time.time()
    if verbose:
        _say(f"compiling module {module!r}: {len(sources)} sources for {ARCH} into {out_dir}")

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        _run([hipcc, *HIPCC_FLAGS, *extra_flags, "-I", str(CSRC), "-c", str(src), "-o", str(obj)])
        return obj

    objects: list[Path] = []
    workers = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "8")), 16))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        pending = {pool.submit(compile_one, src): src for src in sources}
        while pending:
            done, _ = concurrent.futures.wait(pending, timeout=15, return_when=concurrent.futures.FIRST_COMPLETED)
            for future in done:
                src = pending.pop(future)
                objects.append(future.result())
                if verbose:
                    _say(f"  {src.name} done ({len(objects)}/{len(sources)}, {time.time() - started:.0f}s)")
            if not done and verbose:
                _say(f"  still compiling {len(pending)} sources ({time.time() - started:.0f}s)")
    lib = library_path(module, out_dir)
    tmp = lib.with_suffix(f".tmp{os.getpid()}.so")
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, sorted(objects)), "-o", str(tmp)])
    os.replace(tmp, lib)
    lib.with_suffix(".stamp").write_text(source_hash(module))
    if verbose:
        _say(f"module {module!r} built in {time.time() - started:.0f}s: {lib}")
    return lib


def ensure_module(module: str, *, verbose: bool = True) -> Path:
    """Path of a current library of ``module``, compiling it first if none is there."""
    directory = build_dir()
    if is_current(module, directory):
        return library_path(module, directory)
    if directory != IN_TREE and is_current(module, IN_TREE):
        return library_path(module, IN_TREE)
    return build_module(module, directory=directory, verbose=verbose)


def build_all(*, verbose: bool = True) -> list[Path]:
    """Compile every module, whether or not a built library is there; modules are compiled
    side by side."""
    modules = all_modules()
    directory = build_dir()
    workers = max(1, min(len(modules), int(os.environ.get("MAX_JOBS", "8")), 16))
    with concurrent.futures.ThreadPoolExecutor(max_workers=workers) as pool:
        return list(pool.map(lambda module: build_module(module, directory=directory, verbose=verbose), modules))


if __name__ == "__main__":
    for built in build_all():
        print(built)
