"""The hardware and software record embedded in every measurement: which device, which ROCm
and torch, and which code.  The keys follow the reference's record
(src/turboserve/hwinfo.py:160-193) so that its readers find them; the facts are an AMD GPU's.

The code is named twice: by the checkout's git state where there is one, and by a digest of
the source files themselves, which also works in a copy of the tree without ``.git`` (a
measurement box).  ``TURBOSERVE_GIT_SHA`` in the environment stands in for the sha there.
"""

from __future__ import annotations

import hashlib
import os
import platform
import socket
import subprocess
import sys
from datetime import datetime, timezone
from pathlib import Path
from typing import Any

SCHEMA_VERSION = 1
PACKAGE_ROOT = Path(__file__).resolve().parent
#: Where a ROCm installation says which release it is.
ROCM_VERSION_FILES = ("/opt/rocm/.info/version", "/opt/rocm/.info/version-dev")


def _git(root: Path, *args: str) -> str | None:
    try:
        done = subprocess.run(["git", *args], cwd=root, capture_output=True, text=True, timeout=10)
    except (OSError, subprocess.SubprocessError):
        return None
    return done.stdout.strip() if done.returncode == 0 else None


def source_digest(root: Path | None = None) -> str:
    """SHA-256 over the package's source files (Python, HIP, headers) and ``bench.py`` beside
    it, by relative path and content: the same for every copy of the same code."""
    root = root or PACKAGE_ROOT
    digest = hashlib.sha256()
    files = sorted(p for p in root.rglob("*") if p.suffix in (".py", ".hip", ".hpp", ".h") and "_lib" not in p.parts)
    bench = root.parent / "bench.py"
    for path in [*files, *([bench] if bench.is_file() else [])]:
        digest.update(str(path.relative_to(root.parent)).encode())
        digest.update(path.read_bytes())
    return digest.hexdigest()


def git_info(root: Path | None = None) -> dict[str, Any]:
    """``sha``, ``branch``, ``dirty`` of the checkout (``None`` where there is none; the sha
    then comes from ``TURBOSERVE_GIT_SHA`` if set) and ``source_digest``."""
    root = root or PACKAGE_ROOT.parent
    sha = _git(root, "rev-parse", "HEAD")
    facts: dict[str, Any] = {"sha": sha or os.environ.get("TURBOSERVE_GIT_SHA") or None, "branch": None, "dirty": None}
    if sha is not None:
        facts["branch"] = _git(root, "rev-parse", "--abbrev-ref", "HEAD")
        facts["dirty"] = bool(_git(root, "status", "--porcelain"))
    facts["source_digest"] = source_digest()
    return facts


def rocm_version() -> str | None:
    for name in ROCM_VERSION_FILES:
        try:
            return Path(name).read_text(encoding="utf-8").strip() or None
        except OSError:
            continue
    return None


def torch_info() -> dict[str, Any]:
    import torch

    devices = []
    if torch.cuda.is_available():
        for index in range(torch.cuda.device_count()):
            props = torch.cuda.get_device_properties(index)
            devices.append({
                "index": index, "name": props.name, "arch": getattr(props, "gcnArchName", None),
                "total_memory_bytes": props.total_memory, "compute_units": props.multi_processor_count,
            })
    return {"version": torch.__version__, "hip_version": getattr(torch.version, "hip", None),
            "gpu_available": bool(devices), "devices": devices}


def collect() -> dict[str, Any]:
    from turboserve_amd import __version__

    record: dict[str, Any] = {"schema_version": SCHEMA_VERSION, "collected_at": datetime.now(timezone.utc).isoformat()}
    record["host"] = {"hostname": socket.gethostname(), "platform": platform.platform(), "machine": platform.machine(),
                      "cpu_count": os.cpu_count()}
    record["python"] = {"version": platform.python_version(), "executable": sys.executable}
    record["torch"] = torch_info()
    record["gpu_name"] = record["torch"]["devices"][0]["name"] if record["torch"]["devices"] else None
    record["rocm_version"] = rocm_version()
    record["git"] = git_info()
    record["package_version"] = __version__
    return record


def brief(record: dict[str, Any] | None = None) -> dict[str, Any]:
    """The few flat facts a measurement's JSON line carries (nested records are lost there)."""
    record = record or collect()
    devices = record["torch"]["devices"]
    return {
        "gpu": record["gpu_name"], "arch": devices[0]["arch"] if devices else None,
        "torch": record["torch"]["version"], "hip": record["torch"]["hip_version"], "rocm": record["rocm_version"],
        "git": (record["git"]["sha"] or "")[:12], "source": record["git"]["source_digest"][:12],
    }
