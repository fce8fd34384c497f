"""The hardware and software record embedded in every measurement
(src/turboserve/hwinfo.py:160-193), for an AMD GPU: the device as torch reports it, the ROCm
and torch versions, and the checkout's git state."""

from __future__ import annotations

import os
import platform
import socket
import subprocess
import sys
from datetime import datetime, timezone
from pathlib import Path
from typing import Any

SCHEMA_VERSION = 1


def _run(cmd: list[str], cwd: Path | None = None) -> str | None:
    try:
        out = subprocess.run(cmd, cwd=cwd, capture_output=True, text=True, timeout=10)
    except (OSError, subprocess.SubprocessError):
        return None
    return out.stdout.strip() if out.returncode == 0 else None


def git_info(root: Path | None = None) -> dict[str, Any]:
    root = root or Path(__file__).resolve().parents[1]
    sha = _run(["git", "rev-parse", "HEAD"], cwd=root)
    if sha is None:
        return {"sha": None, "branch": None, "dirty": None}
    return {
        "sha": sha,
        "branch": _run(["git", "rev-parse", "--abbrev-ref", "HEAD"], cwd=root),
        "dirty": bool(_run(["git", "status", "--porcelain"], cwd=root)),
    }


def torch_info() -> dict[str, Any]:
    import torch

    info: dict[str, Any] = {
        "version": torch.__version__,
        "hip_version": getattr(torch.version, "hip", None),
        "gpu_available": torch.cuda.is_available(),
        "devices": [],
    }
    if torch.cuda.is_available():
        for index in range(torch.cuda.device_count()):
            props = torch.cuda.get_device_properties(index)
            info["devices"].append({
                "index": index,
                "name": props.name,
                "arch": getattr(props, "gcnArchName", None),
                "total_memory_bytes": props.total_memory,
                "compute_units": props.multi_processor_count,
            })
    return info


def collect() -> dict[str, Any]:
    from turboserve_amd import __version__

    torch_facts = torch_info()
    devices = torch_facts["devices"]
    return {
        "schema_version": SCHEMA_VERSION,
        "collected_at": datetime.now(timezone.utc).isoformat(),
        "host": {
            "hostname": socket.gethostname(),
            "platform": platform.platform(),
            "machine": platform.machine(),
            "cpu_count": os.cpu_count(),
        },
        "python": {"version": platform.python_version(), "executable": sys.executable},
        "gpu_name": devices[0]["name"] if devices else None,
        "rocm_version": _run(["cat", "/opt/rocm/.info/version"]),
        "torch": torch_facts,
        "git": git_info(),
        "package_version": __version__,
    }
