"""Where the kernel sources live and where compiled code objects are cached."""
from __future__ import annotations

import hashlib
import os
import sys
import tempfile
from pathlib import Path

PACKAGE_NAME = "kermac_amd"
PACKAGE_VERSION = "0.1.0"


def get_package_name() -> str:
    return PACKAGE_NAME


def get_package_version() -> str:
    return PACKAGE_VERSION


def get_kernel_source_dir() -> Path:
    """Directory of the device headers compiled at run time."""
    return Path(__file__).resolve().parents[1] / "csrc" / "kernels"


def cache_root() -> Path:
    """``$KERMAC_AMD_CACHE_DIR`` or ``<user cache>/kermac_amd/<version>/<env id>/``.

    The environment id separates Python installations, like the reference's
    per-venv cache root (module_cache/paths.py:50-71).
    """
    override = os.environ.get("KERMAC_AMD_CACHE_DIR")
    if override:
        target = Path(override)
    else:
        base = Path(os.environ.get("XDG_CACHE_HOME") or Path.home() / ".cache")
        env_id = hashlib.sha256(sys.prefix.encode()).hexdigest()[:12]
        target = base / PACKAGE_NAME / PACKAGE_VERSION / env_id
    try:
        target.mkdir(parents=True, exist_ok=True)
        return target
    except OSError:
        return Path(tempfile.mkdtemp(prefix=f"{PACKAGE_NAME}-cache-"))
