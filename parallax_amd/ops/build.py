"""On-demand in-tree build of the HIP extensions.

A fresh checkout holds sources only. Entry points that must work there (the
trace replayer) call ensure_extensions() with the extensions their model
needs; whatever is missing is compiled once with the checkout's setup.py
(hipcc, gfx950) and lands beside the sources, where later calls find it.
"""

from __future__ import annotations

import importlib
import os
import subprocess
import sys
from typing import Iterable, List

from ..utils.logging_config import get_logger

logger = get_logger("ops.build")

REPO_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def _importable(name: str) -> bool:
    try:
        importlib.import_module(f"parallax_amd.ops.{name}")
        return True
    except ImportError:
        return False


def ensure_extensions(names: Iterable[str]) -> List[str]:
    """Build the named extensions ('_C', '_mix') that cannot be imported yet.
    Returns the ones that were built. Build output goes to stderr."""
    missing = [n for n in names if not _importable(n)]
    if not missing:
        return []
    env = dict(os.environ)
    env["PARALLAX_EXT"] = ",".join(missing)
    env.setdefault("PYTORCH_ROCM_ARCH", "gfx950")
    env.setdefault("MAX_JOBS", str(min(16, os.cpu_count() or 4)))
    if "/opt/rocm/bin" not in env.get("PATH", ""):
        env["PATH"] = env.get("PATH", "") + os.pathsep + "/opt/rocm/bin"
    logger.info("building HIP extension(s) %s in %s", missing, REPO_ROOT)
    subprocess.run(
        [sys.executable, "setup.py", "build_ext", "--inplace"],
        cwd=REPO_ROOT, env=env, check=True, stdout=sys.stderr, stderr=sys.stderr,
    )
    importlib.invalidate_caches()
    still = [n for n in missing if not _importable(n)]
    if still:
        raise RuntimeError(f"extension(s) {still} did not build")
    return missing
