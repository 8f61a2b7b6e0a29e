"""In-tree build of the HIP extension on demand.

A fresh checkout has no _bee2bee_hip.so. Entry points that must work from
one (bin/trace_run) call ensure_built(): on a machine with a GPU and
without a loadable extension it runs `setup.py build_ext --inplace` once,
serialized across processes by a lock file, and leaves CPU-only machines
alone (they run the torch reference ops).
"""
from __future__ import annotations

import fcntl
import importlib
import importlib.util
import os
import subprocess
import sys

REPO = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
_EXT = "bee2bee_amd.ops._bee2bee_hip"


def _loadable() -> bool:
    try:
        importlib.import_module(_EXT)
        return True
    except Exception:  # noqa: BLE001 — absent or stale; rebuild decides
        sys.modules.pop(_EXT, None)
        return False


def _present() -> bool:
    try:
        return importlib.util.find_spec(_EXT) is not None
    except Exception:  # noqa: BLE001
        return False


def build(verbose: bool = False) -> None:
    env = dict(os.environ, PYTORCH_ROCM_ARCH="gfx950")
    env.setdefault("MAX_JOBS", str(min(16, os.cpu_count() or 4)))
    out = None if verbose else subprocess.PIPE
    r = subprocess.run([sys.executable, "setup.py", "build_ext", "--inplace"],
                       cwd=REPO, env=env, stdout=out, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        if r.stdout:
            sys.stderr.write(r.stdout.decode("utf-8", "replace")[-8000:])
        raise RuntimeError("building the HIP extension failed")
    importlib.invalidate_caches()


def ensure_built(force: bool = False) -> None:
    if not force:
        if _present():
            return
        import torch

        if not torch.cuda.is_available():
            return
    with open(os.path.join(REPO, ".build.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if force or not _present():
            build()
