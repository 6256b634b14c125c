"""Cross-process GPU mutex and context warm-up (``python/cleave/runtime/gpu.py:15-82``).

Every run / validate / time of a candidate holds an exclusive ``flock`` keyed by the physical
GPU, so parallel candidate workers never overlap on the device and timings stay clean.  The
key is the device UUID reported by the native library (the reference shells out to
``nvidia-smi``), falling back to the visible-devices string.
"""

from __future__ import annotations

import contextlib
import fcntl
import os

from ..core.settings import Settings

_lock_path = None
_context_ready = False


def _gpu_lock_key() -> str:
    visible = os.environ.get("HIP_VISIBLE_DEVICES", os.environ.get("ROCR_VISIBLE_DEVICES"))
    fallback = (visible or "all").replace(",", "_")
    try:
        from . import shim

        if shim.available() and shim.device_count() > 0:
            uuid = shim.device_info(0).get("uuid")
            if uuid:
                return f"GPU-{uuid}"
    except Exception:  # noqa: BLE001 - the lock still works with the fallback key
        pass
    return fallback


def _create_parallel_env():
    """Resolve the lock file once per process."""
    global _lock_path
    if _lock_path is None:
        root = Settings.from_env().runtime_root
        os.makedirs(root, exist_ok=True)
        _lock_path = str(root / f"gpu_{_gpu_lock_key()}.lock")
    return _lock_path


def _ensure_gpu_context():
    """Create the HIP primary context through torch before the first module load."""
    global _context_ready
    if _context_ready:
        return
    try:
        import torch

        if torch.cuda.is_available():
            torch.cuda.init()
            torch.zeros(1, device="cuda")
            _context_ready = True
    except Exception:  # noqa: BLE001 - callers fail on their own first GPU call instead
        return


@contextlib.contextmanager
def _gpu_exec_guard():
    path = _create_parallel_env()
    _ensure_gpu_context()
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as handle:
        fcntl.flock(handle.fileno(), fcntl.LOCK_EX)
        try:
            yield
        finally:
            fcntl.flock(handle.fileno(), fcntl.LOCK_UN)
