"""Content-addressed cache paths under ``current_session().cache_root / "persistent"``
(``python/cleave/pipeline/cache.py:13-50``)."""

from __future__ import annotations

import functools
import hashlib
import json
from pathlib import Path

SCHEMA = 1


@functools.lru_cache(maxsize=None)
def build_id() -> str:
    """Package version plus a digest of the kernel templates and the native library source:
    a cached kernel is only reused by the code that produced it."""
    from .. import __version__
    from ..codegen import TEMPLATE_DIR
    from ..runtime.shim import CSRC_DIR

    h = hashlib.sha256()
    for path in sorted([*TEMPLATE_DIR.glob("*.hip"), *CSRC_DIR.glob("*.cpp")]):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    return f"{__version__}+{h.hexdigest()[:12]}"


def digest(*parts) -> str:
    blob = json.dumps([SCHEMA, build_id(), *parts], sort_keys=True, default=str, separators=(",", ":"))
    return hashlib.sha256(blob.encode()).hexdigest()


def root() -> Path:
    from ..core.session import current_session

    return current_session().cache_root / "persistent"


def superopt_key(program, max_ops: int, split: tuple, concat_matmul: bool) -> str:
    return digest("superopt", program.fingerprint(), int(max_ops), sorted(split), bool(concat_matmul))


def checkpoint_path(key: str) -> Path:
    d = root() / "superopt" / key[:2] / key
    d.mkdir(parents=True, exist_ok=True)
    return d / "checkpoint.json"


def kernel_dir(name: str, key: str) -> Path:
    return root() / "kernels" / f"{name}-{key[:16]}"
