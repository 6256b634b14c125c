"""Where finished work is kept between runs, addressed by what produced it.

Everything lives under ``<session cache root>/persistent``: graph-search checkpoints under
``superopt/<k0k1>/<key>/checkpoint.json`` and saved kernels under ``kernels/<name>-<key16>/``
(the reference lays its cache out the same way, ``python/cleave/pipeline/cache.py:13-50``).  A
key is a SHA-256 over the inputs that determine the result *and* over this build of the back
end (templates, native library and the package's own Python sources: the recogniser and the
schedule policy decide what a checkpoint holds), so nothing saved by another build is picked up.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

LAYOUT_VERSION = 1
_build_id = None


def _fed(hasher, label: str, path: Path) -> None:
    hasher.update(label.encode() + b"\0" + path.read_bytes())


def build_id() -> str:
    """``<package version>+<12 hex>``: the hex digests every kernel template, the native
    library's source and every Python source of the package, name by name."""
    global _build_id
    if _build_id is not None:
        return _build_id
    from .. import __version__
    from ..codegen import TEMPLATE_DIR
    from ..runtime.shim import CSRC_DIR

    package = Path(__file__).resolve().parent.parent
    hasher = hashlib.sha256()
    for folder, pattern in ((TEMPLATE_DIR, "*.hip"), (CSRC_DIR, "*.cpp")):
        for source in sorted(folder.glob(pattern)):
            _fed(hasher, source.name, source)
    for source in sorted(package.rglob("*.py")):
        _fed(hasher, str(source.relative_to(package)), source)
    _build_id = f"{__version__}+{hasher.hexdigest()[:12]}"
    return _build_id


def digest(*parts) -> str:
    """Key of ``parts`` (anything JSON can write; other objects by their ``str``)."""
    canonical = json.dumps([LAYOUT_VERSION, build_id(), list(parts)], sort_keys=True, default=str,
                           separators=(",", ":"))
    return hashlib.sha256(canonical.encode()).hexdigest()


def root() -> Path:
    from ..core.session import current_session

    return Path(current_session().cache_root, "persistent")


def superopt_key(program, max_ops: int, split: tuple, concat_matmul: bool) -> str:
    return digest("superopt", program.fingerprint(), int(max_ops), sorted(split), bool(concat_matmul))


def checkpoint_path(key: str) -> Path:
    """The checkpoint file for ``key``; its directory is created."""
    home = root().joinpath("superopt", key[:2], key)
    home.mkdir(parents=True, exist_ok=True)
    return home / "checkpoint.json"


def kernel_dir(name: str, key: str) -> Path:
    return root().joinpath("kernels", name + "-" + key[:16])
