"""Build the in-tree HIP extensions on demand.

`setup.py build_ext --inplace` builds everything; `ensure_built([...])`
builds only the named extensions when their shared objects are missing (a
fresh checkout), so a first run compiles what it needs and no more."""

from __future__ import annotations

import glob
import importlib
import os
import subprocess
import sys
from typing import Iterable

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def is_built(name: str) -> bool:
    return bool(glob.glob(os.path.join(_ROOT, "sutro_amd", name + ".*.so")))


def ensure_built(names: Iterable[str]) -> None:
    missing = [n for n in names if not is_built(n)]
    if not missing:
        return
    env = dict(os.environ)
    env["PYTORCH_ROCM_ARCH"] = "gfx950"
    env["SUTRO_AMD_EXTENSIONS"] = ",".join(missing)
    subprocess.run([sys.executable, "setup.py", "-q", "build_ext", "--inplace"],
                   cwd=_ROOT, env=env, check=True, stdout=sys.stderr)
    importlib.invalidate_caches()
