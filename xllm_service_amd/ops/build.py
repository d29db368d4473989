"""In-tree, on-demand build of a named HIP extension.

`ensure_built("_ops_hybrid")` compiles that one extension with setup.py
(XLLM_BUILD_EXT selects it) when its shared object is missing, so a worker
started from a source checkout compiles what its model needs and nothing
else. A lock file serialises concurrent first starts.
"""
from __future__ import annotations

import fcntl
import glob
import importlib
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(
    os.path.abspath(__file__))))
PKG = os.path.join(ROOT, "xllm_service_amd")


def is_built(name: str) -> bool:
    return bool(glob.glob(os.path.join(PKG, name + ".*.so")))


def ensure_built(name: str, log=sys.stderr) -> None:
    if is_built(name):
        return
    os.makedirs(os.path.join(ROOT, "build"), exist_ok=True)
    with open(os.path.join(ROOT, "build", f".{name}.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)
        if is_built(name):
            return
        print(f"[build] compiling {name} for gfx950 ...", file=log, flush=True)
        env = dict(os.environ, PYTORCH_ROCM_ARCH="gfx950",
                   XLLM_BUILD_EXT=name)
        env.setdefault("MAX_JOBS", "8")
        p = subprocess.run(
            [sys.executable, "setup.py", "build_ext", "--inplace"],
            cwd=ROOT, env=env, stdout=subprocess.PIPE,
            stderr=subprocess.STDOUT, text=True)
        if p.returncode != 0 or not is_built(name):
            print(p.stdout[-8000:], file=log, flush=True)
            raise RuntimeError(f"building {name} failed")
        print(f"[build] {name} ready", file=log, flush=True)
    importlib.invalidate_caches()
