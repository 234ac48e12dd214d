"""Build the in-tree HIP extensions on demand (a fresh checkout on a GPU
box has none).  Imports nothing that touches the GPU."""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys


def _built(repo: str, module: str) -> bool:
    return bool(glob.glob(os.path.join(repo, "polyrl_amd", module + ".*.so")))


def ensure_extension(repo: str, which: str = "seq") -> bool:
    """Compile ``which`` ("seq", "core" or "all") in-tree if its module is
    missing and a HIP compiler is present.  Build output goes to stderr.
    Returns True when the modules exist afterwards."""
    need = {"seq": ["_hip_seq"], "core": ["_hip"],
            "all": ["_hip", "_hip_seq"]}[which]
    if all(_built(repo, m) for m in need):
        return True
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        return False
    import fcntl
    env = dict(os.environ)
    env["PYTORCH_ROCM_ARCH"] = "gfx950"
    env["POLYRL_EXT"] = which
    env.setdefault("MAX_JOBS", "8")
    with open(os.path.join(repo, ".build.lock"), "w") as lock:
        fcntl.flock(lock, fcntl.LOCK_EX)     # one builder per checkout
        if not all(_built(repo, m) for m in need):
            subprocess.run([sys.executable, "setup.py", "build_ext",
                            "--inplace"], cwd=repo, env=env, check=True,
                           stdout=sys.stderr, stderr=sys.stderr)
    return all(_built(repo, m) for m in need)
