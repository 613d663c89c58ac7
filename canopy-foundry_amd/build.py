"""Builds libcf_fp8.so (hand-written HIP for gfx950) in-tree with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB = Path(os.environ.get("CF_LIB_OUT", PKG / "libcf_fp8.so"))

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", f"-I{INCLUDE}", f"-I{CSRC}",
]


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, obj: Path, extra: list[str]) -> None:
    cmd = [HIPCC, *FLAGS, *extra, "-c", str(src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build(force: bool = True, extra: list[str] | None = None, jobs: int = 8) -> Path:
    """Compiles every .hip under csrc/ and links libcf_fp8.so next to this file."""
    extra = list(extra or [])
    objdir = Path(os.environ.get("CF_OBJ_DIR", CSRC / "build"))
    objdir.mkdir(exist_ok=True, parents=True)
    srcs = sources()
    hdrs = list(CSRC.glob("*.hpp")) + list(INCLUDE.glob("*.h"))
    newest_hdr = max((h.stat().st_mtime for h in hdrs), default=0.0)
    todo = []
    for s in srcs:
        o = objdir / (s.stem + ".o")
        if force or not o.exists() or o.stat().st_mtime < max(s.stat().st_mtime, newest_hdr):
            todo.append((s, o))
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as ex:
        list(ex.map(lambda so: _compile(so[0], so[1], extra), todo))
    objs = [str(objdir / (s.stem + ".o")) for s in srcs]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *objs]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
