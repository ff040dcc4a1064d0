"""Builds libpllm_hip.so (gfx950) in-tree with hipcc.

    python -m pocketllm_amd.build

One object per csrc/*.hip, compiled in parallel, linked into pocketllm_amd/libpllm_hip.so.
"""
from __future__ import annotations

import concurrent.futures
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ_DIR = PKG / "build"
LIB = PKG / "libpllm_hip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out, file=sys.stderr)


def build_library(verbose: bool = True, jobs: int = 8, incremental: bool = False) -> Path:
    """Compiles every csrc/*.hip and links the library.  incremental=True (python -m pocketllm_amd.build --incremental) skips
    sources whose object file is newer than the source and than every header."""
    OBJ_DIR.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    objs = [OBJ_DIR / (s.stem + ".o") for s in sources]
    newest_header = max(h.stat().st_mtime for h in [*CSRC.glob("*.h"), *CSRC.glob("*.inc"), *(PKG.parent / "include").glob("*.h")])
    todo = [(s, o) for s, o in zip(sources, objs)
            if not (incremental and o.exists() and o.stat().st_mtime > max(s.stat().st_mtime, newest_header))]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = [pool.submit(_run, ["hipcc", *HIPCC_FLAGS, "-c", str(s), "-o", str(o)]) for s, o in todo]
        for f in futs:
            f.result()
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *map(str, objs), "-o", str(LIB)])
    if verbose:
        print(f"built {LIB} from {len(sources)} sources")
    return LIB


if __name__ == "__main__":
    build_library(incremental="--incremental" in sys.argv[1:])
