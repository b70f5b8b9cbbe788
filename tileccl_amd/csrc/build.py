"""Build ``libtileccl_hip.so`` in-tree for gfx950 with hipcc.

    python -m tileccl_amd.csrc.build

The library is a single translation unit (``tccl_api.hip`` plus headers).  It is built
next to the Python package so that it travels with the source tree.
"""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE.parent / "libtileccl_hip.so"
SOURCES = [HERE / "tccl_api.hip"]
HEADERS = [HERE / "tccl_device.h", HERE / "tccl_gemm.h", HERE / "tccl_gemm256.h", HERE / "tccl_comm.h", HERE.parent.parent / "include" / "tileccl_hip.h"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Wno-comment",
    # hipcc -O3 must not form packed-fp32 instructions on this hardware pool.
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def build(verbose: bool = False, extra: list[str] | None = None) -> Path:
    """Compile unconditionally; raises ``RuntimeError`` with the compiler output on failure."""
    cmd = ["hipcc", *FLAGS, *(extra or []), *map(str, SOURCES), "-o", str(OUT)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{proc.stderr}")
    if verbose and proc.stderr:
        # The host pass reports the packed-fp32 feature as unknown; that is expected.
        print(proc.stderr, file=sys.stderr)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
