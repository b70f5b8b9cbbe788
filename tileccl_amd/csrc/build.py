"""Build ``libtileccl_hip.so`` in-tree for gfx950 with hipcc.

    python -m tileccl_amd.csrc.build

The library is two translation units (``tccl_api.hip``: entry points and the kernels for
row-major B; ``tccl_kmajor.hip``: the large-tile kernels for k-major B) compiled side by side
and linked.  It is built next to the Python package so that it travels with the source tree.
"""

from __future__ import annotations

import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE.parent / "libtileccl_hip.so"
SOURCES = [HERE / "tccl_api.hip", HERE / "tccl_kmajor.hip"]
HEADERS = [HERE / "tccl_device.h", HERE / "tccl_gemm.h", HERE / "tccl_gemm256.h", HERE / "tccl_kernels256.h", HERE / "tccl_comm.h",
           HERE / "tccl_staged.h", HERE / "tccl_probe.h", HERE.parent.parent / "include" / "tileccl_hip.h"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wno-comment",
    # hipcc -O3 must not form packed-fp32 instructions on this hardware pool.
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, cwd=HERE, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}\n{proc.stderr}")
    if verbose and proc.stderr:
        # The host pass reports the packed-fp32 feature as unknown; that is expected.
        print(proc.stderr, file=sys.stderr)


def build(verbose: bool = False, extra: list[str] | None = None) -> Path:
    """Compile unconditionally; raises ``RuntimeError`` with the compiler output on failure."""
    with tempfile.TemporaryDirectory(prefix="tccl_build_") as tmp:
        objects = [str(Path(tmp) / (src.stem + ".o")) for src in SOURCES]
        with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
            jobs = [
                pool.submit(_run, ["hipcc", *FLAGS, *(extra or []), "-c", str(src), "-o", obj], verbose)
                for src, obj in zip(SOURCES, objects)
            ]
            for job in jobs:
                job.result()
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", str(OUT)], verbose)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
