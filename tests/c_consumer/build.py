"""Compile ``allgather_from_c.c`` with gcc against the public header and the built library.

``python tests/c_consumer/build.py`` or ``build()``; the binary lands beside the source and finds
the library through a path relative to itself, so the tree can be moved as a whole.
"""

from __future__ import annotations

import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
SOURCE = HERE / "allgather_from_c.c"
BINARY = HERE / "allgather_from_c"
ROCM = Path("/opt/rocm")


def command(output: Path = BINARY) -> list[str]:
    return [
        "gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-Werror",
        f"-I{ROCM / 'include'}", f"-I{ROOT / 'include'}", str(SOURCE), "-o", str(output),
        f"-L{ROOT / 'tileccl_amd'}", "-ltileccl_hip", f"-L{ROCM / 'lib'}", "-lamdhip64",
        "-Wl,-rpath,$ORIGIN/../../tileccl_amd", f"-Wl,-rpath,{ROCM / 'lib'}",
    ]  # fmt: skip


def build(output: Path = BINARY) -> Path:
    subprocess.run(command(output), check=True, capture_output=True, text=True)
    return output


if __name__ == "__main__":
    print(build())
