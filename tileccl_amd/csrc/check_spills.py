"""Guard against register spills inside the K loops of the large-tile kernels.

``python -m tileccl_amd.csrc.check_spills`` compiles ``tccl_api.hip`` and ``tccl_kmajor.hip`` to
assembly (about two minutes) and, for every ``gemm256_kernel`` / ``fused256_kernel``
instantiation, counts the scratch-memory instructions that lie between the kernel's first and last
MFMA, i.e. inside its K loops.  A register that the compiler keeps in scratch memory there is
reloaded through the same queue as the operand loads, so the reload waits for all of them: a
handful of such reloads per K step has cost the fused launches more than a third of their time.
The fused kernels run at the register limit; changes to the K step or to the background transfer
should be followed by this check.  Exit status 1 if any count exceeds ``--allow`` (default: the
two reloads of the rarely taken block-change path of the all-gather kernels).

The count over the whole kernel is printed as well.  In an all-gather kernel the accesses outside
the K loops sit on rarely taken paths; in a reduce-scatter kernel (third template argument true)
they sit in the reduction phases, between loads of the addends, and are marked: 32 of them made
the 8192 x 4096 x 2048 reduce-scatter 4 % slower.
"""

from __future__ import annotations

import argparse
import re
import subprocess
import sys
import tempfile
from pathlib import Path

from tileccl_amd.csrc.build import FLAGS, HERE, SOURCES


def kernels(asm: str):
    """(name, vgprs, scratch instructions in the K loops, scratch instructions in all) per large-tile kernel."""
    counts = dict(re.findall(r"\.name:\s+(\S+)\n(?:.*\n)*?\s+\.vgpr_count:\s+(\d+)", asm))
    for match in re.finditer(r"^(_ZN4tccl1[45](?:gemm|fused)256_kernel\w*):", asm, flags=re.M):
        name = match.group(1)
        body = asm[match.end(): asm.index(".Lfunc_end", match.end())].split("\n")
        mfma = [i for i, line in enumerate(body) if "v_mfma" in line]
        scratch = [i for i, line in enumerate(body) if "scratch_" in line]
        inside = [i for i in scratch if mfma and mfma[0] < i < mfma[-1]]
        yield name, int(counts.get(name, 0)), len(inside), len(scratch)


def is_reduce(name: str) -> bool:
    """Whether the mangled name is a fused kernel instantiated for reduce-scatter (first bool argument)."""
    match = re.search(r"fused256_kernelI.*?Lb([01])E", name)
    return bool(match) and match.group(1) == "1"


def report(asm: str, allow: int) -> int:
    worst = 0
    for name, vgprs, inside, total in kernels(asm):
        worst = max(worst, inside)
        flag = "  <-- spills in the K loop" if inside > allow else ""
        if not flag and total and is_reduce(name):
            flag = "  (scratch accesses in a reduce-scatter kernel)"
        print(f"{name}: {vgprs} VGPRs, scratch instructions {inside} in K loops / {total} in all{flag}")
    return worst


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--allow", type=int, default=2, help="scratch instructions tolerated inside a kernel's K loops")
    ap.add_argument("asm", nargs="*", help="check these assembly files instead of compiling the sources")
    args = ap.parse_args()
    worst = 0
    for path in args.asm:
        worst = max(worst, report(Path(path).read_text(), args.allow))
    if args.asm:
        return 1 if worst > args.allow else 0
    with tempfile.TemporaryDirectory(prefix="tccl_spills_") as tmp:
        for src in SOURCES:
            out = Path(tmp) / (src.stem + ".s")
            cmd = ["hipcc", *FLAGS, "-S", "--cuda-device-only", str(src), "-o", str(out)]
            subprocess.run(cmd, check=True, capture_output=True, text=True, cwd=HERE)
            worst = max(worst, report(out.read_text(), args.allow))
    return 1 if worst > args.allow else 0


if __name__ == "__main__":
    sys.exit(main())
