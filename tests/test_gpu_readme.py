"""The Python example of README.md runs as written."""

import re
from pathlib import Path

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_readme_example_runs(lib):
    text = (Path(__file__).resolve().parent.parent / "README.md").read_text()
    block = re.search(r"```python\n(.*?)```", text, flags=re.S).group(1)
    scope: dict = {}
    exec(compile(block, "README.md", "exec"), scope)
    torch.cuda.synchronize()
    ref = scope["A"].float() @ scope["B"].float()
    assert torch.allclose(scope["C"].float(), ref, rtol=1e-2, atol=1e-1)
    op, A2, B2 = scope["op"], scope["A2"], scope["B2"]
    op.check_faults()
    assert tuple(op.out.shape) == (8192, 4096)
    assert all(bool((x == 2.0).all()) for x in scope["xs"])
    for h in scope["heaps"] + scope["ranks"]:
        h.cleanup()
    for c in scope["ctxs"]:
        c.heap.cleanup()
