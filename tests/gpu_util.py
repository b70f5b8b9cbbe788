"""Helpers shared by the GPU parity tests: seeded CPU inputs copied into heap slices, so the
oracle (CPU) and the HIP path (GPU) see identical bits."""

from __future__ import annotations

import torch


def seeded(shape, seed: int, dtype=torch.float16, scale: float = 1.0) -> torch.Tensor:
    """fp32 normal samples from a CPU generator, scaled, then cast (the benchmark configurations' recipe)."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def into_heap(heap, cpu: torch.Tensor) -> torch.Tensor:
    t = heap.allocate_tensor(tuple(cpu.shape), cpu.dtype)
    t.copy_(cpu)
    return t


def bits(t: torch.Tensor) -> torch.Tensor:
    """Reinterpret 16-bit floats as int16 so comparisons are on bytes, not values."""
    return t.contiguous().view(torch.int16) if t.element_size() == 2 else t.contiguous().view(torch.int32)


def assert_gemm_close(got: torch.Tensor, ref32: torch.Tensor, rtol=1e-2, atol=1e-1, tight: float | None = None):
    """The reference's own tolerance (tests/test_gemm_allscatter_smoke.py:39-40), plus an
    optional tighter bound on the worst absolute error."""
    got32 = got.float().cpu()
    assert torch.allclose(got32, ref32, rtol=rtol, atol=atol), (got32 - ref32).abs().max()
    if tight is not None:
        assert (got32 - ref32).abs().max().item() <= tight
