"""Marshalling between torch tensors and the C ABI descriptors.

Everything here is host bookkeeping: it validates what the kernels assume (contiguity,
dtypes, device) and hands raw device pointers down.  The launches go to torch's current
stream, like the reference's Triton launches do.
"""

from __future__ import annotations

import ctypes as C
import sys
from dataclasses import dataclass, field

import torch

from tileccl_amd import _lib

_DTYPE_CODES = {
    torch.float16: _lib.F16,
    torch.bfloat16: _lib.BF16,
    torch.float32: _lib.F32,
}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPE_CODES[torch.float8_e4m3fn] = _lib.F8E4M3

VARIANTS = {"s0": _lib.S0_BULK, "s1": _lib.S1_TILE, "s2": _lib.S2_TILEGROUP}
DEFAULT_SPIN_LIMIT_NS = 2_000_000_000


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype} is not supported by the HIP kernels") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr() -> int:
    """torch's current stream on the heap's device as a ``hipStream_t`` value.  The raw accessor
    costs well under a microsecond; building a ``torch.cuda.Stream`` object costs ~9 us, a fifth
    of a c1-sized launch."""
    if _raw_stream is not None:
        return int(_raw_stream(0))  # every emulated rank lives on device 0
    return int(torch.cuda.current_stream().cuda_stream)


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else int(t.data_ptr())


def _row_major(t: torch.Tensor, name: str) -> int:
    """Leading dimension of a 2-D tensor whose rows are contiguous."""
    if t.ndim != 2:
        raise ValueError(f"{name} must be 2-D, got {t.ndim}-D")
    if t.shape[1] > 1 and t.stride(1) != 1:
        raise ValueError(
            f"{name} must have contiguous rows (stride(1) == 1), got strides {tuple(t.stride())}; "
            "call .contiguous() first"
        )
    return int(t.stride(0)) if t.shape[0] > 1 else int(t.shape[1])


def _vector_elems(t: torch.Tensor) -> int:
    return 16 // t.element_size()


def _rows_vectorised(t: torch.Tensor, ld: int) -> bool:
    """Rows of pitch ``ld`` start on 16-byte boundaries (what the kernels' row vectors need)."""
    return t.data_ptr() % 16 == 0 and ld % _vector_elems(t) == 0


def _b_layout(B: torch.Tensor) -> tuple[int, int] | None:
    """(ldb, flag bits) of a B operand the kernels read in place: rows contiguous, or the ``.t()``
    view of a tensor whose rows are contiguous (k-major: the layout of a linear layer's weight).
    ``None`` for every other layout; the reference's kernels take any strides
    (``/root/reference/tileccl/kernels/gemm.py:139-151``) and these are the two forms with 16-byte
    vector access."""
    K, N = B.shape
    if N == 1 or B.stride(1) == 1:
        ld = int(B.stride(0)) if K > 1 else int(N)
        return (ld, 0) if ld >= N and _rows_vectorised(B, ld) else None
    if K == 1 or B.stride(0) == 1:
        ld = int(B.stride(1)) if N > 1 else int(K)
        return (ld, _lib.GEMM_B_KMAJOR) if ld >= K and _rows_vectorised(B, ld) else None
    return None


_PACKED: dict[tuple, torch.Tensor] = {}
_PACKED_LIMIT = 8


def pack_operand(t: torch.Tensor, rows: int, cols: int, role: str) -> torch.Tensor:
    """``t`` as a dense ``rows x cols`` matrix (zero beyond ``t``'s own shape), written by one
    ``tccl_pack_matrix`` launch on the current stream.  The buffer is kept per (role, shape, dtype,
    stream) and reused by the next call with that key, which the stream orders behind this one's GEMM,
    unless a descriptor that has not been dropped yet still points at it."""
    key = (role, rows, cols, t.dtype, t.device, stream_ptr())
    out = _PACKED.pop(key, None)
    if out is not None and sys.getrefcount(out) > 2:  # this name and the call's argument
        out = None
    if out is None:
        while len(_PACKED) >= _PACKED_LIMIT:
            _PACKED.pop(next(iter(_PACKED)))
        out = torch.empty((rows, cols), dtype=t.dtype, device=t.device)
    _PACKED[key] = out  # most recently used last
    rc = _lib.load().tccl_pack_matrix(
        ptr(t), int(t.stride(0)), int(t.stride(1)), int(t.shape[0]), int(t.shape[1]),
        ptr(out), cols, rows, cols, t.element_size(), stream_ptr(),
    )
    _lib.check(rc, f"tccl_pack_matrix[{role}]")
    return out


def gemm_operands(A: torch.Tensor, B: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, int, int, int, int]:
    """(A, B, K, lda, ldb, flag bits) as the kernels read them.  An operand they can address in place
    (16-byte row vectors: A with contiguous rows, B with contiguous rows or columns, K a whole number
    of vectors) is passed through; any other layout the reference's pointer arithmetic accepts
    (``/root/reference/tileccl/kernels/gemm.py:63-66,139-151``: a transposed A, strided slices, odd K)
    is packed into a dense buffer first, K zero-filled up to the next whole vector, which adds exact zeros
    to every dot product."""
    for name, t in (("A", A), ("B", B)):
        if t.ndim != 2:
            raise ValueError(f"{name} must be 2-D, got {t.ndim}-D")
        if any(s < 0 for s in t.stride()):
            raise ValueError(f"{name} has negative strides {tuple(t.stride())}")
    M, K = A.shape
    vec = _vector_elems(A)
    k_pad = (K + vec - 1) // vec * vec
    lda = int(A.stride(0)) if M > 1 else int(K)
    if k_pad != K or (K > 1 and A.stride(1) != 1) or lda < K or not _rows_vectorised(A, lda):
        A, lda = pack_operand(A, M, k_pad, "A"), k_pad
    layout = _b_layout(B) if k_pad == K else None
    if layout is None:
        N = B.shape[1]
        B, layout = pack_operand(B, k_pad, N, "B"), (N, 0)
    return A, B, k_pad, lda, layout[0], layout[1]


def gemm_desc(
    A: torch.Tensor,
    B: torch.Tensor,
    C_out: torch.Tensor,
    *,
    block_m: int = 128,
    block_n: int = 128,
    group_m: int = 8,
    alpha: float = 1.0,
    num_wgs: int = 0,
    macro_tile: int = 0,
    flags: int = 0,
    column_shards: int = 0,
) -> _lib.GemmDesc:
    if not (A.is_cuda and B.is_cuda and C_out.is_cuda):
        raise ValueError("GEMM operands must be device tensors")
    if A.dtype != B.dtype:
        raise ValueError(f"A and B must share a dtype, got {A.dtype} and {B.dtype}")
    M, K = A.shape
    K2, N = B.shape
    if K2 != K:
        raise ValueError(f"B.shape[0] must equal A.shape[1]: got {K2} vs {K}")
    if column_shards > 1:  # C stacks the column blocks of A @ B as row blocks
        if N % column_shards:
            raise ValueError(f"B.shape[1]={N} must be divisible by column_shards={column_shards}")
        M, N = M * column_shards, N // column_shards
    if tuple(C_out.shape) != (M, N):
        raise ValueError(f"C shape mismatch: expected ({M}, {N}), got {tuple(C_out.shape)}")
    A, B, K, lda, ldb, b_flags = gemm_operands(A, B)
    d = _lib.GemmDesc()
    d.operands = (A, B)  # a packed operand lives as long as the descriptor
    d.A, d.B, d.C = ptr(A), ptr(B), ptr(C_out)
    d.M, d.N, d.K = int(M), int(N), int(K)
    d.lda, d.ldb, d.ldc = lda, ldb, _row_major(C_out, "C")
    d.in_dtype, d.out_dtype = dtype_code(A.dtype), dtype_code(C_out.dtype)
    d.alpha = float(alpha)
    d.block_m, d.block_n, d.group_m = int(block_m), int(block_n), int(group_m)
    d.num_wgs = int(num_wgs)
    d.macro_tile = int(macro_tile)
    d.flags = int(flags) | b_flags
    d.column_shards = int(column_shards)
    return d


def heap_view(heap_bases: torch.Tensor, rank: int, world_size: int) -> _lib.HeapView:
    v = _lib.HeapView()
    v.heap_bases = ptr(heap_bases)
    v.rank, v.world_size = int(rank), int(world_size)
    return v


def transport_desc(directions: int, copy_elems: int, reduce_elems: int | None, num_comm_wgs: int) -> _lib.TransportDesc:
    t = _lib.TransportDesc()
    t.directions = int(directions)
    t.copy_elems = int(copy_elems)
    t.reduce_elems = int(reduce_elems or 0)
    t.num_comm_wgs = int(num_comm_wgs)
    return t


@dataclass
class DevicePlan:
    """Device-resident copy of a ``TileGroupPlan``'s vectors (uploaded once per plan)."""

    n_groups: int
    group_table: torch.Tensor
    row_starts: torch.Tensor
    row_ends: torch.Tensor
    tile_counts: torch.Tensor

    @classmethod
    def upload(cls, plan, device: str = "cuda:0") -> "DevicePlan":
        def dev(values) -> torch.Tensor:
            return torch.tensor(list(values), dtype=torch.int32, device=device)

        return cls(
            n_groups=plan.n_groups,
            group_table=plan.group_table.to(device=device, dtype=torch.int32).contiguous(),
            row_starts=dev(plan.row_starts()),
            row_ends=dev(plan.row_ends()),
            tile_counts=dev(plan.tile_counts()),
        )


@dataclass
class SyncWords:
    """Signal words of one fused operation plus the launch epoch.

    Counters grow monotonically: TileGroup launch ``e`` (1-based) treats group ``g`` as ready
    at ``counter[g] >= e * tile_counts[g]``, and tile-by-tile launch ``e`` stores ``e`` into
    ``locks[tile]`` and treats a tile as ready at ``locks[tile] >= e``, so repeated launches
    need no reset kernel and a flag of an earlier launch is never mistaken for this one's.
    The two kinds of launch count separately (``epoch`` / ``lock_epoch``): each numbers the
    launches that wrote its own words.  Ranks that wait on each other's words must have issued
    the same number of launches.  ``reset()`` zeroes the words and restarts both numbers,
    which is also what happens automatically before the 32-bit words could overflow.

    A launch recorded into a HIP graph replays with the arguments it was recorded with, so
    its epoch cannot advance.  A TileGroup launch issued while the stream is capturing is
    therefore preceded by fill kernels that clear the counters (recorded with it; never a
    memset node) and runs as epoch 1; from then on every launch of these words does the
    same, captured or not, so replays and eager launches can alternate freely.
    """

    locks: torch.Tensor | None = None
    counter: torch.Tensor | None = None
    barrier: torch.Tensor | None = None
    plan: DevicePlan | None = None
    host_plan: object | None = None  # the TileGroupPlan `plan` was uploaded from
    trace_comm_counter: torch.Tensor | None = None
    trace_start_clock: torch.Tensor | None = None
    trace_ready_clock: torch.Tensor | None = None
    trace_done_clock: torch.Tensor | None = None
    fault: torch.Tensor = field(default_factory=lambda: torch.zeros(1, dtype=torch.int64, device="cuda:0"))
    epoch: int = 0
    lock_epoch: int = 0
    spin_limit_ns: int = DEFAULT_SPIN_LIMIT_NS
    max_tasks_per_tile: int = 1 << 16
    clear_every_launch: bool = False  # set by the first launch recorded into a graph

    def reset(self) -> None:
        for t in (self.locks, self.counter, self.barrier, self.trace_comm_counter, self.trace_start_clock,
                  self.trace_ready_clock, self.trace_done_clock, self.fault):
            if t is not None:
                t.zero_()
        self.epoch = 0
        self.lock_epoch = 0

    def next_epoch(self, variant: str = "s2") -> int:
        """Number the launch about to be issued: ``"s2"`` advances ``epoch``, ``"s1"`` ``lock_epoch``."""
        tile_by_tile = variant == "s1"
        if self.clear_every_launch or torch.cuda.is_current_stream_capturing():
            self.clear_every_launch = True
            for t in (self.locks, self.counter, self.barrier):
                if t is not None:
                    t.zero_()
            self.epoch = self.lock_epoch = 0
        elif max(self.epoch, self.lock_epoch) >= (1 << 30) // self.max_tasks_per_tile:
            torch.cuda.current_stream().synchronize()
            self.reset()
        if tile_by_tile:
            self.lock_epoch += 1
            return self.lock_epoch
        self.epoch += 1
        return self.epoch

    def desc(self, variant: str = "s2") -> _lib.SyncDesc:
        s = _lib.SyncDesc()
        s.locks = ptr(self.locks)
        s.counter = ptr(self.counter)
        s.barrier = ptr(self.barrier)
        if self.plan is not None:
            s.group_table = ptr(self.plan.group_table)
            s.row_starts = ptr(self.plan.row_starts)
            s.row_ends = ptr(self.plan.row_ends)
            s.tile_counts = ptr(self.plan.tile_counts)
            s.n_groups = self.plan.n_groups
        s.epoch = max(self.lock_epoch if variant == "s1" else self.epoch, 1)
        s.trace_comm_counter = ptr(self.trace_comm_counter)
        s.trace_start_clock = ptr(self.trace_start_clock)
        s.trace_ready_clock = ptr(self.trace_ready_clock)
        s.trace_done_clock = ptr(self.trace_done_clock)
        s.fault = ptr(self.fault)
        s.spin_limit_ns = int(self.spin_limit_ns)
        return s

    def raise_if_faulted(self) -> None:
        """Synchronises the stream; raises if a device-side wait ran into its deadline."""
        torch.cuda.current_stream().synchronize()
        if int(self.fault.item()) != 0:
            self.fault.zero_()
            raise RuntimeError(
                "a communication workgroup gave up waiting for a tile/TileGroup signal "
                f"(spin limit {self.spin_limit_ns} ns); the output of this launch is incomplete"
            )


def byref(x):
    return C.byref(x) if x is not None else None
