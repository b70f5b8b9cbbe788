"""GEMM-output AllGather and GEMM-to-ReduceScatter in the S0 / S1 / S2 variants.

These are the operations behind the reference's headline tables (README.md:66-84).  The
kernels that produced those tables are not part of the reference tree; what is there is
the contract they consumed, and these classes wire exactly that contract to the HIP
kernels:

    spec  = all_gather_spec / reduce_scatter_spec            (collective_spec.py:75-80)
    plan  = build_tile_group_plan(..., row_split_boundaries)  (tile_group.py:244-301)
    tp    = build_p2p_transport_plan(comm_mode, copy_elems)   (transport.py:66-86)
    wg    = tp.build_wg_plan(total_sms, num_comm_wgs, ...)    (wg.py:54-90)
    sig   = allocate_tile_group_signals(heap, n_groups, ...)  (signal.py:43-66)

World size 2 (or more, up to 8) is emulated on one GPU: a peer is another slice of the
same arena.  ``directions`` says which transfers one launch carries out: ``push`` (this
rank's rows to the peers), ``pull`` (the peers' rows into this rank's slice) or both,
which is the full two-rank exchange running through one HBM.
"""

from __future__ import annotations

import ctypes as C

import torch

from tileccl_amd import _launch, _lib
from tileccl_amd.v2.collective_spec import CollectiveSpec, all_gather_spec, reduce_scatter_spec
from tileccl_amd.v2.heap import SymmetricHeap
from tileccl_amd.v2.signal import TileGroupSignalState, allocate_tile_group_signals
from tileccl_amd.v2.tile_group import TileGroupPlan, build_tile_group_plan
from tileccl_amd.v2.transport import CommMode, P2PTransportPlan, build_p2p_transport_plan

PEER_READY = 1 << 30  # word value that marks a resident peer's tiles / groups as complete for every launch


def _directions(value) -> int:
    if isinstance(value, int):
        return value
    if isinstance(value, CommMode):
        return _lib.DIR_PUSH if value is CommMode.PUSH else _lib.DIR_PULL
    names = {"push": _lib.DIR_PUSH, "pull": _lib.DIR_PULL, "both": _lib.DIR_PUSH | _lib.DIR_PULL}
    if value not in names:
        raise ValueError(f"unknown directions={value!r}; expected one of {sorted(names)}")
    return names[value]


class _FusedBase:
    kind = "base"

    def __init__(
        self,
        heap: SymmetricHeap,
        *,
        block_m: int = 128,
        block_n: int = 128,
        group_m: int = 8,
        target_group_tiles: int | None = None,
        tau_min_bytes: int = 262144,
        max_groups: int = 64,
        transport: P2PTransportPlan | None = None,
        num_comm_wgs: int = 0,
        num_gemm_wgs: int = 0,
        macro_tile: int = 0,
        trace: bool = False,
        spin_limit_ns: int = _launch.DEFAULT_SPIN_LIMIT_NS,
    ) -> None:
        self.heap = heap
        self.rank, self.world_size = heap.rank, heap.world_size
        self.block_m, self.block_n, self.group_m = block_m, block_n, group_m
        self.target_group_tiles = target_group_tiles
        self.tau_min_bytes, self.max_groups = tau_min_bytes, max_groups
        self.transport = transport or build_p2p_transport_plan(comm_mode="push", copy_elems=16384)
        self.num_comm_wgs, self.num_gemm_wgs = num_comm_wgs, num_gemm_wgs
        self.macro_tile = macro_tile
        self.trace = trace
        self.spin_limit_ns = spin_limit_ns
        self.spec: CollectiveSpec | None = None
        self.plan: TileGroupPlan | None = None
        self.signals: TileGroupSignalState | None = None
        self.words: _launch.SyncWords | None = None
        self.locks: torch.Tensor | None = None

    # -- planning -----------------------------------------------------------------------
    def _build_plan(self, M: int, N: int, elem_bytes: int, spec: CollectiveSpec) -> None:
        self.spec = spec
        self.plan = build_tile_group_plan(
            M,
            N,
            self.block_m * self.block_n * elem_bytes,
            target_group_tiles=self.target_group_tiles,
            max_groups=self.max_groups,
            block_m=self.block_m,
            block_n=self.block_n,
            group_m=self.group_m,
            tau_min_bytes=self.tau_min_bytes,
            row_split_boundaries=spec.row_split_boundaries(M),
        )
        spec.validate_tile_groups(M, self.plan.groups)
        n = self.plan.n_groups
        self.signals = allocate_tile_group_signals(heap=self.heap, n_groups=n, device="cuda:0")
        self.signals.reset()
        tiles = int(self.plan.group_table.numel())
        self.locks = self.heap.allocate_signal_buffer(tiles)
        self.words = _launch.SyncWords(
            locks=self.locks,
            counter=self.signals.counter,
            barrier=self.signals.barrier,
            plan=_launch.DevicePlan.upload(self.plan),
            host_plan=self.plan,
            spin_limit_ns=self.spin_limit_ns,
        )
        if self.trace:
            self.words.trace_comm_counter = self.signals.trace_comm_counter
            self.words.trace_start_clock = self.signals.trace_start_clock
            self.words.trace_ready_clock = self.signals.trace_ready_clock
            self.words.trace_done_clock = self.signals.trace_done_clock

    def wg_plan(self, total_sms: int):
        """The reference-style workgroup plan of this operation (for reporting)."""
        assert self.plan is not None
        comm = self.num_comm_wgs or total_sms // 5
        return self.transport.build_wg_plan(
            total_sms=total_sms, num_comm_wgs=comm, max_group_elems=self.plan.max_group_elems
        )

    def mark_peers_ready(self) -> None:
        """Emulation aid: declare every peer's tiles and TileGroups complete.

        A peer's ``counter`` / ``locks`` sit at the same offsets of its slice.  With the peers'
        data resident (not produced by a concurrently running peer), their words are preset so
        that pulls and reductions never wait on them.
        """
        assert self.signals is not None and self.locks is not None
        for peer in range(self.world_size):
            if peer == self.rank:
                continue
            self.heap.peer_view(self.signals.counter, peer).fill_(PEER_READY)
            self.heap.peer_view(self.locks, peer).fill_(PEER_READY)

    def _descs(self, directions: int, variant: str):
        assert self.words is not None
        if variant not in _launch.VARIANTS:
            raise ValueError(f"unknown variant {variant!r}; expected one of {sorted(_launch.VARIANTS)}")
        view = _launch.heap_view(self.heap.get_heap_bases(), self.rank, self.world_size)
        transport = _launch.transport_desc(
            directions, self.transport.copy_elems, self.transport.reduce_elems, self.num_comm_wgs
        )
        if variant != "s0":  # S1 launches number the locks they write, S2 launches the counters
            self.words.next_epoch(variant)
        return view, transport, self.words.desc(variant)

    def check_faults(self) -> None:
        if self.words is not None:
            self.words.raise_if_faulted()


class FusedGemmAllGather(_FusedBase):
    """Gate 1: ``out[rank*M:(rank+1)*M] = A @ B``, and the row blocks are exchanged.

    ``out`` (``world_size*M x N``) must live in the heap; every rank's ``out`` sits at the
    same slice offset, so rank ``r``'s block goes to rows ``[r*M, (r+1)*M)`` of every slice
    (layout of ``tile_allgather``, reference primitives/collectives.py:613-663).
    """

    kind = "all_gather"

    def __init__(self, heap: SymmetricHeap, M: int, N: int, dtype: torch.dtype = torch.float16, *,
                 directions="both", **kwargs) -> None:
        super().__init__(heap, **kwargs)
        self.M, self.N, self.dtype = M, N, dtype
        self.directions = _directions(directions if directions is not None else self.transport.comm_mode)
        self.out = heap.allocate_tensor((self.world_size * M, N), dtype)
        self.local_block = self.out[self.rank * M : (self.rank + 1) * M]
        self._build_plan(M, N, self.out.element_size(), all_gather_spec(world_size=self.world_size))

    def peer_out(self, peer: int) -> torch.Tensor:
        return self.heap.peer_view(self.out, peer)

    def __call__(self, A: torch.Tensor, B: torch.Tensor, variant: str = "s2", alpha: float = 1.0,
                 scale_a: float = 1.0, scale_b: float = 1.0) -> torch.Tensor:
        alpha = float(alpha) * float(scale_a) * float(scale_b)  # per-tensor dequantisation scales of fp8 inputs
        gemm = _launch.gemm_desc(
            A, B, self.local_block, block_m=self.block_m, block_n=self.block_n, group_m=self.group_m,
            alpha=alpha, num_wgs=self.num_gemm_wgs, macro_tile=self.macro_tile,
        )
        view, transport, sync = self._descs(self.directions, variant)
        rc = _lib.load().tccl_gemm_allgather(
            C.byref(gemm), _launch.ptr(self.out), int(self.out.stride(0)), C.byref(view), C.byref(sync),
            C.byref(transport), _launch.VARIANTS[variant], _launch.stream_ptr(),
        )
        _lib.check(rc, f"tccl_gemm_allgather[{variant}]")
        return self.out


class FusedGemmReduceScatter(_FusedBase):
    """Gate 2: ``partial = A @ B`` (``M x N``), then ``out = cast(sum over ranks of partial[shard])``.

    ``partial`` lives in the heap at the same offset on every rank; rank ``r`` owns rows
    ``[r*M/ws, (r+1)*M/ws)`` and pulls the peers' partial rows (the pull-reduce of
    ``tile_reduce_scatter``, reference primitives/collectives.py:730-783), accumulating in
    fp32.  With ``emulate_peer`` the launch also performs the other owners' reductions into
    their slices, i.e. the whole two-rank operation on one GPU.

    ``own_rows_in_registers``: in the one-launch variants on the 256 x 256 tile (shards of
    whole tiles) the rows this rank owns never leave the accumulators as a partial: the peers'
    partials are added in the GEMM epilogue.  ``out`` is bit-identical; those rows of
    ``partial`` keep whatever they held.  Ignored where it does not apply.
    """

    kind = "reduce_scatter"

    def __init__(self, heap: SymmetricHeap, M: int, N: int, *, partial_dtype: torch.dtype = torch.float32,
                 out_dtype: torch.dtype = torch.float16, emulate_peer: bool = True,
                 own_rows_in_registers: bool = False, **kwargs) -> None:
        kwargs.setdefault("transport", build_p2p_transport_plan(comm_mode="pull", copy_elems=16384, reduce_elems=16384))
        super().__init__(heap, **kwargs)
        self.M, self.N = M, N
        self.emulate_peer = emulate_peer
        self.own_rows_in_registers = own_rows_in_registers
        spec = reduce_scatter_spec(world_size=self.world_size)
        self.shard_rows = spec.shard_rows(M)
        self.partial = heap.allocate_tensor((M, N), partial_dtype)
        self.out = heap.allocate_tensor((self.shard_rows, N), out_dtype)
        self._build_plan(M, N, self.partial.element_size(), spec)

    def peer_partial(self, peer: int) -> torch.Tensor:
        return self.heap.peer_view(self.partial, peer)

    def peer_out(self, peer: int) -> torch.Tensor:
        return self.heap.peer_view(self.out, peer)

    def __call__(self, A: torch.Tensor, B: torch.Tensor, variant: str = "s2", alpha: float = 1.0,
                 scale_a: float = 1.0, scale_b: float = 1.0) -> torch.Tensor:
        alpha = float(alpha) * float(scale_a) * float(scale_b)  # per-tensor dequantisation scales of fp8 inputs
        gemm = _launch.gemm_desc(
            A, B, self.partial, block_m=self.block_m, block_n=self.block_n, group_m=self.group_m,
            alpha=alpha, num_wgs=self.num_gemm_wgs, macro_tile=self.macro_tile,
            flags=_lib.GEMM_OWN_ROWS_IN_REGISTERS if self.own_rows_in_registers else 0,
        )
        view, transport, sync = self._descs(_lib.DIR_PULL, variant)
        rc = _lib.load().tccl_gemm_reducescatter(
            C.byref(gemm), _launch.ptr(self.out), _launch.dtype_code(self.out.dtype), int(self.out.stride(0)),
            C.byref(view), C.byref(sync), C.byref(transport), int(self.emulate_peer),
            _launch.VARIANTS[variant], _launch.stream_ptr(),
        )
        _lib.check(rc, f"tccl_gemm_reducescatter[{variant}]")
        return self.out
