"""CPU restatement of the fused GEMM + collective semantics (test infrastructure only).

All arithmetic is torch on the CPU.  Follows
    GEMM: fp32 accumulate, one cast to the output type
        /root/reference/tileccl/kernels/gemm.py:139-167, patterns/bulk_sync.py:213-238
    scatter placement of a tile into a peer's C
        /root/reference/tileccl/patterns/_helpers.py:145-157
    fan-out to every peer but self
        /root/reference/tileccl/patterns/_helpers.py:161-199
    all-gather layout [block_rank0 | block_rank1 | ...]
        /root/reference/tileccl/primitives/collectives.py:628-663
    reduce-scatter: owner's chunk first, then peers ascending
        /root/reference/tileccl/primitives/collectives.py:766-783
    (this build accumulates the reduction in fp32 and rounds once, as its north star asks;
     the reference accumulates in the tensor dtype)
    chained gather -> GEMM -> scatter: column block p of the gathered input is rank p's shard
        /root/reference/tileccl/patterns/chained_ag_gemm_rs.py:262-340 (gather), :343-391 (GEMM),
        :393-425 (every tile stored to every peer)
"""

from __future__ import annotations

import torch


def gemm(A: torch.Tensor, B: torch.Tensor, out_dtype: torch.dtype, alpha: float = 1.0) -> torch.Tensor:
    """``cast(alpha * (A.float() @ B.float()))``; fp8 inputs are dequantised exactly by ``.float()``."""
    acc = A.float() @ B.float()
    if alpha != 1.0:
        acc = acc * alpha
    return acc.to(out_dtype)


def scatter_into_peer(peer_C: torch.Tensor, local_C: torch.Tensor, src_col_offset: int, cols: int,
                      dst_ld: int, dst_col_offset: int) -> None:
    """Vectorised placement: peer_flat[r*dst_ld + dst_col_offset + j] = local_C[r, src_col_offset + j]."""
    M = local_C.shape[0]
    flat = peer_C.reshape(-1)
    rows = torch.arange(M).unsqueeze(1) * dst_ld
    js = torch.arange(cols).unsqueeze(0)
    flat[(rows + dst_col_offset + js).reshape(-1)] = local_C[:, src_col_offset:src_col_offset + cols].reshape(-1)


def scatter_into_peer_by_tiles(peer_C, local_C, src_col_offset, cols, dst_ld, dst_col_offset,
                               block_m=128, block_n=128) -> None:
    """Element loop over tiles with the reference's mask, for small cases (_helpers.py:148-157)."""
    M, N = local_C.shape
    flat = peer_C.reshape(-1)
    for tm in range(-(-M // block_m)):
        for tn in range(-(-N // block_n)):
            for r in range(tm * block_m, min((tm + 1) * block_m, M)):
                for c in range(tn * block_n, min((tn + 1) * block_n, N)):
                    if src_col_offset <= c < src_col_offset + cols:
                        flat[r * dst_ld + dst_col_offset + (c - src_col_offset)] = local_C[r, c]


def gemm_allscatter(As, Bs, Cs, specs) -> None:
    """All ranks of one process: every rank computes its C, then scatters to every peer.

    ``specs[r]`` carries the four placement integers of rank ``r``; ranks run in rank order,
    like sequential single-process launches do.
    """
    world = len(As)
    for r in range(world):
        Cs[r].copy_(gemm(As[r], Bs[r], Cs[r].dtype))
        s = specs[r]
        for p in range(world):
            if p != r:
                scatter_into_peer(Cs[p], Cs[r], s["src_col_offset"], s["cols"], s["dst_ld"], s["dst_col_offset"])


def allgather_exchange(outs, rank: int, M: int, push: bool = True, pull: bool = True) -> None:
    """Rank's own block goes to every peer (push); every peer's block comes in (pull)."""
    world = len(outs)
    for p in range(world):
        if p == rank:
            continue
        if push:
            outs[p][rank * M:(rank + 1) * M] = outs[rank][rank * M:(rank + 1) * M]
        if pull:
            outs[rank][p * M:(p + 1) * M] = outs[p][p * M:(p + 1) * M]


def gemm_allgather(A, B, outs, rank: int, push: bool = True, pull: bool = True, alpha: float = 1.0) -> None:
    M = A.shape[0]
    outs[rank][rank * M:(rank + 1) * M] = gemm(A, B, outs[rank].dtype, alpha)
    allgather_exchange(outs, rank, M, push, pull)


def reduce_rows(partials, owner: int, out_dtype: torch.dtype) -> torch.Tensor:
    """Owner's shard: fp32 sum, owner first then the other ranks ascending, one rounding."""
    world = len(partials)
    shard = partials[0].shape[0] // world
    lo, hi = owner * shard, (owner + 1) * shard
    acc = partials[owner][lo:hi].float().clone()
    for p in range(world):
        if p != owner:
            acc += partials[p][lo:hi].float()
    return acc.to(out_dtype)


def gemm_reducescatter(A, B, partials, outs, rank: int, emulate_peer: bool = True, alpha: float = 1.0) -> None:
    """partials[rank] = A@B (partial dtype); outs[o] = reduce(owner o) for the owners handled."""
    partials[rank].copy_(gemm(A, B, partials[rank].dtype, alpha))
    for owner in range(len(partials)):
        if owner == rank or emulate_peer:
            outs[owner].copy_(reduce_rows(partials, owner, outs[owner].dtype))


def gather_cols(shards) -> torch.Tensor:
    """Gathered input: shard p occupies columns [p*K_shard, (p+1)*K_shard) (chained_ag_gemm_rs.py:270-337).

    The reference kernel offsets workspace rows by the column stride (:298, :353), which makes
    rows overlap; this follows the layout its docstring and its (M, K) workspace state."""
    M, ks = shards[0].shape
    out = torch.empty(M, ks * len(shards), dtype=shards[0].dtype)
    for p, s in enumerate(shards):
        out[:, p * ks : (p + 1) * ks] = s
    return out


def chained_ag_gemm_rs(shards, W, outs, rank: int, alpha: float = 1.0) -> torch.Tensor:
    """outs[q] = gather_cols(shards) @ W for every rank q (rank ``rank`` computes, all receive).  Returns the gathered input."""
    gathered = gather_cols(shards)
    result = gemm(gathered, W, outs[rank].dtype, alpha)
    for o in outs:
        o.copy_(result)
    return gathered


# ---- stand-alone collectives on flat tensors (one entry per rank) ---------------------------
# tile_allgather  /root/reference/tileccl/primitives/collectives.py:613-663
# tile_scatter    :671-727      tile_reduce_scatter :730-783      tile_broadcast :791-836
# host restatement of the reduction in the reference itself: :2513-2546 (ascending rank order
# in the tensor dtype; here fp32, owner first, one rounding -- see the module docstring)


def allgather(tensors):
    """Every rank's output: the ranks' blocks one after the other."""
    full = torch.cat([t.reshape(-1) for t in tensors])
    return [full.clone() for _ in tensors]


def broadcast(tensors, root: int):
    """Every rank's tensor after the call: the root's."""
    return [tensors[root].clone() for _ in tensors]


def scatter(tensor_root: torch.Tensor, world: int):
    """Rank i's output: chunk i of the root's tensor."""
    block = tensor_root.numel() // world
    flat = tensor_root.reshape(-1)
    return [flat[i * block : (i + 1) * block].clone() for i in range(world)]


def reduce_scatter(tensors, out_dtype: torch.dtype):
    """Rank r's output: the sum over ranks of their chunk r."""
    world = len(tensors)
    rows = [t.reshape(world, -1) for t in tensors]
    return [reduce_rows(rows, r, out_dtype).reshape(-1) for r in range(world)]


def allreduce(tensors):
    """Every rank's tensor after all calls: the reduced chunks one after the other."""
    full = torch.cat(reduce_scatter(tensors, tensors[0].dtype))
    return [full.clone() for _ in tensors]


def allreduce_staged(tensors):
    """Every rank's tensor after the staged all-reduce (the protocol of _allreduce_staged_kernel,
    /root/reference/tileccl/primitives/collectives.py:840-962): the ranks' values added in
    ascending rank order in fp32 and rounded once, the same bits on every rank.  (The reference
    kernel adds in the tensor dtype starting from the rank's own values; for two ranks, and for
    values whose sums are exact, the two agree.)"""
    acc = tensors[0].float()
    for t in tensors[1:]:
        acc = acc + t.float()
    return [acc.to(tensors[0].dtype) for _ in tensors]


def allreduce_staged_reference_order(tensors):
    """What the REFERENCE's staged all-reduce leaves on each rank (_allreduce_staged_kernel,
    /root/reference/tileccl/primitives/collectives.py:883-935): rank r starts from its own values and adds
    the other ranks' snapshots in ascending rank order, every addition in the tensor's dtype (``_reduce_op``
    on the loaded values, :388-400), so for three or more ranks and inexact sums the ranks may end up with
    different bits.  This build deliberately does not reproduce that (``allreduce_staged`` above: fp32, rank
    order, one rounding, the same bits everywhere); this function exists so that the tests can hold the
    distance between the two: for two ranks and for exact sums they coincide, otherwise they differ by
    rounding only."""
    out = []
    for r, own in enumerate(tensors):
        acc = own.clone()
        for p, t in enumerate(tensors):
            if p != r:
                acc = (acc + t).to(own.dtype)  # torch adds 16-bit CPU tensors exactly and rounds once to the dtype
        out.append(acc)
    return out


def rounding_bound(tensors, additions: int):
    """Element-wise bound on the difference between two orders / precisions of the same sum of ``tensors``:
    ``additions`` roundings, each at most one unit in the last place of a partial sum, itself at most the sum
    of the magnitudes."""
    eps = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7, torch.float32: 2.0**-23}[tensors[0].dtype]
    return additions * eps * sum(t.float().abs() for t in tensors)


def expected_counters(tile_counts, epoch: int = 1):
    """counter[g] after ``epoch`` launches without reset: every tile of the group signalled once each."""
    return [epoch * t for t in tile_counts]
