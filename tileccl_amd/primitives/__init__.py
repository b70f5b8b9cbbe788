"""Host launchers of the stand-alone collectives and of block put / get, on the HIP copy and
reduce kernels (reference: ``/root/reference/tileccl/primitives/__init__.py``)."""

from tileccl_amd.primitives.collectives import (
    MAX_COLLECTIVE_WORLD_SIZE,
    allgather,
    allreduce,
    allgather_staged,
    allreduce_staged,
    broadcast_staged,
    reduce_scatter_staged,
    scatter_staged,
    broadcast,
    reduce_scatter,
    scatter,
)
from tileccl_amd.primitives.communication import copy_block, get, put

__all__ = [
    "MAX_COLLECTIVE_WORLD_SIZE",
    "allgather",
    "allreduce",
    "allgather_staged",
    "allreduce_staged",
    "broadcast_staged",
    "reduce_scatter_staged",
    "scatter_staged",
    "broadcast",
    "copy_block",
    "get",
    "put",
    "reduce_scatter",
    "scatter",
]
