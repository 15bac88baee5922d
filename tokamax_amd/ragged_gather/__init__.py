"""Token permute / un-permute ops next to the ragged dot: `ragged_gather`, `ragged_scatter`,
`ragged_gather_reduce` (tokamax/_src/ops/ragged_gather, ragged_scatter, ragged_gather_reduce)."""

from tokamax_amd.ragged_gather.ops import (
    HipRaggedGather,
    HipRaggedGatherReduce,
    HipRaggedScatter,
    ragged_gather,
    ragged_gather_reduce,
    ragged_scatter,
)

__all__ = ["HipRaggedGather", "HipRaggedGatherReduce", "HipRaggedScatter", "ragged_gather", "ragged_gather_reduce",
           "ragged_scatter"]
