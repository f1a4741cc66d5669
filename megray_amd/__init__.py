"""MI355X-native virtual-rank backend for MegRay's data-parallel hot path."""
from .api import (MAX_RANKS, Backend, Collective, DType, FoldOrder, MegRayError, ReduceOp, Schedule, Status,
                  all_gather, all_reduce, all_to_all, broadcast, chunk_partition, describe, fold_order,
                  gather, get_dtype_size, reduce, reduce_scatter, scatter)

__all__ = [
    "MAX_RANKS", "Backend", "Collective", "DType", "FoldOrder", "MegRayError", "ReduceOp", "Schedule",
    "Status", "all_gather", "all_reduce", "all_to_all", "broadcast", "chunk_partition", "describe",
    "fold_order", "gather", "get_dtype_size", "reduce", "reduce_scatter", "scatter",
]
