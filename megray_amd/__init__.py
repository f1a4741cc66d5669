"""MI355X-native virtual-rank backend for MegRay's data-parallel hot path."""
from .api import (MAX_RANKS, Backend, Client, Collective, CollectivePlan, Communicator, DType, FoldOrder, MegRayError,
                  RankBuffers, ReduceOp, Schedule, Status, all_gather, all_reduce, all_to_all, broadcast, chunk_partition,
                  create_server, describe, fold_order, gather, get_communicator, get_dtype_size, get_free_port,
                  place_tensors, probe_bounded_wait, rank_buffers_layout, reduce, reduce_scatter, reduce_to_root, scatter)

__all__ = [
    "MAX_RANKS", "Backend", "Client", "Collective", "CollectivePlan", "Communicator", "DType", "FoldOrder", "MegRayError",
    "RankBuffers", "ReduceOp", "Schedule", "Status", "all_gather", "all_reduce", "all_to_all", "broadcast",
    "chunk_partition", "create_server", "describe", "fold_order", "gather", "get_communicator", "get_dtype_size",
    "get_free_port", "place_tensors", "probe_bounded_wait", "rank_buffers_layout", "reduce", "reduce_scatter",
    "reduce_to_root", "scatter",
]
