"""MI355X-native virtual-rank backend for MegRay's data-parallel hot path."""
from .api import (MAX_RANKS, Backend, Client, Collective, CollectivePlan, Communicator, DType, FoldOrder, MegRayError, ReduceOp,
                  Schedule, Status, all_gather, all_reduce, all_to_all, broadcast, chunk_partition, create_server,
                  describe, fold_order, gather, get_communicator, get_dtype_size, get_free_port, probe_bounded_wait, reduce,
                  reduce_scatter, reduce_to_root, scatter)

__all__ = [
    "MAX_RANKS", "Backend", "Client", "Collective", "CollectivePlan", "Communicator", "DType", "FoldOrder", "MegRayError",
    "ReduceOp", "Schedule", "Status", "all_gather", "all_reduce", "all_to_all", "broadcast", "chunk_partition",
    "create_server", "describe", "fold_order", "gather", "get_communicator", "get_dtype_size", "get_free_port",
    "probe_bounded_wait", "reduce", "reduce_scatter", "reduce_to_root", "scatter",
]
