"""Tree-based invariant kernels: the TP-invariant matmul and the shard combine."""
from .tree_based_matmul import matmul_tp_persistent, choose_leaf_k  # noqa: F401
from .tree_based_all_reduce import tree_all_reduce_sum, tree_all_reduce_sum_native, tree_combine  # noqa: F401
