"""MI355X-native aggregation hot path of a full-batch, graph-partitioned GCN/GraphSAGE
trainer: CSR SpMM forward / transposed backward, pre- and post-aggregation, behind the
operator names the reference trainer uses (``computation_ops.spmm``, ``SPMM_forward``,
``SPMM_backward``, ``Aggregator``)."""
from . import computation_ops  # noqa: F401
from .sparse_tensor import SparseTensor  # noqa: F401
from .spmm_kernel import SPMM_forward, SPMM_backward  # noqa: F401
from .aggregator import Aggregator  # noqa: F401

__all__ = ["computation_ops", "SparseTensor", "SPMM_forward", "SPMM_backward", "Aggregator"]
