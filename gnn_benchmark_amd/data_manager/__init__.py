from .CommBuffer import CommBuffer, CommBufferForQuantization
from .CommSplits import CommSplits
from .DataLoader import get_distributed_graph, get_distributed_graph_for_pre_aggressive, load_graph_structures
from .DataProcessor import DataProcessor, DataProcessorForPreAggresive
from .DistributedGraph import DistributedGraph, DistributedGraphForPre
from .PartitionFiles import divide_edges_into_local_and_remote, save_partition_files

__all__ = ["CommBuffer", "CommBufferForQuantization", "CommSplits", "DataProcessor", "DataProcessorForPreAggresive", "DistributedGraph",
           "DistributedGraphForPre", "get_distributed_graph", "get_distributed_graph_for_pre_aggressive",
           "load_graph_structures", "divide_edges_into_local_and_remote", "save_partition_files"]
