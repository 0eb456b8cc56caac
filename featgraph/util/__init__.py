"""Adjacency partitioning utilities under the reference's import path (python/featgraph/util/__init__.py:1)."""
from featgraph_amd.util import util_convert_csr_to_dds, util_partition_adj_coo_2d  # noqa: F401

__all__ = ["util_convert_csr_to_dds", "util_partition_adj_coo_2d"]
