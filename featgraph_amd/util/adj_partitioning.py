"""Host-side adjacency re-orderings for cache blocking.

Same names, arguments and outputs as the reference's featgraph.util
(util/adj_partitioning.py:7-57 and :60-128).  The reference cuts the matrix
into blocks with scipy slicing, one block at a time; here both functions are a
single stable sort over per-nonzero block keys, which produces the same arrays
in O(nnz log nnz) whatever the number of blocks.
"""
import numpy as np

__all__ = ["util_convert_csr_to_dds", "util_partition_adj_coo_2d"]


def _block_width(extent, parts):
    if parts < 1:
        raise ValueError("the number of partitions must be at least 1")
    return max(1, (extent + parts - 1) // parts)


def util_convert_csr_to_dds(adj_scipy_csr, num_col_partitions):
    """Split a CSR matrix into column blocks (source-vertex partitioning), "DDS" layout.

    Block p holds the columns [p*w, (p+1)*w) with w = ceil(num_cols / P); the
    last block takes what is left (reference util/adj_partitioning.py:42-47).

    Returns
    -------
    s1_pos : [P * (num_rows + 1)], dtype of indptr
        For block p, entries p*(num_rows+1) .. give that block's row pointer
        into s1_idx / vals (already offset by the blocks before it).
    s1_idx : [nnz], dtype of indices
        Block-local column ids, block after block, each block in CSR order.
    vals : [nnz], dtype of data
    """
    num_rows, num_cols = adj_scipy_csr.shape
    indptr, indices, data = adj_scipy_csr.indptr, adj_scipy_csr.indices, adj_scipy_csr.data
    parts = int(num_col_partitions)
    width = _block_width(num_cols, parts)
    block = indices.astype(np.int64) // width
    # nonzeros are already in (row, position) order, so a stable sort by block
    # leaves every block in CSR order
    order = np.argsort(block, kind="stable")
    vals = data[order]
    s1_idx = (indices[order].astype(np.int64) - block[order] * width).astype(indices.dtype)
    rows = np.repeat(np.arange(num_rows, dtype=np.int64), np.diff(indptr))
    counts = np.bincount(block * num_rows + rows, minlength=parts * num_rows).reshape(parts, num_rows)
    pos = np.zeros((parts, num_rows + 1), dtype=np.int64)
    np.cumsum(counts, axis=1, out=pos[:, 1:])
    pos[1:] += np.cumsum(pos[:-1, -1])[:, None]
    return pos.reshape(-1).astype(indptr.dtype), s1_idx, vals


def util_partition_adj_coo_2d(adj_scipy_coo, num_row_partitions, num_col_partitions):
    """Re-order the edges of a COO matrix block by block over a 2-D grid.

    Blocks are rows [i*h, (i+1)*h) x columns [j*w, (j+1)*w) with h, w the
    ceil-divided extents, visited row-major (reference
    util/adj_partitioning.py:100-104); inside a block edges are ordered by row,
    then by column (:95, :119).  Edge ids are 1-based positions in the input.

    Unlike the reference (:92) the caller's matrix is left untouched: its
    `data` is not overwritten with the edge ids.  A matrix that stores the same
    (row, col) pair twice is rejected (the reference would merge the two ids
    into their sum).

    Returns
    -------
    edge_id_list, row_indices, col_indices : [nnz] each; ids are int32, the
    index arrays keep the dtype of the input's row / col.
    """
    num_rows, num_cols = adj_scipy_coo.shape
    row, col = adj_scipy_coo.row, adj_scipy_coo.col
    nnz = row.shape[0]
    if col.shape[0] != nnz:
        raise ValueError("length of row indices and that of col indices do not match")
    height = _block_width(num_rows, int(num_row_partitions))
    width = _block_width(num_cols, int(num_col_partitions))
    r64, c64 = row.astype(np.int64), col.astype(np.int64)
    block = (r64 // height) * int(num_col_partitions) + c64 // width
    order = np.lexsort((c64, r64, block))
    cell = r64[order] * num_cols + c64[order]
    if nnz > 1 and np.any(cell[1:] == cell[:-1]):
        raise ValueError("duplicate (row, col) entries are not supported by 2-D partitioning")
    return (order + 1).astype(np.int32), row[order], col[order]
