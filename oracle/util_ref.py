"""Brute-force restatement of the reference's adjacency partitioning.

TEST INFRASTRUCTURE ONLY.  Plain Python loops over blocks, rows and nonzeros,
for small matrices: what the reference obtains through scipy slicing is spelled
out entry by entry.
"""
import numpy as np


def convert_csr_to_dds(indptr, indices, data, num_cols, num_col_partitions):
    """util/adj_partitioning.py:29-57: per column block, the block's CSR (local column ids)."""
    num_rows = len(indptr) - 1
    width = (num_cols + num_col_partitions - 1) // num_col_partitions
    s1_pos, s1_idx, vals = [], [], []
    for p in range(num_col_partitions):
        lo = p * width
        hi = num_cols if p == num_col_partitions - 1 else (p + 1) * width
        for r in range(num_rows):
            s1_pos.append(len(s1_idx))                      # indptr of the block + running offset (:50)
            for e in range(indptr[r], indptr[r + 1]):
                if lo <= indices[e] < hi:
                    s1_idx.append(indices[e] - lo)          # block-local column id (:51)
                    vals.append(data[e])                    # (:49)
        s1_pos.append(len(s1_idx))
    return np.array(s1_pos), np.array(s1_idx), np.array(vals)


def partition_adj_coo_2d(row, col, num_rows, num_cols, num_row_partitions, num_col_partitions):
    """util/adj_partitioning.py:85-128: ids 1..nnz (:92), CSR with sorted rows (:95), blocks row-major (:103-104)."""
    nnz = len(row)
    per_row = [[] for _ in range(num_rows)]
    for e in range(nnz):
        per_row[row[e]].append((col[e], e + 1))
    for lst in per_row:
        lst.sort()
    height = (num_rows + num_row_partitions - 1) // num_row_partitions
    width = (num_cols + num_col_partitions - 1) // num_col_partitions
    ids, rows, cols = [], [], []
    for bi in range(num_row_partitions):
        r_lo = bi * height
        r_hi = num_rows if bi == num_row_partitions - 1 else (bi + 1) * height
        for bj in range(num_col_partitions):
            c_lo = bj * width
            c_hi = num_cols if bj == num_col_partitions - 1 else (bj + 1) * width
            for r in range(r_lo, min(r_hi, num_rows)):
                for c, eid in per_row[r]:
                    if c_lo <= c < c_hi:
                        ids.append(eid)
                        rows.append(r)
                        cols.append(c)
    return np.array(ids), np.array(rows), np.array(cols)
