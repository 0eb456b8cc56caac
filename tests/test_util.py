"""Adjacency partitioning utilities: the reference's golden vectors, a brute-force
restatement, and structural invariants.  All outputs are integer / index data: exact equality."""
import json
import os

import numpy as np
import pytest
import scipy.sparse

from conftest import reference_test_matrix
from featgraph_amd.util import util_convert_csr_to_dds, util_partition_adj_coo_2d
from oracle import util_ref

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "util_5x5.json")))


def _golden_coo():
    m = scipy.sparse.coo_matrix((np.array(GOLDEN["edge_id"]), (np.array(GOLDEN["row"]), np.array(GOLDEN["col"]))),
                                shape=tuple(GOLDEN["shape"]), dtype="int32")
    assert np.array_equal(m.toarray(), np.array(GOLDEN["dense"]))
    return m


def test_dds_golden_vectors_of_the_reference():
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(_golden_coo().tocsr(), GOLDEN["dds_num_col_partitions"])
    assert np.array_equal(vals, GOLDEN["dds_vals"])
    assert np.array_equal(s1_idx, GOLDEN["dds_s1_idx"])
    assert np.array_equal(s1_pos, GOLDEN["dds_s1_pos"])


def test_coo2d_golden_vector_of_the_reference():
    ids, rows, cols = util_partition_adj_coo_2d(_golden_coo(), GOLDEN["coo2d_num_row_partitions"],
                                                GOLDEN["coo2d_num_col_partitions"])
    assert np.array_equal(ids, GOLDEN["coo2d_edge_id"])
    # the ids index the original edge list
    assert np.array_equal(rows, np.array(GOLDEN["row"])[ids - 1])
    assert np.array_equal(cols, np.array(GOLDEN["col"])[ids - 1])


def test_brute_force_restatement_reproduces_the_golden_vectors():
    m = _golden_coo().tocsr()
    pos, idx, vals = util_ref.convert_csr_to_dds(m.indptr, m.indices, m.data, 5, 2)
    assert np.array_equal(pos, GOLDEN["dds_s1_pos"]) and np.array_equal(idx, GOLDEN["dds_s1_idx"])
    assert np.array_equal(vals, GOLDEN["dds_vals"])
    ids, _, _ = util_ref.partition_adj_coo_2d(GOLDEN["row"], GOLDEN["col"], 5, 5, 2, 2)
    assert np.array_equal(ids, GOLDEN["coo2d_edge_id"])


@pytest.mark.parametrize("shape,P", [((127, 255), 1), ((127, 255), 4), ((127, 255), 7), ((31, 10), 16), ((9, 64), 3)])
def test_dds_equals_brute_force(shape, P):
    adj = reference_test_matrix("csr", seed=11, shape=shape, density=0.15)
    got = util_convert_csr_to_dds(adj, P)
    want = util_ref.convert_csr_to_dds(adj.indptr, adj.indices, adj.data, shape[1], P)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    s1_pos, s1_idx, vals = got
    assert s1_pos.dtype == adj.indptr.dtype and s1_idx.dtype == adj.indices.dtype and vals.dtype == adj.data.dtype
    assert s1_pos.shape == (P * (shape[0] + 1),) and s1_pos[0] == 0 and s1_pos[-1] == adj.nnz
    # re-globalised columns rebuild the matrix
    width = (shape[1] + P - 1) // P
    rebuilt = np.zeros(shape, dtype=np.float64)
    for p in range(P):
        seg = s1_pos[p * (shape[0] + 1):(p + 1) * (shape[0] + 1)]
        for r in range(shape[0]):
            for e in range(seg[r], seg[r + 1]):
                rebuilt[r, s1_idx[e] + p * width] += vals[e]
    assert np.array_equal(rebuilt, adj.toarray().astype(np.float64))


def test_dds_keeps_unsorted_row_order_inside_a_block():
    indptr = np.array([0, 4], dtype=np.int32)
    indices = np.array([5, 1, 4, 0], dtype=np.int32)
    data = np.array([1, 2, 3, 4], dtype=np.float32)
    adj = scipy.sparse.csr_matrix((data, indices, indptr), shape=(1, 6))
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(adj, 2)
    assert np.array_equal(vals, [2, 4, 1, 3]) and np.array_equal(s1_idx, [1, 0, 2, 1])
    assert np.array_equal(s1_pos, [0, 2, 2, 4])


@pytest.mark.parametrize("shape,Pr,Pc", [((127, 255), 1, 1), ((127, 255), 4, 4), ((127, 255), 3, 5),
                                         ((20, 33), 32, 2), ((64, 9), 2, 16)])
def test_coo2d_equals_brute_force_and_invariants(shape, Pr, Pc):
    coo = reference_test_matrix("coo", seed=12, shape=shape, density=0.2)
    perm = np.random.default_rng(12).permutation(coo.nnz)          # callers may hand edges in any order
    coo = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=shape)
    data_before = coo.data.copy()
    ids, rows, cols = util_partition_adj_coo_2d(coo, Pr, Pc)
    want = util_ref.partition_adj_coo_2d(coo.row, coo.col, shape[0], shape[1], Pr, Pc)
    for g, w in zip((ids, rows, cols), want):
        assert np.array_equal(g, w)
    assert ids.dtype == np.int32 and rows.dtype == coo.row.dtype and cols.dtype == coo.col.dtype
    assert np.array_equal(np.sort(ids), np.arange(1, coo.nnz + 1))  # a permutation of 1..nnz
    assert np.array_equal(rows, coo.row[ids - 1]) and np.array_equal(cols, coo.col[ids - 1])
    h, w_ = (shape[0] + Pr - 1) // Pr, (shape[1] + Pc - 1) // Pc
    block = (rows // h) * Pc + cols // w_
    assert np.all(np.diff(block) >= 0)                              # blocks in row-major order
    same = np.diff(block) == 0
    key = rows.astype(np.int64) * shape[1] + cols
    assert np.all(np.diff(key)[same] > 0)                           # (row, col) ascending inside a block
    assert np.array_equal(coo.data, data_before)                    # the caller's matrix is untouched
    # edge_mapping round trip (module/sddmm.py:49, tests/test_module_sddmm.py:31-32)
    per_edge = np.arange(coo.nnz) * 10.0
    assert np.array_equal(per_edge[ids - 1][np.argsort(ids)], per_edge)


def test_coo2d_rejects_duplicate_edges():
    coo = scipy.sparse.coo_matrix((np.ones(3), (np.array([0, 1, 0]), np.array([2, 1, 2]))), shape=(3, 3))
    with pytest.raises(ValueError):
        util_partition_adj_coo_2d(coo, 2, 2)
