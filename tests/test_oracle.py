"""Pins the CPU checker (oracle/) before anything is compared with it.

Every check here is independent of the oracle's own formula text: library
routines (scipy's csr.dot, numpy gather-sum, einsum: the closed forms the
reference's own tests use, tests/test_module_spmm.py:29-30 and
tests/test_module_sddmm.py:34-37), integer cases that float32 represents
exactly, hand-computed cases where a different summation order or a fused
multiply-add gives a different float, and structural invariants.
"""
import numpy as np
import pytest
import scipy.sparse

from conftest import reference_test_matrix
from featgraph_amd import datasets
from featgraph_amd.util import util_convert_csr_to_dds
from oracle import ref


def _int_case(seed=0, shape=(61, 83), density=0.2, F=24):
    """Small integers only: every product and partial sum is exact in float32."""
    rng = np.random.default_rng(seed)
    adj = scipy.sparse.random(shape[0], shape[1], density=density, format="csr", random_state=rng)
    adj.data = rng.integers(1, 5, adj.nnz).astype(np.float32)
    feat = rng.integers(-8, 9, (shape[1], F)).astype(np.float32)
    return adj.astype(np.float32), feat


# ---------------------------------------------------------------- SpMM (CSR, x86 nest)
@pytest.mark.parametrize("P", [1, 4])
def test_spmm_matches_scipy_like_the_reference_tests(adj_127x255, P):
    adj = adj_127x255
    feat = np.random.default_rng(1).random((adj.shape[1], 128), dtype=np.float32)
    out = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat, P)
    np.testing.assert_allclose(adj.dot(feat), out, rtol=1e-4, atol=1e-4)  # the reference's own tolerance
    exact = adj.astype(np.float64).dot(feat.astype(np.float64))
    np.testing.assert_allclose(out, exact, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("P", [1, 2, 8])
def test_spmm_exact_on_integers(P):
    adj, feat = _int_case()
    want = adj.astype(np.int64).dot(feat.astype(np.int64))
    got = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat, P)
    assert np.array_equal(got, want.astype(np.float32))


def test_spmm_nonsquare_shapes_and_empty_rows():
    indptr = np.array([0, 0, 2, 2, 3], dtype=np.int32)      # rows 0 and 2 are empty
    indices = np.array([4, 0, 2], dtype=np.int32)
    vals = np.array([0.5, 2.0, 3.0], dtype=np.float32)
    feat = np.arange(10, dtype=np.float32).reshape(5, 2) + 1
    out = ref.spmm_csr_x86(indptr, indices, vals, feat)
    want = np.array([[0, 0], [0.5 * 9 + 2 * 1, 0.5 * 10 + 2 * 2], [0, 0], [15, 18]], dtype=np.float32)
    assert np.array_equal(out, want)
    assert not np.signbit(out[0]).any()                       # empty rows are +0


def test_spmm_sums_sequentially_in_csr_order():
    # (((0 + 1e8) + 1) - 1e8) + 1 = 1 in float32; pairwise or reversed orders give 0 or 2
    indptr = np.array([0, 4, 8], dtype=np.int32)
    indices = np.array([0, 1, 2, 3, 3, 2, 1, 0], dtype=np.int32)
    vals = np.ones(8, dtype=np.float32)
    feat = np.array([[1e8], [1.0], [-1e8], [1.0]], dtype=np.float32)
    out = ref.spmm_csr_x86(indptr, indices, vals, feat)
    assert out[0, 0] == 1.0       # 1e8, 1, -1e8, 1
    assert out[1, 0] == 0.0       # 1, -1e8, 1, 1e8 : ((1 - 1e8) + 1) + 1e8 = 0


def test_spmm_rounds_product_and_sum_separately():
    # v*x = 1 + 2^-11 + 2^-24 rounds to 1 + 2^-11; a fused multiply-add would leave 2^-24
    v = np.float32(1 + 2.0 ** -12)
    indptr = np.array([0, 2], dtype=np.int32)
    indices = np.array([0, 1], dtype=np.int32)
    vals = np.array([1.0, v], dtype=np.float32)
    feat = np.array([[-(1 + 2.0 ** -11)], [v]], dtype=np.float32)
    out = ref.spmm_csr_x86(indptr, indices, vals, feat)
    assert out[0, 0] == 0.0


def test_spmm_single_term_is_one_rounded_product():
    rng = np.random.default_rng(3)
    n = 50
    indptr = np.arange(n + 1, dtype=np.int32)
    indices = rng.integers(0, n, n).astype(np.int32)
    vals = rng.random(n, dtype=np.float32)
    feat = rng.standard_normal((n, 16), dtype=np.float32)
    out = ref.spmm_csr_x86(indptr, indices, vals, feat)
    assert np.array_equal(out, vals[:, None] * feat[indices])


def test_spmm_tiling_and_row_permutation_do_not_change_bits(adj_127x255):
    adj = adj_127x255
    feat = np.random.default_rng(2).standard_normal((adj.shape[1], 64), dtype=np.float32)
    base = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat, 1)
    for P in (2, 4, 16, 64):
        assert np.array_equal(base, ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat, P))
    perm = np.random.default_rng(5).permutation(adj.shape[0])
    padj = adj[perm]
    assert np.array_equal(base[perm], ref.spmm_csr_x86(padj.indptr, padj.indices, padj.data, feat, 1))


def test_spmm_duplicate_and_unsorted_columns_add_in_stored_order():
    indptr = np.array([0, 4], dtype=np.int32)
    indices = np.array([2, 0, 2, 1], dtype=np.int32)
    vals = np.array([1, 2, 3, 4], dtype=np.float32)
    feat = np.array([[1.0], [10.0], [100.0]], dtype=np.float32)
    assert ref.spmm_csr_x86(indptr, indices, vals, feat)[0, 0] == 100 + 2 + 300 + 40


def test_spmm_linearity_on_integers():
    adj, feat = _int_case(seed=4)
    feat2 = np.random.default_rng(9).integers(-8, 9, feat.shape).astype(np.float32)
    f = lambda x: ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, x)
    assert np.array_equal(f(feat + feat2), f(feat) + f(feat2))


def test_spmm_f64_matches_numpy_double(adj_127x255):
    adj = adj_127x255
    feat = np.random.default_rng(6).standard_normal((adj.shape[1], 33), dtype=np.float32)
    want = adj.astype(np.float64).dot(feat.astype(np.float64))
    np.testing.assert_allclose(ref.spmm_csr_f64(adj.indptr, adj.indices, adj.data, feat), want, rtol=1e-13, atol=1e-13)


def test_spmm_rejects_indivisible_feature_tiling():
    adj, feat = _int_case()
    with pytest.raises(RuntimeError):
        ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat, 5)


# ---------------------------------------------------------------- SpMM (DDS, x86 nest)
@pytest.mark.parametrize("P_col,P_feat", [(4, 1), (4, 4), (7, 2)])
def test_dds_spmm_matches_scipy(adj_127x255, P_col, P_feat):
    adj = adj_127x255
    feat = np.random.default_rng(1).random((adj.shape[1], 128), dtype=np.float32)
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(adj, P_col)
    out = ref.spmm_dds_x86(s1_pos, s1_idx, vals, feat, adj.shape[0], P_col, P_feat)
    np.testing.assert_allclose(adj.dot(feat), out, rtol=1e-4, atol=1e-4)


def test_dds_spmm_exact_on_integers_and_single_block_equals_csr():
    adj, feat = _int_case(seed=7)
    want = adj.astype(np.int64).dot(feat.astype(np.int64)).astype(np.float32)
    for P_col in (1, 2, 5):
        s1_pos, s1_idx, vals = util_convert_csr_to_dds(adj, P_col)
        assert np.array_equal(ref.spmm_dds_x86(s1_pos, s1_idx, vals, feat, adj.shape[0], P_col, 2), want)
    adj2 = reference_test_matrix("csr", seed=8)
    feat2 = np.random.default_rng(8).standard_normal((adj2.shape[1], 32), dtype=np.float32)
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(adj2, 1)
    assert np.array_equal(ref.spmm_dds_x86(s1_pos, s1_idx, vals, feat2, adj2.shape[0], 1, 1),
                          ref.spmm_csr_x86(adj2.indptr, adj2.indices, adj2.data, feat2, 1))


# ---------------------------------------------------------------- SDDMM
def _closed_form_sddmm(coo, src, dst):
    return (src[coo.col].astype(np.float64) * dst[coo.row].astype(np.float64)).sum(axis=-1)


@pytest.mark.parametrize("P", [1, 4])
def test_sddmm_matches_numpy_like_the_reference_tests(P):
    coo = reference_test_matrix("coo", seed=0)
    rng = np.random.default_rng(1)
    src = rng.random((coo.shape[1], 128), dtype=np.float32)   # one row per COLUMN
    dst = rng.random((coo.shape[0], 128), dtype=np.float32)   # one row per ROW
    out = ref.sddmm_x86(coo.row, coo.col, src, dst, P)
    np.testing.assert_allclose((src[coo.col] * dst[coo.row]).sum(axis=-1), out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, _closed_form_sddmm(coo, src, dst), rtol=1e-5, atol=1e-5)


def test_sddmm_exact_on_integers_and_tiling_bits():
    coo = reference_test_matrix("coo", seed=2, shape=(40, 70), density=0.3)
    rng = np.random.default_rng(2)
    src = rng.integers(-8, 9, (70, 24)).astype(np.float32)
    dst = rng.integers(-8, 9, (40, 24)).astype(np.float32)
    want = (src[coo.col].astype(np.int64) * dst[coo.row].astype(np.int64)).sum(-1).astype(np.float32)
    for P in (1, 2, 3, 24):
        assert np.array_equal(ref.sddmm_x86(coo.row, coo.col, src, dst, P), want)
    srcf = rng.standard_normal((70, 24), dtype=np.float32)
    dstf = rng.standard_normal((40, 24), dtype=np.float32)
    base = ref.sddmm_x86(coo.row, coo.col, srcf, dstf, 1)
    for P in (2, 4, 12):
        assert np.array_equal(base, ref.sddmm_x86(coo.row, coo.col, srcf, dstf, P))


def test_sddmm_src_goes_with_col_and_dst_with_row():
    row = np.array([0, 1], dtype=np.int32)
    col = np.array([2, 0], dtype=np.int32)
    src = np.array([[1, 0], [0, 0], [0, 3]], dtype=np.float32)    # 3 columns
    dst = np.array([[5, 7], [11, 13]], dtype=np.float32)          # 2 rows
    out = ref.sddmm_x86(row, col, src, dst)
    assert np.array_equal(out, np.array([3 * 7, 1 * 11], dtype=np.float32))


def test_sddmm_sums_sequentially_in_k():
    row = np.zeros(1, dtype=np.int32)
    col = np.zeros(1, dtype=np.int32)
    src = np.array([[1e8, 1.0, -1e8, 1.0]], dtype=np.float32)
    dst = np.ones((1, 4), dtype=np.float32)
    assert ref.sddmm_x86(row, col, src, dst)[0] == 1.0
    assert ref.sddmm_x86(row, col, src, dst, 2)[0] == 1.0


def test_sddmm_symmetry_permutation_duplicates():
    coo = reference_test_matrix("coo", seed=3, shape=(30, 50), density=0.3)
    rng = np.random.default_rng(3)
    src = rng.standard_normal((50, 16), dtype=np.float32)
    dst = rng.standard_normal((30, 16), dtype=np.float32)
    base = ref.sddmm_x86(coo.row, coo.col, src, dst)
    # swapping the roles on the transposed matrix gives the same products (multiplication commutes)
    assert np.array_equal(base, ref.sddmm_x86(coo.col, coo.row, dst, src))
    perm = rng.permutation(coo.nnz)
    assert np.array_equal(base[perm], ref.sddmm_x86(coo.row[perm], coo.col[perm], src, dst))
    row2, col2 = np.concatenate([coo.row, coo.row]), np.concatenate([coo.col, coo.col])
    assert np.array_equal(np.concatenate([base, base]), ref.sddmm_x86(row2, col2, src, dst))


def test_sddmm_fast_and_f64_variants_agree_with_closed_form():
    coo = reference_test_matrix("coo", seed=4)
    rng = np.random.default_rng(4)
    src = rng.standard_normal((coo.shape[1], 100), dtype=np.float32)
    dst = rng.standard_normal((coo.shape[0], 100), dtype=np.float32)
    exact = _closed_form_sddmm(coo, src, dst)
    np.testing.assert_allclose(ref.sddmm_f64(coo.row, coo.col, src, dst), exact, rtol=1e-13, atol=1e-13)
    for par in (False, True):
        np.testing.assert_allclose(ref.sddmm_x86_fast(coo.row, coo.col, src, dst, par), exact, rtol=1e-5, atol=1e-4)


# ---------------------------------------------------------------- multi-head closed forms
def test_sddmm_mh_matches_einsum_and_reduces_to_vanilla():
    coo = reference_test_matrix("coo", seed=5, shape=(60, 45), density=0.2)
    rng = np.random.default_rng(5)
    src = rng.standard_normal((45, 8, 16), dtype=np.float32)
    dst = rng.standard_normal((60, 8, 16), dtype=np.float32)
    out = ref.sddmm_mh(coo.row, coo.col, src, dst)
    want = np.einsum("ehd,ehd->eh", src[coo.col].astype(np.float64), dst[coo.row].astype(np.float64))
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-5)
    for h in range(8):   # head h alone is a vanilla SDDMM, bit for bit
        assert np.array_equal(out[:, h], ref.sddmm_x86(coo.row, coo.col, np.ascontiguousarray(src[:, h]),
                                                       np.ascontiguousarray(dst[:, h])))
    isrc = rng.integers(-4, 5, (45, 3, 5)).astype(np.float32)
    idst = rng.integers(-4, 5, (60, 3, 5)).astype(np.float32)
    iwant = np.einsum("ehd,ehd->eh", isrc[coo.col].astype(np.int64), idst[coo.row].astype(np.int64))
    assert np.array_equal(ref.sddmm_mh(coo.row, coo.col, isrc, idst), iwant.astype(np.float32))


def test_spmm_mh_matches_per_head_scipy_and_reduces_to_vanilla():
    adj = reference_test_matrix("csr", seed=6, shape=(70, 55), density=0.15)
    rng = np.random.default_rng(6)
    H, D = 4, 12
    w = rng.random((adj.nnz, H), dtype=np.float32)
    src = rng.standard_normal((55, H, D), dtype=np.float32)
    out = ref.spmm_mh(adj.indptr, adj.indices, w, src)
    for h in range(H):
        a_h = scipy.sparse.csr_matrix((w[:, h].astype(np.float64), adj.indices, adj.indptr), shape=adj.shape)
        np.testing.assert_allclose(out[:, h], a_h.dot(src[:, h].astype(np.float64)), rtol=1e-5, atol=1e-5)
        assert np.array_equal(out[:, h], ref.spmm_csr_x86(adj.indptr, adj.indices, np.ascontiguousarray(w[:, h]),
                                                          np.ascontiguousarray(src[:, h])))


def test_softmax_weights_sum_to_one_per_row_and_head():
    adj = datasets.config_graph("c4-mini")
    w = datasets.softmax_edge_weights(adj, 8)
    sums = np.add.reduceat(w.astype(np.float64), adj.indptr[:-1][np.diff(adj.indptr) > 0], axis=0)
    np.testing.assert_allclose(sums, 1.0, rtol=0, atol=1e-5)


# ---------------------------------------------------------------- DDS nest: per-block sums, then their sum
def test_dds_adds_block_sums_not_terms():
    """One row, columns [0,1 | 2,3] in two blocks, values 1e8, 1, -1e8, 1 (features all one).  Term by term the
    float32 sum is 1 (fgref_spmm_csr_x86); block by block it is (1e8 + 1) + (-1e8 + 1) = 1e8 + (-1e8) = 0,
    which is what the reference's DDS nest computes (op/vanilla_spmm.py:201-218)."""
    adj = scipy.sparse.csr_matrix((np.array([1e8, 1, -1e8, 1], np.float32), np.arange(4, dtype=np.int32),
                                   np.array([0, 4], np.int32)), shape=(1, 4))
    feat = np.ones((4, 2), np.float32)
    assert np.all(ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat) == 1.0)
    s1_pos, s1_idx, vals = util_convert_csr_to_dds(adj, 2)
    assert np.all(ref.spmm_dds_x86(s1_pos, s1_idx, vals, feat, 1, 2) == 0.0)


# ---------------------------------------------------------------- generalised message / reduce / edge functions
def _rows_with_edges(adj):
    return np.flatnonzero(np.diff(adj.indptr) > 0)


@pytest.mark.parametrize("msg", ["mul", "add", "sub", "div", "copy_u"])
@pytest.mark.parametrize("reduce", ["sum", "max", "min", "mean"])
def test_generalised_spmm_against_numpy_reduceat(msg, reduce):
    adj, feat = _int_case(seed=3)
    adj.data = np.random.default_rng(4).choice(np.array([1, 2, 4], np.float32), adj.nnz)   # exact quotients too
    out = ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, msg, reduce)
    u, e = feat[adj.indices].astype(np.float64), adj.data.astype(np.float64)[:, None]
    terms = {"mul": u * e, "add": u + e, "sub": u - e, "div": u / e, "copy_u": u}[msg]
    rows = _rows_with_edges(adj)
    starts = adj.indptr[rows]
    fold = {"sum": np.add, "mean": np.add, "max": np.maximum, "min": np.minimum}[reduce].reduceat(terms, starts, axis=0)
    if reduce == "mean":
        fold = fold / np.diff(adj.indptr)[rows][:, None]
    want = np.zeros((adj.shape[0], feat.shape[1]))
    want[rows] = fold
    if reduce == "mean":
        np.testing.assert_allclose(out, want, rtol=1e-6, atol=0)       # one rounded division of an exact sum
    else:
        assert np.array_equal(out, want.astype(np.float32))            # integers and dyadic quotients: exact
    assert np.all(out[np.diff(adj.indptr) == 0] == 0)                  # rows without edges give 0 under every reducer


def test_generalised_spmm_mul_sum_is_the_vanilla_nest(adj_127x255):
    adj = adj_127x255
    feat = np.random.default_rng(5).standard_normal((adj.shape[1], 40), dtype=np.float32)
    assert np.array_equal(ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, "mul", "sum"),
                          ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat))
    # float operands: max / min pick an existing term exactly; sum stays within rounding of float64
    for msg in ("add", "div"):
        u, e = feat[adj.indices], adj.data[:, None] + np.float32(0.5)
        terms = (u + e) if msg == "add" else (u / e)
        rows = _rows_with_edges(adj)
        got = ref.spmm_general(adj.indptr, adj.indices, adj.data + np.float32(0.5), feat, msg, "max")
        assert np.array_equal(got[rows], np.maximum.reduceat(terms, adj.indptr[rows], axis=0))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_generalised_sddmm_against_numpy(op):
    coo = reference_test_matrix("coo", seed=2)
    rng = np.random.default_rng(6)
    src = rng.standard_normal((coo.shape[1], 24), dtype=np.float32)
    dst = rng.standard_normal((coo.shape[0], 24), dtype=np.float32) + np.float32(3.0)
    a, b = src[coo.col], dst[coo.row]
    want = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op]        # one rounded operation each
    assert np.array_equal(ref.sddmm_general(coo.row, coo.col, src, dst, op), want)


def test_edge_softmax_against_scipy_and_its_invariants():
    import scipy.special
    adj = datasets.config_graph("c4-mini")
    H = 4
    scores = (np.random.default_rng(7).standard_normal((adj.nnz, H)) * 5).astype(np.float32)
    out = ref.edge_softmax(adj.indptr, scores)
    for r in (0, 1, 17, 4242, adj.shape[0] - 1):
        sl = slice(adj.indptr[r], adj.indptr[r + 1])
        np.testing.assert_allclose(out[sl], scipy.special.softmax(scores[sl].astype(np.float64), axis=0), rtol=1e-6)
    rows = _rows_with_edges(adj)
    np.testing.assert_allclose(np.add.reduceat(out.astype(np.float64), adj.indptr[rows], axis=0), 1.0, atol=1e-5)
    shifted = ref.edge_softmax(adj.indptr, scores + np.float32(8.0))          # shift invariance (8 is exact to add)
    np.testing.assert_allclose(shifted, out, rtol=1e-5, atol=1e-9)
    uniform = ref.edge_softmax(adj.indptr, np.zeros((adj.nnz, H), np.float32))
    deg = np.repeat(np.diff(adj.indptr), np.diff(adj.indptr))
    np.testing.assert_allclose(uniform, (1.0 / deg)[:, None].repeat(H, 1), rtol=1e-6)


def _masked_scores():
    """Three rows of 70 edges (longer than one wave step), one head-pair: -inf first, -inf in the middle, all -inf."""
    indptr = np.array([0, 70, 140, 210, 213], dtype=np.int32)
    scores = (np.random.default_rng(23).standard_normal((213, 2)) * 3).astype(np.float32)
    scores[0, :] = -np.inf            # before the row's first finite score
    scores[1, 0] = -np.inf
    scores[70 + 33, :] = -np.inf      # between finite scores
    scores[140:210, 1] = -np.inf      # every score of (row 2, head 1)
    scores[210, 0] = -np.inf          # a short row whose first score is masked
    return indptr, scores


def test_edge_softmax_masked_edges_against_scipy():
    """A score of -inf is a masked edge: weight exactly 0, the others as if it were absent (scipy.special.softmax);
    a row and head with nothing but -inf is 0/0 = NaN there, and in the checker too."""
    import scipy.special
    indptr, scores = _masked_scores()
    with np.errstate(invalid="ignore"):
        out = ref.edge_softmax(indptr, scores)
        for r in range(4):
            sl = slice(indptr[r], indptr[r + 1])
            want = scipy.special.softmax(scores[sl].astype(np.float64), axis=0)
            np.testing.assert_allclose(out[sl], want, rtol=1e-6, equal_nan=True)
    assert out[0, 0] == 0 and out[0, 1] == 0 and out[1, 0] == 0 and out[103, 0] == 0 and out[210, 0] == 0
    assert np.isnan(out[140:210, 1]).all() and np.isfinite(out[140:210, 0]).all()
    assert abs(out[:70, 0].astype(np.float64).sum() - 1) < 1e-6


def test_attention_against_dense_masked_softmax():
    """The composed checker against the textbook dense form: softmax over a row's stored entries of Q K^T, times V
    (float64 einsum on a matrix small enough to densify), with separate and with shared key / value."""
    import scipy.special
    rng = np.random.default_rng(11)
    adj = scipy.sparse.random(37, 53, density=0.15, format="lil", random_state=rng)
    adj[5] = 0
    adj[36] = 0                                                              # rows without entries give zeros
    adj = adj.tocsr()
    adj.sort_indices()
    H, D = 4, 8
    key = rng.standard_normal((53, H, D), dtype=np.float32)
    value = rng.standard_normal((53, H, D), dtype=np.float32)
    query = rng.standard_normal((37, H, D), dtype=np.float32)
    mask = adj.toarray() != 0
    for val in (value, None):
        v = key if val is None else val
        scores = np.einsum("rhd,chd->hrc", query.astype(np.float64), key.astype(np.float64))
        scores = np.where(mask[None], scores, -np.inf)
        with np.errstate(invalid="ignore"):
            weights = np.nan_to_num(scipy.special.softmax(scores, axis=2))    # rows without entries: all zero
        want = np.einsum("hrc,chd->rhd", weights, v.astype(np.float64))
        got = ref.attention_mh(adj.indptr, adj.indices, key, query, val)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    assert (np.diff(adj.indptr) == 0).any() and not got[np.diff(adj.indptr) == 0].any()


# ---------------------------------------------------------------- multi-head generalised SpMM, softmax backward
@pytest.mark.parametrize("msg", ["mul", "add", "sub", "div", "copy_u"])
@pytest.mark.parametrize("reduce", ["sum", "max", "min", "mean"])
def test_multi_head_generalised_spmm_against_numpy_reduceat_per_head(msg, reduce):
    """Per head np.add / maximum / minimum.reduceat over exact terms (small integers, weights 1, 2, 4)."""
    adj, _ = _int_case(seed=6)
    H, D = 3, 5
    rng = np.random.default_rng(8)
    feat = rng.integers(-4, 5, (adj.shape[1], H, D)).astype(np.float32)
    w = rng.choice(np.array([1, 2, 4], np.float32), (adj.nnz, H))
    out = ref.spmm_mh_general(adj.indptr, adj.indices, w, feat, msg, reduce)
    rows = _rows_with_edges(adj)
    for h in range(H):
        u, e = feat[adj.indices, h].astype(np.float64), w[:, h].astype(np.float64)[:, None]
        terms = {"mul": u * e, "add": u + e, "sub": u - e, "div": u / e, "copy_u": u}[msg]
        fold = {"sum": np.add, "mean": np.add, "max": np.maximum, "min": np.minimum}[reduce].reduceat(
            terms, adj.indptr[rows], axis=0)
        if reduce == "mean":
            fold = fold / np.diff(adj.indptr)[rows][:, None]
            np.testing.assert_allclose(out[rows, h], fold, rtol=1e-6, atol=0)
        else:
            assert np.array_equal(out[rows, h], fold.astype(np.float32))
    assert np.all(out[np.diff(adj.indptr) == 0] == 0)


def test_multi_head_generalised_spmm_reduces_to_its_relatives(adj_127x255):
    adj = adj_127x255
    rng = np.random.default_rng(9)
    feat = rng.standard_normal((adj.shape[1], 4, 6), dtype=np.float32)
    w = rng.random((adj.nnz, 4), dtype=np.float32) + np.float32(0.5)
    # (mul, sum) is the multi-head operator of config 5 bit for bit
    assert np.array_equal(ref.spmm_mh_general(adj.indptr, adj.indices, w, feat, "mul", "sum"),
                          ref.spmm_mh(adj.indptr, adj.indices, w, feat))
    # one head is the single-head generalised operator
    for msg, reduce in (("add", "max"), ("div", "mean"), ("sub", "min")):
        one = ref.spmm_mh_general(adj.indptr, adj.indices, w[:, :1].copy(), feat[:, :1].copy(), msg, reduce)
        assert np.array_equal(one[:, 0], ref.spmm_general(adj.indptr, adj.indices, w[:, 0].copy(),
                                                          feat[:, 0].copy(), msg, reduce))
    # heads never mix: head 2 of the 4-head result equals the operator run on head 2 alone
    full = ref.spmm_mh_general(adj.indptr, adj.indices, w, feat, "mul", "max")
    alone = ref.spmm_general(adj.indptr, adj.indices, w[:, 2].copy(), feat[:, 2].copy(), "mul", "max")
    assert np.array_equal(full[:, 2], alone)


def test_edge_softmax_backward_against_torch_autograd_and_identities():
    """The gradient formula against a library routine (torch.softmax's own backward, float64, per row) and what the
    mathematics fixes: the gradients of a row sum to zero (the weights sum to one whatever the scores), and a
    gradient that is constant over a row gives zero."""
    import torch
    adj = datasets.config_graph("c4-mini")
    H = 3
    rng = np.random.default_rng(12)
    scores = (rng.standard_normal((adj.nnz, H)) * 2).astype(np.float32)
    grad = rng.standard_normal((adj.nnz, H)).astype(np.float32)
    weights = ref.edge_softmax(adj.indptr, scores)
    got = ref.edge_softmax_backward(adj.indptr, weights, grad)
    for r in (0, 3, 29, 1000, adj.shape[0] - 1):
        sl = slice(adj.indptr[r], adj.indptr[r + 1])
        s = torch.tensor(scores[sl], dtype=torch.float64, requires_grad=True)
        torch.softmax(s, dim=0).backward(torch.tensor(grad[sl], dtype=torch.float64))
        np.testing.assert_allclose(got[sl], s.grad.numpy(), rtol=2e-5, atol=1e-7)
    rows = _rows_with_edges(adj)
    sums = np.add.reduceat(got.astype(np.float64), adj.indptr[rows], axis=0)
    np.testing.assert_allclose(sums, 0.0, atol=1e-6)
    const = np.repeat(rng.standard_normal((adj.shape[0], H)).astype(np.float32), np.diff(adj.indptr), axis=0)
    np.testing.assert_allclose(ref.edge_softmax_backward(adj.indptr, weights, const), 0.0, atol=1e-6)
    # a wrong sign or a dropped row term would survive neither check; a single-edge row has gradient exactly 0
    single = np.flatnonzero(np.diff(adj.indptr) == 1)
    assert single.size and np.all(got[adj.indptr[single]] == 0)


@pytest.mark.parametrize("shared", [False, True])
def test_attention_backward_against_torch_autograd_of_the_dense_form(shared):
    """All three gradients of the composed attention checker against torch's autograd of the textbook dense form
    softmax(mask(Q K^T)) V in float64 (a matrix small enough to densify; rows without entries included)."""
    import torch
    rng = np.random.default_rng(13)
    adj = scipy.sparse.random(23, 31, density=0.2, format="lil", random_state=rng)
    adj[4] = 0
    adj = adj.tocsr()
    adj.sort_indices()
    H, D = 2, 4
    key = rng.standard_normal((31, H, D), dtype=np.float32)
    value = None if shared else rng.standard_normal((31, H, D), dtype=np.float32)
    query = rng.standard_normal((23, H, D), dtype=np.float32)
    dout = rng.standard_normal((23, H, D), dtype=np.float32)
    d_key, d_query, d_value = ref.attention_mh_backward(adj.indptr, adj.indices, key, query, value, dout)
    k = torch.tensor(key, dtype=torch.float64, requires_grad=True)
    q = torch.tensor(query, dtype=torch.float64, requires_grad=True)
    v = k if shared else torch.tensor(value, dtype=torch.float64, requires_grad=True)
    mask = torch.tensor(adj.toarray() != 0)
    s = torch.einsum("rhd,chd->hrc", q, k).masked_fill(~mask[None], float("-inf"))
    a = torch.nan_to_num(torch.softmax(s, dim=2))                       # rows without entries: all zero
    out = torch.einsum("hrc,chd->rhd", a, v)
    out.backward(torch.tensor(dout, dtype=torch.float64))
    np.testing.assert_allclose(d_key, k.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(d_query, q.grad.numpy(), rtol=1e-4, atol=1e-5)
    if not shared:
        np.testing.assert_allclose(d_value, v.grad.numpy(), rtol=1e-4, atol=1e-5)
    assert not d_query[4].any()
