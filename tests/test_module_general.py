"""GPU parity of the generalised operators (message / reduce / edge-function slots) and of the SpMM backward,
through the module layer and the C ABI, against the CPU checker (oracle/) and numpy closed forms.

Bars: generalised SpMM bit-exact (the kernel folds each row in CSR order with one rounded operation per step, as
the checker does); elementwise SDDMM bit-exact (one rounded operation per element); the backward inherits the
bars of the two vanilla kernels it is made of.
"""
import numpy as np
import pytest
import scipy.sparse

from conftest import reference_test_matrix
from featgraph_amd import datasets, nd, placeholder
from featgraph_amd.module import (GeneralizedSDDMMhip, GeneralizedSpMMhip, VanillaSDDMMhip, VanillaSpMMGradhip,
                                  VanillaSpMMhip)
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-4
MSGS = ["mul", "add", "sub", "div", "copy_u"]
REDUCES = ["sum", "max", "min", "mean"]


def _run_general_spmm(adj, feat, msg, reduce):
    module = GeneralizedSpMMhip(adj, msg, reduce)
    module.build([placeholder(feat.shape)], {}, {})
    module.out_tvm.tensor.fill_(7.0)                      # every element must be overwritten, empty rows too
    return module.run([nd.array(feat, module.ctx)]).asnumpy()


@pytest.mark.parametrize("msg", MSGS)
@pytest.mark.parametrize("reduce", REDUCES)
def test_every_message_and_reducer_on_the_reference_matrix_family(adj_127x255, msg, reduce):
    adj = adj_127x255.copy()
    adj.data = adj.data + np.float32(0.25)                # keep divisors away from zero
    for F in (128, 5):                                    # float4 lanes; scalar lanes with a partial tile
        feat = np.random.default_rng(F).standard_normal((adj.shape[1], F), dtype=np.float32)
        out = _run_general_spmm(adj, feat, msg, reduce)
        assert np.array_equal(out, ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, msg, reduce)), F


@pytest.mark.parametrize("reduce", REDUCES)
def test_hub_rows_empty_rows_and_unsorted_duplicate_columns(reduce):
    adj = datasets.config_graph("c2-mini")                # rows of up to 3,000 nonzeros
    feat = datasets.spmm_operands(adj, 64)
    for msg in ("mul", "add"):
        out = _run_general_spmm(adj, feat, msg, reduce)
        assert np.array_equal(out, ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, msg, reduce)), msg
    # rows 1 and 3 empty, row 2 with descending and repeated columns: the fold follows the stored order
    raw = scipy.sparse.csr_matrix((np.array([2, 1, 4, 3, 5], np.float32), np.array([3, 1, 1, 0, 2], np.int32),
                                   np.array([0, 1, 1, 4, 4, 5], np.int32)), shape=(5, 4))
    small = np.random.default_rng(9).standard_normal((4, 12), dtype=np.float32)
    out = _run_general_spmm(raw, small, "sub", reduce)
    assert np.array_equal(out, ref.spmm_general(raw.indptr, raw.indices, raw.data, small, "sub", reduce))
    assert np.all(out[[1, 3]] == 0)


@pytest.mark.parametrize("msg", MSGS)
@pytest.mark.parametrize("reduce", REDUCES)
def test_column_block_passes_fold_in_the_same_order(msg, reduce):
    """With column blocks the fold of a row runs pass by pass, its state carried in the output: the same bits as
    the single pass, for blocks so narrow that many (row, pass) runs are empty and rows start in a late pass, with
    rows without nonzeros, and with a not-a-number as a row's first and as a later message."""
    from featgraph_amd import _lib
    adj = datasets.config_graph("c2-mini").tolil()
    adj[5] = 0
    adj[4242] = 0
    adj = adj.tocsr()
    adj.sort_indices()
    adj.data = (adj.data + np.float32(0.25)).astype(np.float32)
    try:
        _lib.config_set("spmm.blocked", 1)
        # 72 floats: a whole 64-float tile and a partial one; 24: one partial 32-float tile; 70 and 30: the row's
        # end cuts a lane's four floats.  Both kernels: the several-rows-per-wave one (also one workgroup per run
        # of 1024 nonzeros and more) and the row-slot one.
        # buffer loads off: the same kernel with 64-bit addresses, as feature matrices of 4 GiB and more take it
        for F, multi, buffer_loads in ((72, -1, -1), (72, 0, -1), (24, -1, -1), (70, -1, -1), (30, -1, -1), (66, -1, -1),
                                       (129, -1, -1), (90, -1, -1), (72, -1, 0), (30, -1, 0)):
            _lib.config_set("spmm.buffer_loads", buffer_loads)
            feat = datasets.spmm_operands(adj, F)
            feat[adj.indices[adj.indptr[7]]] = np.nan         # first message of row 7 (and wherever else the vertex occurs)
            feat[adj.indices[adj.indptr[9] + 3]] = np.nan     # a later message of row 9
            want = ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, msg, reduce)
            _lib.config_set("spmm.general_multi", multi)
            for block_cols in (64, 1500):
                _lib.config_set("spmm.block_cols", block_cols)
                module = GeneralizedSpMMhip(adj, msg, reduce)
                text = module.lower_to_ir([placeholder(feat.shape)], {}, {})
                assert "column blocks" in text and ("rows-per-wave" in text) == (multi != 0)
                module.build([placeholder(feat.shape)], {}, {})
                module.out_tvm.tensor.fill_(7.0)
                out = module.run([nd.array(feat, module.ctx)]).asnumpy()
                assert np.array_equal(out, want, equal_nan=True), (F, multi, block_cols)
                assert not out[5].any() and not out[4242].any()
    finally:
        _lib.config_set("spmm.blocked", -1)
        _lib.config_set("spmm.block_cols", 0)
        _lib.config_set("spmm.general_multi", -1)
        _lib.config_set("spmm.buffer_loads", -1)


def test_mul_sum_is_the_vanilla_kernel_and_max_min_match_numpy(adj_127x255):
    adj = adj_127x255
    feat = np.random.default_rng(2).standard_normal((adj.shape[1], 96), dtype=np.float32)
    vanilla = VanillaSpMMhip(adj)
    vanilla.build([placeholder(feat.shape)], {}, {})
    assert np.array_equal(_run_general_spmm(adj, feat, "mul", "sum"), vanilla.run([nd.array(feat, vanilla.ctx)]).asnumpy())
    rows = np.flatnonzero(np.diff(adj.indptr) > 0)
    terms = feat[adj.indices]                              # copy_u: the terms are the gathered rows themselves
    assert np.array_equal(_run_general_spmm(adj, feat, "copy_u", "max")[rows],
                          np.maximum.reduceat(terms, adj.indptr[rows], axis=0))
    assert np.array_equal(_run_general_spmm(adj, feat, "copy_u", "min")[rows],
                          np.minimum.reduceat(terms, adj.indptr[rows], axis=0))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_elementwise_edge_functions(op):
    coo = reference_test_matrix("coo", seed=4)
    rng = np.random.default_rng(5)
    for F in (128, 6, 1):
        src = rng.standard_normal((coo.shape[1], F), dtype=np.float32)
        dst = rng.standard_normal((coo.shape[0], F), dtype=np.float32) + np.float32(3.0)
        module = GeneralizedSDDMMhip(coo, op)
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        assert out.shape == (coo.nnz, F)
        assert np.array_equal(out, ref.sddmm_general(coo.row, coo.col, src, dst, op)), F
        a, b = src[coo.col], dst[coo.row]
        assert np.array_equal(out, {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op])


def test_dot_edge_function_is_the_vanilla_module():
    coo = reference_test_matrix("coo", seed=4)
    src, dst = datasets.sddmm_operands(coo, 128)
    outs = []
    for module in (GeneralizedSDDMMhip(coo, "dot"), VanillaSDDMMhip(coo)):
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        outs.append(module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy())
    assert outs[0].shape == (coo.nnz,) and np.array_equal(outs[0], outs[1])


def test_elementwise_edge_function_on_a_large_edge_list():
    adj = datasets.config_graph("c4-mini")
    coo = adj.tocoo()
    src, dst = datasets.sddmm_operands(coo, 32)
    module = GeneralizedSDDMMhip(coo, "mul")
    module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    assert np.array_equal(out, src[coo.col] * dst[coo.row])
    # summing the elementwise products over the feature axis is the dot product, up to summation order
    np.testing.assert_allclose(out.astype(np.float64).sum(-1), ref.sddmm_f64(coo.row, coo.col, src, dst),
                               rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_elementwise_edge_functions_over_row_runs(op):
    """A row-sorted list with column blocks takes the row-run schedule (Dst tile in registers, one store per gathered
    Src tile); one rounded operation per element, so the bits are those of the edge-parallel kernel and of numpy.
    Feature lengths: tiles of 16, 32 and 64 floats, a partial last tile, several tiles; 30 is not a multiple of 4
    and a shuffled list has no row runs of its own: both keep the edge-parallel kernel."""
    from featgraph_amd import _lib
    csr = datasets.config_graph("c2-mini").tocsr()
    csr = scipy.sparse.vstack([csr[:50], scipy.sparse.csr_matrix((2, csr.shape[1]), dtype=csr.dtype), csr[50:]]).tocsr()
    coo = csr.tocoo()
    rng = np.random.default_rng(6)
    try:
        _lib.config_set("sddmm.blocked", 1)
        for block_cols in (700, 64):
            _lib.config_set("sddmm.block_cols", block_cols)
            for F in (8, 16, 32, 64, 72, 200, 30):
                src = rng.standard_normal((coo.shape[1], F), dtype=np.float32)
                dst = rng.standard_normal((coo.shape[0], F), dtype=np.float32) + np.float32(3.0)
                module = GeneralizedSDDMMhip(coo, op)
                ph = [placeholder(src.shape), placeholder(dst.shape)]
                assert ("row runs" in module.lower_to_ir(ph, {}, {})) == (F % 4 == 0)
                module.build(ph, {}, {})
                module.out_tvm.tensor.fill_(7.0)                 # every element must be written
                out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
                a, b = src[coo.col], dst[coo.row]
                assert np.array_equal(out, {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op]), (block_cols, F)
        perm = rng.permutation(coo.nnz)
        shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
        src = rng.standard_normal((coo.shape[1], 64), dtype=np.float32)
        dst = rng.standard_normal((coo.shape[0], 64), dtype=np.float32) + np.float32(3.0)
        module = GeneralizedSDDMMhip(shuffled, op)
        ph = [placeholder(src.shape), placeholder(dst.shape)]
        assert "row runs" not in module.lower_to_ir(ph, {}, {})
        module.build(ph, {}, {})
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        assert np.array_equal(out, ref.sddmm_general(shuffled.row, shuffled.col, src, dst, op))
    finally:
        _lib.config_set("sddmm.blocked", -1)
        _lib.config_set("sddmm.block_cols", 0)


def test_bad_operator_names_and_codes():
    from featgraph_amd import _lib
    adj = reference_test_matrix("csr", seed=0)
    with pytest.raises(ValueError):
        GeneralizedSpMMhip(adj, "pow", "sum")
    with pytest.raises(ValueError):
        GeneralizedSpMMhip(adj, "mul", "prod")
    with pytest.raises(ValueError):
        GeneralizedSDDMMhip(adj.tocoo(), "xor")
    L = _lib.lib()
    assert L.fg_sddmm_coo_general_f32(4, 8, 8, 8, 8, 8, 4, 9, None) == -1
    assert L.fg_spmm_csr_general_f32(None, None, None, None, 4, 0, 0, None) == -1


# ---------------------------------------------------------------- backward of vanilla SpMM
@pytest.mark.parametrize("name,F", [("c2-mini", 64), ("c4-mini", 32)])
def test_spmm_backward_is_transpose_spmm_and_sddmm(name, F):
    adj = datasets.config_graph(name)
    n_rows, n_cols = adj.shape
    rng = np.random.default_rng(11)
    x = rng.standard_normal((n_cols, F), dtype=np.float32)
    dout = rng.standard_normal((n_rows, F), dtype=np.float32)
    grad = VanillaSpMMGradhip(adj)
    grad.build([placeholder(x.shape)])
    dx, da = grad.run([nd.array(x, grad.ctx), nd.array(dout, grad.ctx)])
    dx, da = dx.asnumpy(), da.asnumpy()
    t = adj.T.tocsr()
    assert np.array_equal(dx, ref.spmm_csr_x86(t.indptr, t.indices, t.data, dout))        # bit-exact on A^T
    np.testing.assert_allclose(dx, adj.T.astype(np.float64).dot(dout.astype(np.float64)), rtol=1e-4, atol=2e-3)
    coo = adj.tocoo()
    np.testing.assert_allclose(da, ref.sddmm_f64(coo.row, coo.col, x, dout), rtol=RTOL, atol=ATOL)
    # the defining identity of a gradient: <A x, dOut> = <x, A^T dOut> = sum_e vals[e] * dA[e]
    lhs = float((adj.astype(np.float64).dot(x.astype(np.float64)) * dout).sum())
    assert abs(lhs - float((x.astype(np.float64) * dx).sum())) <= 1e-6 * abs(lhs) + 1e-2
    assert abs(lhs - float((adj.data.astype(np.float64) * da).sum())) <= 1e-6 * abs(lhs) + 1e-2


def _random_csr(rng, n_rows, n_cols, mean_deg, hubs):
    deg = np.minimum(rng.poisson(mean_deg, n_rows), n_cols)
    deg[rng.integers(0, n_rows, hubs)] = np.minimum(rng.integers(n_cols // 2, n_cols + 1, hubs), n_cols)
    deg[rng.random(n_rows) < 0.15] = 0
    indptr = np.zeros(n_rows + 1, dtype=np.int32)
    np.cumsum(deg, out=indptr[1:])
    indices = np.concatenate([np.sort(rng.choice(n_cols, d, replace=False)) for d in deg] + [np.empty(0, np.int64)])
    vals = (rng.standard_normal(int(indptr[-1])) + 3.0).astype(np.float32)     # divisors away from zero
    return scipy.sparse.csr_matrix((vals, indices.astype(np.int32), indptr), shape=(n_rows, n_cols))


@pytest.mark.parametrize("seed", range(16))
def test_random_structures_messages_and_reducers_under_random_schedules(seed):
    """Seeded random matrices (empty rows, rows that fill half the columns and more), a random message and reducer,
    random pass widths, long-run thresholds, grid sizes and kernel choice; infinities and a not-a-number among the
    features.  Bit-exact against the checker."""
    from featgraph_amd import _lib
    rng = np.random.default_rng(3000 + seed)
    n_rows, n_cols = int(rng.integers(1, 400)), int(rng.integers(1, 3000))
    adj = _random_csr(rng, n_rows, n_cols, float(rng.choice([0.5, 3, 20, 90])), int(rng.integers(0, 4)))
    keys = {"spmm.blocked": int(rng.integers(0, 2)), "spmm.block_cols": int(rng.choice([1, 5, 64, 300, 1 << 20])),
            "spmm.multi_long": int(rng.choice([0, 4, 64, 700])), "spmm.multi_blocks": int(rng.choice([0, 1, 2])),
            "spmm.relay": int(seed % 3 != 0), "spmm.general_multi": int(seed % 4 != 0)}
    try:
        for k, v in keys.items():
            _lib.config_set(k, v)
        for F in rng.choice([1, 4, 8, 20, 24, 32, 36, 64, 100, 128, 200], 4, replace=False):
            msg, reduce = str(rng.choice(MSGS)), str(rng.choice(REDUCES))
            feat = rng.standard_normal((n_cols, int(F))).astype(np.float32)
            feat[rng.integers(0, n_cols, 3), rng.integers(0, int(F), 3)] = [np.inf, -np.inf, np.nan]
            out = _run_general_spmm(adj, feat, msg, reduce)
            want = ref.spmm_general(adj.indptr, adj.indices, adj.data, feat, msg, reduce)
            assert np.array_equal(out, want, equal_nan=True), (seed, int(F), msg, reduce, keys)
    finally:
        for k in keys:
            _lib.config_set(k, 0 if k in ("spmm.block_cols", "spmm.multi_long", "spmm.multi_blocks") else -1)
