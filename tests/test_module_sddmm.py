"""GPU parity tests of the SDDMM modules, through the module layer and the C ABI.

Bar: float32 results within rtol=1e-5 / atol=1e-4 of the CPU restatement (whose
k-order the reference does not pin) and of the float64 closed form; structure
properties (edge order, duplicates, permutations) hold bit for bit.
"""
import numpy as np
import pytest
import scipy.sparse

from conftest import reference_test_matrix
from featgraph_amd import _lib, datasets, nd, placeholder
from featgraph_amd.module import MultiHeadSDDMMhip, VanillaSDDMMhip
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-4


def _run_sddmm(adj, src_np, dst_np, cls=VanillaSDDMMhip, schedule_args=None):
    module = cls(adj)
    module.build([placeholder(src_np.shape), placeholder(dst_np.shape)], {}, schedule_args or {})
    out = module.run([nd.array(src_np, module.ctx), nd.array(dst_np, module.ctx)])
    return out.asnumpy()


@pytest.fixture
def config_guard():
    yield
    _lib.config_set("sddmm.group", 0)
    _lib.config_set("sddmm.batches", 0)
    _lib.config_set("sddmm.block_cols", 0)
    _lib.config_set("sddmm.rows_blocks", 0)
    _lib.config_set("sddmm.rows_wide", 0)
    for key in ("sddmm.blocked", "sddmm.fast", "sddmm.buffer_loads", "sddmm.rows", "sddmm.sorted_copy", "sddmm.regroup",
                "sddmm.xcd", "spmm.pad_rows"):
        _lib.config_set(key, -1)


# the reference's own test on its matrix family (tests/test_module_sddmm.py:44-70)
@pytest.mark.parametrize("num_cuda_blocks", [32, 256])
def test_vanilla_sddmm_hip_like_the_reference_cuda_test(num_cuda_blocks):
    coo = reference_test_matrix("coo", seed=0)
    rng = np.random.default_rng(1)
    src = rng.random((coo.shape[1], 128)).astype("float32")
    dst = rng.random((coo.shape[0], 128)).astype("float32")
    out = _run_sddmm(coo, src, dst, schedule_args={"num_cuda_blocks": num_cuda_blocks})
    lhs, rhs = src[coo.col], dst[coo.row]
    np.testing.assert_allclose((lhs * rhs).sum(axis=-1), out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, ref.sddmm_x86(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(out, ref.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("F", [1, 2, 3, 4, 7, 8, 16, 30, 32, 33, 64, 100, 128, 256, 260, 512, 513])
def test_feature_lengths(F):
    coo = reference_test_matrix("coo", seed=F)
    src, dst = datasets.sddmm_operands(coo, F)
    out = _run_sddmm(coo, src, dst)
    assert out.shape == (coo.nnz,)
    np.testing.assert_allclose(out, ref.sddmm_x86(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


def test_exact_on_integers_and_operand_roles():
    coo = reference_test_matrix("coo", seed=3, shape=(90, 41), density=0.3)
    rng = np.random.default_rng(3)
    src = rng.integers(-8, 9, (41, 64)).astype(np.float32)        # one row per COLUMN
    dst = rng.integers(-8, 9, (90, 64)).astype(np.float32)        # one row per ROW
    want = (src[coo.col].astype(np.int64) * dst[coo.row].astype(np.int64)).sum(-1).astype(np.float32)
    assert np.array_equal(_run_sddmm(coo, src, dst), want)


@pytest.mark.parametrize("F", [32, 64, 128, 512])
def test_powerlaw_graph_row_sorted_and_shuffled(F):
    adj = datasets.config_graph("c2-mini")
    coo = adj.tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    out = _run_sddmm(coo, src, dst)
    np.testing.assert_allclose(out, ref.sddmm_x86(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    perm = np.random.default_rng(4).permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    assert np.array_equal(_run_sddmm(shuffled, src, dst), out[perm])     # edge order is only an order


def test_c1_configuration_and_committed_golden():
    import os
    adj = datasets.config_graph("c1").tocoo()
    src, dst = datasets.sddmm_operands(adj, 64)
    out = _run_sddmm(adj, src, dst)
    np.testing.assert_allclose(out, ref.sddmm_x86(adj.row, adj.col, src, dst), rtol=RTOL, atol=ATOL)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_sddmm_f64.npz"))
    np.testing.assert_allclose(out[gold["edges"]], gold["out_edges"], rtol=RTOL, atol=ATOL)


def test_duplicates_tails_and_empty_edge_lists(config_guard):
    rng = np.random.default_rng(5)
    src = rng.standard_normal((17, 48), dtype=np.float32)
    dst = rng.standard_normal((23, 48), dtype=np.float32)
    for nnz in (1, 63, 64, 65, 255, 257, 1000):
        row = rng.integers(0, 23, nnz).astype(np.int32)
        col = rng.integers(0, 17, nnz).astype(np.int32)
        coo = scipy.sparse.coo_matrix((np.ones(nnz, np.float32), (row, col)), shape=(23, 17))
        out = _run_sddmm(coo, src, dst)
        np.testing.assert_allclose(out, ref.sddmm_x86(row, col, src, dst), rtol=RTOL, atol=ATOL)
        twice = scipy.sparse.coo_matrix((np.ones(2 * nnz, np.float32), (np.tile(row, 2), np.tile(col, 2))), shape=(23, 17))
        assert np.array_equal(_run_sddmm(twice, src, dst), np.tile(out, 2))
        for batches in (1, 3):
            _lib.config_set("sddmm.batches", batches)
            assert np.array_equal(_run_sddmm(coo, src, dst), out)
        _lib.config_set("sddmm.batches", 0)
    empty = scipy.sparse.coo_matrix((23, 17), dtype=np.float32)
    assert _run_sddmm(empty, src, dst).shape == (0,)


def test_swapping_operand_roles_on_the_transpose_gives_the_same_bits():
    coo = reference_test_matrix("coo", seed=6, shape=(50, 70), density=0.2)
    src, dst = datasets.sddmm_operands(coo, 96)
    t = scipy.sparse.coo_matrix((coo.data, (coo.col, coo.row)), shape=(70, 50))     # same edge order, roles swapped
    assert np.array_equal(_run_sddmm(coo, src, dst), _run_sddmm(t, dst, src))


def test_group_sizes_agree_within_rounding(config_guard):
    coo = reference_test_matrix("coo", seed=7)
    src, dst = datasets.sddmm_operands(coo, 64)
    want = ref.sddmm_f64(coo.row, coo.col, src, dst)
    for g in (1, 2, 4, 8, 16):
        _lib.config_set("sddmm.group", g)
        np.testing.assert_allclose(_run_sddmm(coo, src, dst), want, rtol=RTOL, atol=ATOL)


# ---------------------------------------------------------------- column-blocked edge list
@pytest.mark.parametrize("F", [4, 32, 64, 100, 128, 260, 512])
def test_column_blocked_edge_list(config_guard, F):
    adj = datasets.config_graph("c2-mini")
    coo = adj.tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    want = ref.sddmm_x86(coo.row, coo.col, src, dst)
    exact = ref.sddmm_f64(coo.row, coo.col, src, dst)
    _lib.config_set("sddmm.rows", 0)                                 # this graph's list is row-sorted: keep it off the row-run kernel
    _lib.config_set("sddmm.blocked", 0)
    plain = _run_sddmm(coo, src, dst)
    outs = []
    for block_cols in (64, 1000):
        _lib.config_set("sddmm.blocked", 1)
        _lib.config_set("sddmm.block_cols", block_cols)
        module = VanillaSDDMMhip(coo)
        text = module.lower_to_ir([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        assert "column-blocked edge list" in text and "column blocks of %d" % block_cols in text
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        module.out_tvm.tensor.fill_(7.0)                             # stale contents must not leak into the sums
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(out, exact, rtol=RTOL, atol=ATOL)
        outs.append(out)
    assert np.array_equal(outs[0], outs[1])                          # the block size only changes the visiting order
    if F <= 64:
        assert np.array_equal(outs[0], plain)                        # one tile: same summation tree as the plain kernel


@pytest.mark.parametrize("sorted_copy", [0, 1])
def test_column_blocked_edge_list_keeps_the_callers_edge_order(config_guard, sorted_copy):
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    _lib.config_set("sddmm.sorted_copy", sorted_copy)              # 0: the edge-list kernel scatters its results
    coo = datasets.config_graph("c2-mini").tocoo()
    rng = np.random.default_rng(8)
    src = rng.integers(-8, 9, (coo.shape[1], 128)).astype(np.float32)
    dst = rng.integers(-8, 9, (coo.shape[0], 128)).astype(np.float32)
    perm = rng.permutation(coo.nnz)                                   # not row-sorted, with a ragged tail
    perm = perm[:coo.nnz - 37]
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    want = (src[shuffled.col].astype(np.int64) * dst[shuffled.row].astype(np.int64)).sum(-1).astype(np.float32)
    assert np.array_equal(_run_sddmm(shuffled, src, dst), want)      # exact on integers, in the caller's order


def test_column_blocked_falls_back_for_odd_lengths_and_heads(config_guard):
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    coo = datasets.config_graph("c2-mini").tocoo()
    for F, blocked in ((3, False), (30, False), (30, True)):         # below four floats no blocked kernel applies;
        _lib.config_set("sddmm.rows", -1 if blocked else 0)          # at 30 the row-run kernel does, the re-ordered
        src, dst = datasets.sddmm_operands(coo, F)                    # edge list (rows = 0) does not
        module = VanillaSDDMMhip(coo)
        text = module.lower_to_ir([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        assert ("column blocks" in text) == (blocked and F >= 4)
        np.testing.assert_allclose(_run_sddmm(coo, src, dst), ref.sddmm_x86(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    _lib.config_set("sddmm.rows", -1)
    src, dst = datasets.sddmm_operands(coo, (4, 16))
    out = _run_sddmm(coo, src, dst, cls=MultiHeadSDDMMhip)
    np.testing.assert_allclose(out, ref.sddmm_mh(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("shape", [(1, 16), (1, 32), (1, 64), (1, 128), (1, 256), (1, 512), (8, 16), (8, 32), (8, 64),
                                   (3, 128)])
def test_unrolled_kernel_against_the_general_one(config_guard, shape):
    H, D = shape
    coo = datasets.config_graph("c4-mini").tocoo()
    cls = VanillaSDDMMhip if H == 1 else MultiHeadSDDMMhip
    src, dst = datasets.sddmm_operands(coo, D if H == 1 else (H, D))
    want = ref.sddmm_mh(coo.row, coo.col, src.reshape(-1, H, D), dst.reshape(-1, H, D)).reshape(-1) if H > 1 \
        else ref.sddmm_x86(coo.row, coo.col, src, dst)
    _lib.config_set("sddmm.blocked", 0)
    outs = {}
    for fast, buf in ((0, 0), (1, 0), (1, 1)):
        _lib.config_set("sddmm.fast", fast)
        _lib.config_set("sddmm.buffer_loads", buf)
        out = _run_sddmm(coo, src, dst, cls=cls).reshape(-1)
        np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)
        outs[(fast, buf)] = out
    assert np.array_equal(outs[(1, 0)], outs[(1, 1)])               # addressing mode cannot change a bit
    if D <= 64:
        assert np.array_equal(outs[(0, 0)], outs[(1, 0)])           # one step per lane: same summation tree


# ---------------------------------------------------------------- row runs of a row-sorted edge list
def _describe(module, src, dst):
    return module.lower_to_ir([placeholder(src.shape), placeholder(dst.shape)], {}, {})


@pytest.mark.parametrize("F", [4, 32, 64, 68, 100, 128, 260, 512])
def test_row_runs_of_a_row_sorted_list(config_guard, F):
    coo = datasets.config_graph("c2-mini").tocoo()                   # derived from CSR: rows ascend, columns ascend within a row
    src, dst = datasets.sddmm_operands(coo, F)
    want = ref.sddmm_x86(coo.row, coo.col, src, dst)
    exact = ref.sddmm_f64(coo.row, coo.col, src, dst)
    _lib.config_set("sddmm.blocked", 1)
    outs = []
    for block_cols, grid in ((64, 0), (1000, 0), (1000, 3)):
        _lib.config_set("sddmm.block_cols", block_cols)
        _lib.config_set("sddmm.rows_blocks", grid)                   # 3 workgroups: every wave walks many runs
        module = VanillaSDDMMhip(coo)
        text = _describe(module, src, dst)
        assert "row runs" in text and "column blocks of %d" % block_cols in text
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        module.out_tvm.tensor.fill_(7.0)                             # stale contents must not leak into the sums
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)
        np.testing.assert_allclose(out, exact, rtol=RTOL, atol=ATOL)
        outs.append(out)
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[1], outs[2])
    _lib.config_set("sddmm.rows", 0)                                 # same tiles, same summation tree as the re-ordered list
    module = VanillaSDDMMhip(coo)
    assert "column-blocked edge list" in _describe(module, src, dst)
    assert np.array_equal(_run_sddmm(coo, src, dst), outs[0])


@pytest.mark.parametrize("F", [5, 6, 7, 30, 31, 62, 63, 65, 66, 70, 127, 129, 130, 131, 250, 258])
def test_row_runs_when_the_row_end_cuts_a_lanes_piece(config_guard, F):
    """Feature lengths that are not a multiple of four floats: the lane whose 16-byte piece the row's end cuts reads
    the four floats that end there and leaves its neighbour's floats out of its sum (also when only one to three
    floats are left for the last tile, where that piece begins in the tile before).  Small integers make every
    summation order exact, so a float counted twice or left out shows as a wrong integer."""
    coo = datasets.config_graph("c2-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    _lib.config_set("sddmm.blocked", 1)
    for block_cols, wide in ((700, 1), (700, 2), (64, 2)):
        _lib.config_set("sddmm.block_cols", block_cols)
        _lib.config_set("sddmm.rows_wide", wide)
        module = VanillaSDDMMhip(coo)
        assert "row runs" in _describe(module, src, dst)
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        module.out_tvm.tensor.fill_(7.0)
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        np.testing.assert_allclose(out, ref.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
        isrc, idst = np.rint(src * 2), np.rint(dst * 2)
        got = module.run([nd.array(isrc, module.ctx), nd.array(idst, module.ctx)]).asnumpy()
        assert np.array_equal(got, ref.sddmm_f64(coo.row, coo.col, isrc, idst).astype(np.float32))


def test_feature_rows_that_are_not_a_multiple_of_a_cache_line_are_gathered_from_padded_copies(config_guard):
    """VanillaSDDMMhip copies both feature matrices to rows of a multiple of 32 floats at every run when the length
    is beyond 64 floats and not one (fg_sddmm_coo_plan_pitched_f32): the same bits as without the copies, also for
    the second run's operands, for a list in any order, and when the row-run kernel is switched off after build."""
    csr = datasets.config_graph("c2-mini").tocsr()
    coo = csr.tocoo()
    perm = np.random.default_rng(8).permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 700)
    for adj in (coo, shuffled):
        for F, pitch in ((90, 96), (172, 192), (136, 160), (96, 0), (40, 0), (65, 0), (100, 0), (130, 0)):
            src, dst = datasets.sddmm_operands(adj, F)
            ph = [placeholder(src.shape), placeholder(dst.shape)]
            _lib.config_set("spmm.pad_rows", 0)
            plain = VanillaSDDMMhip(adj)
            assert "pitch of" not in plain.lower_to_ir(ph, {}, {})
            plain.build(ph, {}, {})
            _lib.config_set("spmm.pad_rows", -1)
            module = VanillaSDDMMhip(adj)
            text = module.lower_to_ir(ph, {}, {})
            assert ("pitch of %d floats" % pitch in text) if pitch else ("pitch of" not in text), text
            module.build(ph, {}, {})
            for scale in (1.0, -0.5):
                a, b = nd.array(src * np.float32(scale), module.ctx), nd.array(dst, module.ctx)
                module.out_tvm.tensor.fill_(7.0)
                assert np.array_equal(module.run([a, b]).asnumpy(), plain.run([a, b]).asnumpy()), (F, scale)
            np.testing.assert_allclose(module.run([a, b]).asnumpy(), ref.sddmm_f64(adj.row, adj.col, src * np.float32(-0.5), dst),
                                       rtol=RTOL, atol=ATOL)
            _lib.config_set("sddmm.rows", 0)              # after build: the pitched call is refused, the plain one runs
            np.testing.assert_allclose(module.run([a, b]).asnumpy(), ref.sddmm_f64(adj.row, adj.col, src * np.float32(-0.5), dst),
                                       rtol=RTOL, atol=ATOL)
            _lib.config_set("sddmm.rows", -1)


@pytest.mark.parametrize("F", [128, 132, 192, 200, 260, 512])
def test_row_runs_with_tiles_of_128_floats(config_guard, F):
    """Feature rows of 128 floats and more go through 128-float tiles (two 16-byte pieces per lane), the rest of a
    row through narrower ones; same results as 64-float tiles within the tolerance (the summation tree differs)."""
    coo = datasets.config_graph("c2-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    exact = ref.sddmm_f64(coo.row, coo.col, src, dst)
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 700)
    outs = {}
    for wide in (1, 2):
        _lib.config_set("sddmm.rows_wide", wide)
        module = VanillaSDDMMhip(coo)
        text = _describe(module, src, dst)
        assert "row runs" in text and "tile=%d floats" % (64 * wide) in text
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        module.out_tvm.tensor.fill_(7.0)
        outs[wide] = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        np.testing.assert_allclose(outs[wide], exact, rtol=RTOL, atol=ATOL)
    isrc, idst = np.rint(src * 2), np.rint(dst * 2)                  # small integers: every order gives the same sum
    _lib.config_set("sddmm.rows_wide", 2)
    assert np.array_equal(_run_sddmm(coo, isrc, idst), ref.sddmm_f64(coo.row, coo.col, isrc, idst).astype(np.float32))


@pytest.mark.parametrize("F", [64, 128, 200])
def test_default_plan_of_a_matrix_wider_than_one_column_block(config_guard, F):
    """40,000 columns: the library sizes the blocks itself (three of the default width, each cut in two), and
    feature rows of 128 floats and more take 128-float tiles over passes of one block."""
    adj = datasets.powerlaw_csr(40000, 60.0, 0.9, 2000, seed=3)
    coo = adj.tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    module = VanillaSDDMMhip(coo)
    text = _describe(module, src, dst)
    assert "row runs" in text and ("tile=128 floats" in text) == (F >= 128), text
    assert ("%d column blocks" % (6 if F >= 128 else 3)) in text, text
    module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    np.testing.assert_allclose(out, ref.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


def test_which_lists_take_the_row_run_kernel(config_guard):
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    coo = datasets.config_graph("c2-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, 64)
    assert "row runs" in _describe(VanillaSDDMMhip(coo), src, dst)
    rng = np.random.default_rng(9)
    perm = rng.permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    # a list in any other order runs the same kernel over a sorted copy ...
    text = _describe(VanillaSDDMMhip(shuffled), src, dst)
    assert "row runs" in text and "sorted by row and column" in text
    _lib.config_set("sddmm.sorted_copy", 0)                          # ... or, without one, the re-ordered edge list
    assert "column-blocked edge list" in _describe(VanillaSDDMMhip(shuffled), src, dst)
    _lib.config_set("sddmm.sorted_copy", -1)
    # rows ascend but the columns inside a row do not: runs of one column block are no longer contiguous
    order = np.lexsort((rng.random(coo.nnz), coo.row))
    ragged = scipy.sparse.coo_matrix((coo.data[order], (coo.row[order], coo.col[order])), shape=coo.shape)
    assert np.all(np.diff(ragged.row) >= 0) and np.any(np.diff(ragged.col)[np.diff(ragged.row) == 0] < 0)
    assert "sorted by row and column" in _describe(VanillaSDDMMhip(ragged), src, dst)
    _lib.config_set("sddmm.sorted_copy", 0)
    assert "column-blocked edge list" in _describe(VanillaSDDMMhip(ragged), src, dst)
    _lib.config_set("sddmm.sorted_copy", -1)
    base = _run_sddmm(coo, src, dst)
    inv = np.empty_like(order)
    inv[order] = np.arange(coo.nnz)
    assert np.array_equal(_run_sddmm(ragged, src, dst)[inv], base)
    # 30 floats: the row's end cuts a lane's piece, which the row-run kernel moves back and masks; below four
    # floats it does not apply
    src30, dst30 = datasets.sddmm_operands(coo, 30)
    assert "row runs" in _describe(VanillaSDDMMhip(coo), src30, dst30)
    src3, dst3 = datasets.sddmm_operands(coo, 3)
    assert "row runs" not in _describe(VanillaSDDMMhip(coo), src3, dst3)


@pytest.mark.parametrize("F,block_cols", [(64, 500), (32, 300), (256, 700), (64, 1000)])
def test_passes_pinned_to_the_dies_change_no_bit(config_guard, F, block_cols):
    """With eight passes or more the row-run kernel numbers its workgroups so that each die keeps to its own
    passes (12, 20, 9 and 6 passes here: whole rounds of eight, a partial last round, and too few to pin): the
    same runs by the same code, so the results equal those of the pass-by-pass numbering bit for bit."""
    coo = datasets.config_graph("c2-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, F)
    _lib.config_set("sddmm.block_cols", block_cols)
    _lib.config_set("sddmm.xcd", 1)
    pinned = _run_sddmm(coo, src, dst)
    _lib.config_set("sddmm.xcd", 0)
    assert np.array_equal(_run_sddmm(coo, src, dst), pinned)
    np.testing.assert_allclose(pinned, ref.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("regroup", [1, 0])
@pytest.mark.parametrize("F", [16, 32, 64, 128, 260, 512])
def test_sorted_copy_of_a_list_in_any_order(config_guard, F, regroup):
    """A shuffled list with edges listed twice and rows without edges: the plan sorts a copy by (row, column), the
    row-run kernel works on the copy and the results return to the caller's positions, through two block-local
    permutations or (regroup = 0) one gather.  Same kernel, same tiles, same runs as for the sorted list, so the
    results are the sorted list's bit for bit."""
    _lib.config_set("sddmm.block_cols", 700)
    _lib.config_set("sddmm.regroup", regroup)
    csr = datasets.config_graph("c2-mini").tocsr()
    csr = scipy.sparse.vstack([csr[:100], scipy.sparse.csr_matrix((3, csr.shape[1]), dtype=csr.dtype), csr[100:]]).tocsr()
    coo = csr.tocoo()
    rng = np.random.default_rng(F)
    twice = rng.integers(0, coo.nnz, 5000)
    order = np.lexsort((np.concatenate([coo.col, coo.col[twice]]), np.concatenate([coo.row, coo.row[twice]])))
    row = np.concatenate([coo.row, coo.row[twice]])[order]
    col = np.concatenate([coo.col, coo.col[twice]])[order]
    base = scipy.sparse.coo_matrix((np.ones(len(row), np.float32), (row, col)), shape=coo.shape)
    perm = rng.permutation(len(row))
    shuffled = scipy.sparse.coo_matrix((base.data[perm], (row[perm], col[perm])), shape=coo.shape)
    src, dst = datasets.sddmm_operands(base, F)
    text = _describe(VanillaSDDMMhip(shuffled), src, dst)
    assert "sorted by row and column" in text
    module = VanillaSDDMMhip(shuffled)
    module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
    module.out_tvm.tensor.fill_(7.0)
    ins = [nd.array(src, module.ctx), nd.array(dst, module.ctx)]
    out = module.run(ins).asnumpy()
    assert np.array_equal(out, _run_sddmm(base, src, dst)[perm])
    np.testing.assert_allclose(out, ref.sddmm_f64(shuffled.row, shuffled.col, src, dst), rtol=RTOL, atol=ATOL)
    assert np.array_equal(module.run(ins).asnumpy(), out)           # the plan's scratch carries nothing between calls
    # through the C ABI into an output that is 4-byte but not 16-byte aligned
    import torch
    room = torch.full((len(row) + 1,), 7.0, dtype=torch.float32, device=module.ctx)
    stream = torch.cuda.current_stream(module.ctx).cuda_stream
    _lib.check(_lib.lib().fg_sddmm_coo_plan_f32(module._plan, ins[0].tensor.data_ptr(), ins[1].tensor.data_ptr(),
                                                room.data_ptr() + 4, 1, F, stream))
    assert np.array_equal(room[1:].cpu().numpy(), out) and float(room[0]) == 7.0


@pytest.mark.parametrize("nnz", [1, 3, 5, 32767, 32768, 32769, 65539])
def test_sorted_copy_sizes_around_the_regrouping_block(config_guard, nnz):
    """Lists of one edge, fewer than four, and one off either side of the 32768-element blocks that the results
    are regrouped in; exact on integer operands."""
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 40)
    rng = np.random.default_rng(nnz)
    n_rows, n_cols, F = 300, 257, 64
    row = rng.integers(0, n_rows, nnz).astype(np.int32)
    col = rng.integers(0, n_cols, nnz).astype(np.int32)
    row[0], row[-1] = n_rows - 1, 0                                   # never row-sorted, except the list of one edge
    coo = scipy.sparse.coo_matrix((np.ones(nnz, np.float32), (row, col)), shape=(n_rows, n_cols))
    src = rng.integers(-8, 9, (n_cols, F)).astype(np.float32)
    dst = rng.integers(-8, 9, (n_rows, F)).astype(np.float32)
    if nnz > 1:
        assert "sorted by row and column" in _describe(VanillaSDDMMhip(coo), src, dst)
    want = (src[col].astype(np.int64) * dst[row].astype(np.int64)).sum(-1).astype(np.float32)
    assert np.array_equal(_run_sddmm(coo, src, dst), want)


def test_row_runs_on_awkward_structures(config_guard):
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 128)
    rng = np.random.default_rng(10)
    n_rows, n_cols = 70, 700
    dense = np.zeros((n_rows, n_cols), dtype=bool)
    dense[5] = True                                                  # 128 edges in every block: runs longer than a wave
    dense[6, :130] = True                                            # 128 + 2
    dense[7, 127:129] = True                                         # one edge on each side of a block border
    dense[20:40] = rng.random((20, n_cols)) < 0.03
    dense[69, 699] = True                                            # rows 0-4, 8-19 and 40-68 stay empty
    csr = scipy.sparse.csr_matrix(dense.astype(np.float32))
    coo = csr.tocoo()
    dup = scipy.sparse.coo_matrix((np.ones(2 * coo.nnz, np.float32), (np.repeat(coo.row, 2), np.repeat(coo.col, 2))),
                                  shape=coo.shape)                   # every edge twice, still sorted
    for F in (64, 96, 200):
        src = rng.integers(-8, 9, (n_cols, F)).astype(np.float32)
        dst = rng.integers(-8, 9, (n_rows, F)).astype(np.float32)
        for adj in (coo, dup):
            module = VanillaSDDMMhip(adj)
            assert "row runs" in _describe(module, src, dst)
            want = (src[adj.col].astype(np.int64) * dst[adj.row].astype(np.int64)).sum(-1).astype(np.float32)
            assert np.array_equal(_run_sddmm(adj, src, dst), want)   # exact on integers
    one = scipy.sparse.coo_matrix((np.ones(1, np.float32), ([69], [3])), shape=(n_rows, n_cols))
    src, dst = datasets.sddmm_operands(one, 64)
    np.testing.assert_allclose(_run_sddmm(one, src, dst), ref.sddmm_f64(one.row, one.col, src, dst), rtol=RTOL, atol=ATOL)


# the reference's partitioned x86 test (tests/test_module_sddmm.py:16-41) with its own parameter triples
# (feat_len 128; num_feat_partitions, num_row_partitions, num_col_partitions) = (1,1,1), (4,1,1), (4,4,4), and two more
@pytest.mark.parametrize("num_feat_partitions,num_row_partitions,num_col_partitions",
                         [(1, 1, 1), (4, 1, 1), (4, 4, 4), (1, 4, 4), (8, 1, 7)])
def test_partition_arguments_like_the_reference_x86_test(num_feat_partitions, num_row_partitions, num_col_partitions):
    coo = reference_test_matrix("coo", seed=0)
    rng = np.random.default_rng(1)
    src = rng.random((coo.shape[1], 128)).astype("float32")
    dst = rng.random((coo.shape[0], 128)).astype("float32")
    module = VanillaSDDMMhip(coo, num_row_partitions, num_col_partitions)
    compute_args = {"num_feat_partitions": num_feat_partitions}
    schedule_args = {"num_feat_partitions": num_feat_partitions}
    module.build([placeholder(src.shape), placeholder(dst.shape)], compute_args, schedule_args)
    text = module.lower_to_ir([placeholder(src.shape), placeholder(dst.shape)], compute_args, schedule_args)
    assert ("%d column blocks" % num_col_partitions in text) == (num_col_partitions > 1)
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    if num_row_partitions != 1 or num_col_partitions != 1:
        out = out[module.edge_mapping]
    np.testing.assert_allclose((src[coo.col] * dst[coo.row]).sum(axis=-1), out, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(out, ref.sddmm_x86(coo.row, coo.col, src, dst, num_feat_partitions), rtol=RTOL, atol=ATOL)


def test_module_surface(adj_127x255):
    coo = adj_127x255.tocoo()
    module = VanillaSDDMMhip(coo)
    assert module.target == "hip"
    with pytest.raises(AssertionError):
        module.edge_mapping                                           # module/sddmm.py:155-156: no partitioning asked for
    with pytest.raises(ValueError):                                   # 8 floats do not split into 3 tiles
        module.build([placeholder((coo.shape[1], 8)), placeholder((coo.shape[0], 8))], {"num_feat_partitions": 3}, {})
    with pytest.raises(AssertionError):
        module.build([placeholder((coo.shape[1], 8)), placeholder((coo.shape[0], 16))], {}, {})
    module.build([placeholder((coo.shape[1], 8)), placeholder((coo.shape[0], 8))], {}, {})
    assert np.all(module.out_tvm.asnumpy() == 0) and module.out_tvm.shape == (coo.nnz,)
    src, dst = datasets.sddmm_operands(coo, 8)
    a = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)])
    b = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)])
    assert a is b is module.out_tvm
    t = module.measure_average_time([nd.array(src, module.ctx), nd.array(dst, module.ctx)], 3)
    assert isinstance(t, float) and 0 < t < 1.0
    with pytest.raises(ValueError):
        module.run([nd.array(dst, module.ctx), nd.array(src, module.ctx)])              # roles swapped: shapes differ


# ---------------------------------------------------------------- multi-head
@pytest.mark.parametrize("H,D", [(8, 16), (8, 32), (8, 64), (3, 5), (2, 130), (1, 64), (5, 4)])
def test_multihead_sddmm_matches_closed_form(H, D):
    coo = datasets.config_graph("c4-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, (H, D))
    out = _run_sddmm(coo, src, dst, cls=MultiHeadSDDMMhip)
    assert out.shape == (coo.nnz, H)
    np.testing.assert_allclose(out, ref.sddmm_mh(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    want = np.einsum("ehd,ehd->eh", src[coo.col].astype(np.float64), dst[coo.row].astype(np.float64))
    np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)


def test_multihead_sddmm_with_one_head_is_the_vanilla_kernel():
    coo = datasets.config_graph("c4-mini").tocoo()
    src, dst = datasets.sddmm_operands(coo, (1, 64))
    mh = _run_sddmm(coo, src, dst, cls=MultiHeadSDDMMhip)
    assert np.array_equal(mh[:, 0], _run_sddmm(coo, src[:, 0], dst[:, 0]))


def test_each_head_is_a_vanilla_sddmm_on_its_slice():
    coo = datasets.config_graph("c4-mini").tocoo()
    H, D = 8, 64
    src, dst = datasets.sddmm_operands(coo, (H, D))
    mh = _run_sddmm(coo, src, dst, cls=MultiHeadSDDMMhip)
    for h in (0, 5):
        one = _run_sddmm(coo, np.ascontiguousarray(src[:, h]), np.ascontiguousarray(dst[:, h]))
        assert np.array_equal(mh[:, h], one)


# ---------------------------------------------------------------- seeded random structures, default kernel choice
@pytest.mark.parametrize("seed", range(10))
def test_random_structures_under_random_schedules(config_guard, seed):
    rng = np.random.default_rng(2000 + seed)
    n_rows, n_cols = int(rng.integers(1, 400)), int(rng.integers(1, 3000))
    dens = float(rng.choice([0.002, 0.02, 0.2]))
    mask = rng.random((n_rows, n_cols)) < dens
    mask[rng.integers(0, n_rows, 2)] |= rng.random((2, n_cols)) < 0.8          # two long rows
    coo = scipy.sparse.csr_matrix(mask.astype(np.float32)).tocoo()
    if rng.random() < 0.3:                                                     # not row-sorted: the edge-list path
        perm = rng.permutation(coo.nnz)
        coo = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    _lib.config_set("sddmm.blocked", int(rng.integers(0, 2)))
    _lib.config_set("sddmm.block_cols", int(rng.choice([1, 5, 64, 300, 1 << 20])))
    _lib.config_set("sddmm.rows_blocks", int(rng.choice([0, 1, 2])))
    module = VanillaSDDMMhip(coo)
    for F in rng.choice([1, 3, 4, 8, 12, 16, 24, 32, 48, 64, 100, 128, 192, 260], 5, replace=False):
        F = int(F)
        src = rng.integers(-8, 9, (n_cols, F)).astype(np.float32)
        dst = rng.integers(-8, 9, (n_rows, F)).astype(np.float32)
        module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
        module.out_tvm.tensor.fill_(-1.0)
        out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
        want = (src[coo.col].astype(np.int64) * dst[coo.row].astype(np.int64)).sum(-1).astype(np.float32)
        assert np.array_equal(out, want), (seed, F)                            # exact on integers


def test_plans_give_their_device_memory_back(config_guard):
    """Plans of every kind (row-sorted list, sorted copy with its routing, re-ordered edge list; SpMM with its
    re-laid ids) built and destroyed in a loop leave the device's free memory where it was."""
    import gc
    import torch
    from featgraph_amd.module import VanillaSpMMhip
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    adj = datasets.config_graph("c2-mini")
    coo = adj.tocoo()
    perm = np.random.default_rng(3).permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)

    def cycle():
        for sorted_copy in (1, 0):
            _lib.config_set("sddmm.sorted_copy", sorted_copy)
            for m in (coo, shuffled):
                VanillaSDDMMhip(m)
        VanillaSpMMhip(adj)
        gc.collect()
        torch.cuda.synchronize()
        torch.cuda.empty_cache()

    cycle()                                                          # first use: allocator pools, code objects
    free0 = torch.cuda.mem_get_info()[0]
    for _ in range(5):
        cycle()
    assert abs(torch.cuda.mem_get_info()[0] - free0) < (8 << 20)    # a plan here holds tens of megabytes
