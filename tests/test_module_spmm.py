"""GPU parity tests of the SpMM modules, through the module layer and the C ABI.

Bar: float32 results equal the CPU restatement of the reference's x86 loop nest
BIT FOR BIT (the kernel keeps its summation order and rounding), which implies
the stated tolerance rtol=1e-5 / atol=1e-4; scipy's csr.dot is checked as the
reference's own tests do (tests/test_module_spmm.py:29-30, rtol=atol=1e-4).
"""
import numpy as np
import pytest
import scipy.sparse

from conftest import reference_test_matrix
from featgraph_amd import _lib, datasets, nd, placeholder
from featgraph_amd.module import MultiHeadSpMMhip, VanillaSpMMhip
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-4   # the tolerance the project states for float32 results


def _run_spmm(adj, feat_np, compute_args=None, schedule_args=None):
    module = VanillaSpMMhip(adj)
    SrcFeat = placeholder((adj.shape[1], feat_np.shape[1]))
    module.build([SrcFeat], compute_args or {}, schedule_args or {})
    src_feat = nd.array(feat_np, module.ctx)
    return module.run([src_feat]).asnumpy()


def _oracle(adj, feat_np, P=1):
    csr = adj.tocsr() if adj.format != "csr" else adj
    return ref.spmm_csr_x86(csr.indptr, csr.indices, csr.data.astype(np.float32), feat_np, P)


@pytest.fixture
def config_guard():
    yield
    for key in ("spmm.vec", "spmm.lpr", "spmm.unroll", "spmm.block_cols", "spmm.pipe_blocks",
                "spmm.multi_blocks", "spmm.multi_long", "spmm.tile_interleave"):
        _lib.config_set(key, 0)
    for key in ("spmm.sorted", "spmm.blocked", "spmm.pipeline",
                "spmm.buffer_loads", "spmm.multi", "spmm.relay", "spmm.pad_rows"):
        _lib.config_set(key, -1)


# the reference's own test, on its matrix family (tests/test_module_spmm.py:37-59)
@pytest.mark.parametrize("num_threads_per_cuda_block", [32, 128, None])
def test_vanilla_spmm_hip_like_the_reference_cuda_test(adj_127x255, num_threads_per_cuda_block):
    adj = adj_127x255
    feat = np.random.default_rng(1).random((adj.shape[1], 128)).astype("float32")
    out = _run_spmm(adj, feat, {}, {"num_threads_per_cuda_block": num_threads_per_cuda_block})
    np.testing.assert_allclose(adj.dot(feat), out, rtol=1e-4, atol=1e-4)
    assert np.array_equal(out, _oracle(adj, feat))


# its x86 test's partition arguments (tests/test_module_spmm.py:16-34): (feat_len, num_col_partitions, num_feat_partitions)
@pytest.mark.parametrize("num_col_partitions,num_feat_partitions", [(1, 1), (4, 1), (4, 4), (300, 2)])
def test_partition_arguments_like_the_reference_x86_test(adj_127x255, num_col_partitions, num_feat_partitions):
    adj = adj_127x255
    feat = np.random.default_rng(3).random((adj.shape[1], 128)).astype("float32")
    module = VanillaSpMMhip(adj, num_col_partitions)
    module.build([placeholder(feat.shape)], {"num_feat_partitions": num_feat_partitions}, {})
    text = module.lower_to_ir([placeholder(feat.shape)], {"num_feat_partitions": num_feat_partitions}, {})
    assert ("column blocks" in text) == (num_col_partitions > 1)
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    np.testing.assert_allclose(adj.dot(feat), out, rtol=1e-4, atol=1e-4)
    assert np.array_equal(out, _oracle(adj, feat, num_feat_partitions))
    # the reference's DDS nest re-associates the sum per block; the kernel stays within tolerance of it too
    s1_pos, s1_idx, vals = __import__("featgraph_amd").util.util_convert_csr_to_dds(adj, min(num_col_partitions, 8))
    dds = ref.spmm_dds_x86(s1_pos, s1_idx, vals, feat, adj.shape[0], min(num_col_partitions, 8), num_feat_partitions)
    np.testing.assert_allclose(out, dds, rtol=RTOL, atol=ATOL)


# ... and its x86 test's feature-partition arguments (:32-34)
@pytest.mark.parametrize("num_feat_partitions", [1, 4, 8])
def test_feature_partitions_never_change_a_bit(adj_127x255, num_feat_partitions):
    adj = adj_127x255
    feat = np.random.default_rng(2).standard_normal((adj.shape[1], 128), dtype=np.float32)
    out = _run_spmm(adj, feat, {"num_feat_partitions": num_feat_partitions})
    assert np.array_equal(out, _oracle(adj, feat, num_feat_partitions))


@pytest.mark.parametrize("F", [1, 2, 3, 4, 7, 8, 16, 30, 32, 33, 64, 100, 128, 256, 260, 512, 513, 1024])
def test_feature_lengths(adj_127x255, F):
    adj = adj_127x255
    feat = np.random.default_rng(F).standard_normal((adj.shape[1], F), dtype=np.float32)
    assert np.array_equal(_run_spmm(adj, feat), _oracle(adj, feat))


def test_c1_configuration_and_committed_golden():
    import hashlib, os
    adj = datasets.config_graph("c1")
    feat = datasets.spmm_operands(adj, 64)
    out = _run_spmm(adj, feat)
    want = _oracle(adj, feat)
    assert np.array_equal(out, want)
    np.testing.assert_allclose(out, ref.spmm_csr_f64(adj.indptr, adj.indices, adj.data, feat), rtol=RTOL, atol=ATOL)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "c1_spmm.npz"))
    assert hashlib.sha256(out.tobytes()).hexdigest() == str(gold["sha256"])
    assert np.array_equal(out[gold["rows"]], gold["out_rows"])


@pytest.mark.parametrize("F", [32, 64, 128, 512])
def test_powerlaw_graph_with_hub_rows(F):
    adj = datasets.config_graph("c2-mini")
    feat = datasets.spmm_operands(adj, F)
    out = _run_spmm(adj, feat)
    assert np.array_equal(out, _oracle(adj, feat))
    np.testing.assert_allclose(out, _oracle(adj, feat, 4), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("key,values", [("spmm.vec", [1, 2, 4]), ("spmm.lpr", [8, 16, 32, 64]),
                                        ("spmm.unroll", [4, 8, 16]), ("spmm.sorted", [0, 1])])
@pytest.mark.parametrize("F", [64, 200])
def test_every_launch_shape_gives_the_same_bits(config_guard, key, values, F):
    adj = datasets.config_graph("c2-mini")
    feat = datasets.spmm_operands(adj, F)
    want = _oracle(adj, feat)
    for v in values:
        _lib.config_set(key, v)
        assert np.array_equal(_run_spmm(adj, feat), want), "%s=%d" % (key, v)


@pytest.mark.parametrize("vec", [1, 2, 4])
@pytest.mark.parametrize("unroll", [4, 8, 16, 32])
@pytest.mark.parametrize("pipe_blocks", [1, 7, 2048])
def test_pipelined_kernel_variants(config_guard, vec, unroll, pipe_blocks):
    _lib.config_set("spmm.lpr", 64)
    _lib.config_set("spmm.pipeline", 1)
    _lib.config_set("spmm.vec", vec)
    _lib.config_set("spmm.unroll", unroll)
    _lib.config_set("spmm.pipe_blocks", pipe_blocks)
    for name, F in (("c2-mini", 200), ("c4-mini", 64), ("c1", 64)):
        adj = datasets.config_graph(name)
        feat = datasets.spmm_operands(adj, F)
        module = VanillaSpMMhip(adj)
        assert "pipelined" in module.lower_to_ir([placeholder(feat.shape)], {}, {})
        module.build([placeholder(feat.shape)], {}, {})
        assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), _oracle(adj, feat)), name


def test_pipelined_kernel_without_buffer_addressing(config_guard):
    _lib.config_set("spmm.lpr", 64)
    _lib.config_set("spmm.pipeline", 1)
    _lib.config_set("spmm.buffer_loads", 0)
    for vec in (1, 4):
        _lib.config_set("spmm.vec", vec)
        adj = datasets.config_graph("c2-mini")
        feat = datasets.spmm_operands(adj, 200)
        assert np.array_equal(_run_spmm(adj, feat), _oracle(adj, feat))


def test_pipelined_kernel_on_degenerate_rows(config_guard):
    _lib.config_set("spmm.lpr", 64)
    _lib.config_set("spmm.pipeline", 1)
    rng = np.random.default_rng(21)
    # rows of length 0, 1, 63, 64, 65, 129 and a long one, fewer rows than waves
    lens = np.array([0, 1, 63, 0, 64, 65, 129, 0, 0, 1000, 2, 0], dtype=np.int64)
    indptr = np.zeros(len(lens) + 1, dtype=np.int32)
    np.cumsum(lens, out=indptr[1:])
    indices = np.concatenate([np.sort(rng.integers(0, 500, l)) for l in lens]).astype(np.int32)
    vals = rng.random(indptr[-1], dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(len(lens), 500))
    feat = rng.standard_normal((500, 70), dtype=np.float32)
    for blocked, block_cols in ((0, 0), (1, 64)):
        _lib.config_set("spmm.blocked", blocked)
        _lib.config_set("spmm.block_cols", block_cols)
        module = VanillaSpMMhip(adj)
        module.build([placeholder(feat.shape)], {}, {})
        module.out_tvm.tensor.fill_(9.0)
        out = module.run([nd.array(feat, module.ctx)]).asnumpy()
        assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, vals, feat))


def test_summation_order_and_unfused_rounding_on_the_gpu():
    # the two hand-computed cases that pin the oracle (tests/test_oracle.py), now on the kernel
    indptr = np.array([0, 4, 8, 10], dtype=np.int32)
    indices = np.array([0, 1, 2, 3, 3, 2, 1, 0, 4, 5], dtype=np.int32)
    v = np.float32(1 + 2.0 ** -12)
    vals = np.array([1, 1, 1, 1, 1, 1, 1, 1, 1, v], dtype=np.float32)
    feat = np.array([[1e8], [1.0], [-1e8], [1.0], [-(1 + 2.0 ** -11)], [v]], dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(3, 6))
    out = _run_spmm(adj, np.repeat(feat, 8, axis=1))
    assert np.all(out[0] == 1.0) and np.all(out[1] == 0.0) and np.all(out[2] == 0.0)


def test_empty_rows_empty_matrix_and_odd_structures():
    rng = np.random.default_rng(7)
    # rows without nonzeros become +0 even though the output buffer is reused
    indptr = np.array([0, 0, 3, 3, 3, 5, 5], dtype=np.int32)
    indices = np.array([2, 0, 2, 1, 1], dtype=np.int32)            # unsorted and duplicated columns
    vals = rng.random(5, dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(6, 3))
    feat = rng.standard_normal((3, 20), dtype=np.float32)
    module = VanillaSpMMhip(adj)
    module.build([placeholder((3, 20))], {}, {})
    module.out_tvm.tensor.fill_(7.0)
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, vals, feat))
    assert np.all(out[[0, 2, 3, 5]] == 0) and not np.signbit(out[0]).any()
    empty = scipy.sparse.csr_matrix((5, 4), dtype=np.float32)
    assert np.array_equal(_run_spmm(empty, np.ones((4, 6), dtype=np.float32)), np.zeros((5, 6), dtype=np.float32))


def test_single_long_row_and_wide_matrix():
    rng = np.random.default_rng(8)
    n_cols = 5000
    cols = rng.integers(0, n_cols, 9001).astype(np.int32)
    adj = scipy.sparse.csr_matrix((rng.random(9001, dtype=np.float32), cols, np.array([0, 9001], dtype=np.int32)),
                                  shape=(1, n_cols))
    feat = rng.standard_normal((n_cols, 96), dtype=np.float32)
    out = _run_spmm(adj, feat)
    assert np.array_equal(out, ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat))


def test_row_plan_is_a_stable_sort_by_descending_degree():
    adj = datasets.config_graph("c2-mini")
    module = VanillaSpMMhip(adj)
    order, max_deg = module.row_order()
    deg = np.diff(adj.indptr)
    assert np.array_equal(order, np.argsort(-deg.astype(np.int64), kind="stable").astype(np.int32))
    assert max_deg == deg.max()
    assert "by-descending-degree" in module.lower_to_ir([placeholder((adj.shape[1], 64))], {}, {})


def test_output_is_allocated_once_and_reused(adj_127x255):
    adj = adj_127x255
    module = VanillaSpMMhip(adj)
    module.build([placeholder((adj.shape[1], 32))], {}, {})
    assert module.target == "hip" and module.out_tvm.shape == (adj.shape[0], 32)
    assert np.all(module.out_tvm.asnumpy() == 0)                      # zero-filled at build (module/spmm.py:110-111)
    rng = np.random.default_rng(9)
    a, b = (rng.standard_normal((adj.shape[1], 32), dtype=np.float32) for _ in range(2))
    out1 = module.run([nd.array(a, module.ctx)])
    first = out1.asnumpy()
    out2 = module.run([nd.array(b, module.ctx)])
    assert out1 is out2 is module.out_tvm                            # same object, overwritten (module/spmm.py:161)
    assert np.array_equal(first, _oracle(adj, a)) and np.array_equal(out2.asnumpy(), _oracle(adj, b))
    t = module.measure_average_time([nd.array(b, module.ctx)], 3)
    assert isinstance(t, float) and 0 < t < 1.0                      # seconds
    assert np.array_equal(module.out_tvm.asnumpy(), _oracle(adj, b))


def test_argument_errors(adj_127x255):
    import torch
    adj = adj_127x255
    module = VanillaSpMMhip(adj)
    with pytest.raises(RuntimeError):
        module.run([nd.array(np.zeros((adj.shape[1], 8), np.float32), module.ctx)])      # before build
    with pytest.raises(ValueError):
        module.build([placeholder((adj.shape[1] + 1, 8))], {}, {})
    with pytest.raises(ValueError):
        module.build([placeholder((adj.shape[1], 10))], {"num_feat_partitions": 4}, {})   # op/vanilla_spmm.py:41
    with pytest.raises(TypeError):
        module.build([placeholder((adj.shape[1], 8))], {"feat_partitions": 2}, {})
    module.build([placeholder((adj.shape[1], 8))], {}, {})
    with pytest.raises(ValueError):
        module.run([nd.array(np.zeros((adj.shape[1], 9), np.float32), module.ctx)])
    with pytest.raises(TypeError):
        module.run([nd.array(np.zeros((adj.shape[1], 8), np.float64), module.ctx)])
    with pytest.raises(ValueError):
        module.run([torch.zeros((adj.shape[1], 8), dtype=torch.float32)])                  # host tensor
    with pytest.raises(ValueError):
        module.run([torch.zeros((8, adj.shape[1]), dtype=torch.float32, device=module.ctx).t()])  # not contiguous
    with pytest.raises(TypeError):
        module.run([np.zeros((adj.shape[1], 8), np.float32)])


def test_index_check_entry_point():
    import ctypes, torch
    idx = torch.tensor([0, 5, -1, 9, 10, 3], dtype=torch.int32, device="cuda")
    n_bad = ctypes.c_int64(-1)
    _lib.check(_lib.lib().fg_check_indices(idx.numel(), idx.data_ptr(), 10, ctypes.byref(n_bad), None))
    assert n_bad.value == 2


# ---------------------------------------------------------------- several rows per wave, 16-byte gathers
def _describe(module, feat):
    return module.lower_to_ir([placeholder(feat.shape)], {}, {})


@pytest.mark.parametrize("blocks", [(0, 0), (1, 7), (1, 100), (1, 1500)])
@pytest.mark.parametrize("long_run", [0, 8, 1 << 20])
def test_rows_per_wave_kernel_gives_the_same_bits(config_guard, blocks, long_run):
    adj = datasets.config_graph("c2-mini")
    _lib.config_set("spmm.blocked", blocks[0])
    _lib.config_set("spmm.block_cols", blocks[1])
    _lib.config_set("spmm.multi_long", long_run)       # 8: nearly every run takes the one-workgroup-per-run path; 2^20: none
    module = VanillaSpMMhip(adj)
    # 17, 33, 65 .. 67, 129 .. 131, 193: the last tile holds one to three floats only; 68 .. 96, 200, 602: a rest of up to 32
    # floats behind whole 64-float tiles runs as a narrower tile in launches of its own
    for F in (4, 5, 7, 8, 16, 17, 20, 30, 31, 32, 33, 36, 63, 64, 65, 66, 67, 68, 70, 90, 96, 101, 127, 129, 130, 131, 193, 200, 250, 512, 602):
        feat = datasets.spmm_operands(adj, F)
        text = _describe(module, feat)
        assert "rows-per-wave" in text and (("column blocks of %d" % blocks[1]) in text) == bool(blocks[0])
        module.build([placeholder(feat.shape)], {}, {})
        module.out_tvm.tensor.fill_(3.0)               # stale contents must not leak into the carried sums
        out = module.run([nd.array(feat, module.ctx)]).asnumpy()
        assert np.array_equal(out, _oracle(adj, feat)), "F=%d" % F


@pytest.mark.parametrize("blocked", [0, 1])
def test_feature_rows_that_are_not_a_multiple_of_a_cache_line_are_gathered_from_a_padded_copy(config_guard, blocked):
    """VanillaSpMMhip copies feature rows of more than 64 floats whose length is not a multiple of 32 to rows that
    are, at every run, and gathers from the copy (fg_pad_rows_f32, fg_spmm_csr_pitched_f32): the same bits, for the
    second run's features as for the first's, with the copy switched off, and when the kernel that reads a pitch is
    switched off after build."""
    adj = datasets.config_graph("c2-mini")
    _lib.config_set("spmm.blocked", blocked)
    _lib.config_set("spmm.block_cols", 700 if blocked else 0)
    module = VanillaSpMMhip(adj)
    for F, pitch in ((72, 96), (100, 128), (130, 160), (250, 256), (96, 0), (30, 0), (40, 0), (65, 0)):
        ph = [placeholder((adj.shape[1], F))]
        text = module.lower_to_ir(ph, {}, {})
        assert ("pitch of %d floats" % pitch in text) if pitch else ("pitch of" not in text), text
        module.build(ph, {}, {})
        for seed in (1, 2):
            feat = np.random.default_rng(seed).standard_normal((adj.shape[1], F), dtype=np.float32)
            module.out_tvm.tensor.fill_(5.0)
            assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), _oracle(adj, feat)), (F, seed)
        _lib.config_set("spmm.multi", 0)                  # after build: the pitched call is refused, the plain one runs
        assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), _oracle(adj, feat)), F
        _lib.config_set("spmm.multi", -1)
    _lib.config_set("spmm.pad_rows", 0)
    ph = [placeholder((adj.shape[1], 100))]
    assert "pitch of" not in module.lower_to_ir(ph, {}, {})
    module.build(ph, {}, {})
    feat = datasets.spmm_operands(adj, 100)
    assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), _oracle(adj, feat))
    _lib.config_set("spmm.pad_rows", -1)


def test_rows_per_wave_kernel_only_where_it_applies(config_guard, adj_127x255):
    module = VanillaSpMMhip(adj_127x255)
    assert "rows-per-wave" in _describe(module, np.empty((255, 64), np.float32))
    assert "rows-per-wave" in _describe(module, np.empty((255, 30), np.float32))           # the row's end cuts a lane's four floats
    assert "rows-per-wave" in _describe(module, np.empty((255, 70), np.float32))           # ... in the second tile
    for F in (66, 129):                                # ... and reaches back into the tile before
        assert "rows-per-wave" in _describe(module, np.empty((255, F), np.float32))
    assert "rows-per-wave" not in _describe(module, np.empty((255, 3), np.float32))        # fewer than four floats in all
    assert "rows-per-wave" not in module.lower_to_ir([placeholder((255, 64))], {"num_feat_partitions": 2}, {})
    _lib.config_set("spmm.lpr", 64)                    # an explicit launch shape asks for the other kernels
    assert "rows-per-wave" not in _describe(module, np.empty((255, 64), np.float32))
    _lib.config_set("spmm.lpr", 0)
    _lib.config_set("spmm.multi", 0)
    assert "rows-per-wave" not in _describe(module, np.empty((255, 64), np.float32))
    feat = datasets.spmm_operands(adj_127x255, 64)
    off = _run_spmm(adj_127x255, feat)
    _lib.config_set("spmm.multi", -1)
    assert np.array_equal(_run_spmm(adj_127x255, feat), off)


@pytest.mark.parametrize("long_run", [0, 16, 300])
def test_rows_per_wave_kernel_on_degenerate_rows(config_guard, long_run):
    _lib.config_set("spmm.multi_long", long_run)
    rng = np.random.default_rng(21)
    # rows of length 0, 1, 63, 64, 65, 129, 255..257 and two long ones; fewer rows than one wave's groups at 16 floats
    lens = np.array([0, 1, 63, 0, 64, 65, 129, 0, 0, 1000, 2, 0, 255, 256, 257, 2100], dtype=np.int64)
    indptr = np.zeros(len(lens) + 1, dtype=np.int32)
    np.cumsum(lens, out=indptr[1:])
    indices = np.concatenate([np.sort(rng.integers(0, 500, l)) for l in lens]).astype(np.int32)
    vals = rng.random(indptr[-1], dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(len(lens), 500))
    # relay 0: the records index the CSR arrays instead of a copy of the ids in visiting order
    for blocked, block_cols, grid, buf, relay in ((0, 0, 0, -1, -1), (1, 64, 0, -1, -1), (1, 64, 0, -1, 0),
                                                 (1, 64, 1, 0, -1), (1, 64, 1, 0, 0), (0, 0, 1, 0, -1)):
        _lib.config_set("spmm.relay", relay)
        _lib.config_set("spmm.blocked", blocked)
        _lib.config_set("spmm.block_cols", block_cols)
        _lib.config_set("spmm.multi_blocks", grid)     # one workgroup: every wave walks several items
        _lib.config_set("spmm.buffer_loads", buf)
        module = VanillaSpMMhip(adj)
        for F in (12, 32, 70 * 4):
            feat = rng.standard_normal((500, F), dtype=np.float32)
            assert "rows-per-wave" in _describe(module, feat)
            module.build([placeholder(feat.shape)], {}, {})
            module.out_tvm.tensor.fill_(9.0)
            out = module.run([nd.array(feat, module.ctx)]).asnumpy()
            assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, vals, feat)), (blocked, grid, F)


def test_rows_per_wave_kernel_with_the_callers_partitions(adj_127x255):
    feat = datasets.spmm_operands(adj_127x255, 64)
    want = _oracle(adj_127x255, feat)
    for P in (1, 2, 7):
        module = VanillaSpMMhip(adj_127x255, P)
        text = _describe(module, feat)
        assert "rows-per-wave" in text and (("%d column blocks" % P) in text) == (P > 1)
        module.build([placeholder(feat.shape)], {}, {})
        assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), want)


def test_very_many_partitions_keep_the_bounds_table_only(config_guard):
    # 16 bytes per row and pass would be 324 MB of records for a 36 KB matrix: the plan skips them and the
    # wave-per-row kernels run the caller's 4500 blocks
    rng = np.random.default_rng(41)
    n = 4500
    adj = scipy.sparse.random(n, n, density=1.0 / n, format="csr", dtype=np.float32, random_state=rng)
    adj.sort_indices()
    feat = rng.standard_normal((n, 8)).astype(np.float32)
    module = VanillaSpMMhip(adj, n)
    text = _describe(module, feat)
    assert "rows-per-wave" not in text and "%d column blocks" % n in text
    module.build([placeholder(feat.shape)], {}, {})
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    assert np.array_equal(out, _oracle(adj, feat))


# ---------------------------------------------------------------- column-blocked passes
@pytest.mark.parametrize("block_cols", [7, 100, 1500])
@pytest.mark.parametrize("shape", [(4, 16, 0), (1, 64, 0), (2, 32, 0), (1, 32, 0), (1, 64, 2), (2, 64, 2)])
def test_column_blocked_passes_give_the_same_bits(config_guard, block_cols, shape):
    adj = datasets.config_graph("c2-mini")
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", block_cols)
    vec, lpr, kind = shape                      # kind: 0 row-slot kernel, 2 pipelined kernel
    _lib.config_set("spmm.vec", vec)
    _lib.config_set("spmm.lpr", lpr)
    _lib.config_set("spmm.pipeline", int(kind == 2))
    for F in (64, 200):
        feat = datasets.spmm_operands(adj, F)
        module = VanillaSpMMhip(adj)
        text = module.lower_to_ir([placeholder(feat.shape)], {}, {})
        assert "column blocks of %d" % block_cols in text and ("pipelined" in text) == (kind == 2)
        module.build([placeholder(feat.shape)], {}, {})
        module.out_tvm.tensor.fill_(3.0)      # stale contents must not leak into the carried sums
        out = module.run([nd.array(feat, module.ctx)]).asnumpy()
        assert np.array_equal(out, _oracle(adj, feat)), "F=%d" % F


def test_column_blocks_with_empty_rows_and_blocks(config_guard):
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 4)
    rng = np.random.default_rng(11)
    indptr = np.array([0, 0, 3, 3, 4, 9, 9], dtype=np.int32)
    indices = np.array([0, 1, 30, 17, 2, 3, 3, 20, 31], dtype=np.int32)      # ascending, with a duplicate
    vals = rng.random(9, dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(6, 32))
    feat = rng.standard_normal((32, 24), dtype=np.float32)
    module = VanillaSpMMhip(adj)
    assert "column blocks" in module.lower_to_ir([placeholder(feat.shape)], {}, {})
    module.build([placeholder(feat.shape)], {}, {})
    module.out_tvm.tensor.fill_(5.0)
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, vals, feat))


def test_unsorted_columns_fall_back_to_the_single_pass(config_guard):
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 8)
    rng = np.random.default_rng(12)
    n = 300
    indptr = np.arange(0, 40 * n + 1, 40, dtype=np.int32)
    indices = rng.integers(0, 64, 40 * n).astype(np.int32)                    # not sorted inside rows
    adj = scipy.sparse.csr_matrix((rng.random(40 * n, dtype=np.float32), indices, indptr), shape=(n, 64))
    feat = rng.standard_normal((64, 64), dtype=np.float32)
    module = VanillaSpMMhip(adj)
    assert "1 launch" in module.lower_to_ir([placeholder(feat.shape)], {}, {})
    module.build([placeholder(feat.shape)], {}, {})
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, adj.data, feat))


def test_multihead_column_blocked(config_guard):
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 999)
    adj = datasets.config_graph("c4-mini")
    H, D = 8, 16
    feat = datasets.spmm_operands(adj, (H, D))
    w = datasets.softmax_edge_weights(adj, H)
    assert np.array_equal(_run_mh(adj, feat, w), ref.spmm_mh(adj.indptr, adj.indices, w, feat))


# ---------------------------------------------------------------- degenerate rows, many rows
def test_degenerate_rows_and_many_rows_with_small_column_blocks(config_guard):
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 64)
    rng = np.random.default_rng(31)
    n_rows, n_cols = 150000, 500
    lens = rng.integers(0, 4, n_rows)
    lens[:12] = [0, 1, 63, 0, 64, 65, 129, 0, 0, 1000, 2, 0]
    indptr = np.zeros(n_rows + 1, dtype=np.int32)
    np.cumsum(lens, out=indptr[1:])
    indices = rng.integers(0, n_cols, indptr[-1]).astype(np.int32)
    key = np.repeat(np.arange(n_rows, dtype=np.int64), lens) * n_cols + indices
    key.sort()
    indices = (key % n_cols).astype(np.int32)                       # ascending inside rows, duplicates allowed
    vals = rng.random(indptr[-1], dtype=np.float32)
    adj = scipy.sparse.csr_matrix((vals, indices, indptr), shape=(n_rows, n_cols))
    for F in (70, 64):
        feat = rng.standard_normal((n_cols, F), dtype=np.float32)
        module = VanillaSpMMhip(adj)
        assert "column blocks" in module.lower_to_ir([placeholder(feat.shape)], {}, {})
        module.build([placeholder(feat.shape)], {}, {})
        module.out_tvm.tensor.fill_(9.0)
        out = module.run([nd.array(feat, module.ctx)]).asnumpy()
        assert np.array_equal(out, ref.spmm_csr_x86(indptr, indices, vals, feat)), F


# ---------------------------------------------------------------- multi-head
def _run_mh(adj, feat, w, compute_args=None):
    module = MultiHeadSpMMhip(adj)
    module.build([placeholder(feat.shape), placeholder(w.shape)], compute_args or {}, {})
    return module.run([nd.array(feat, module.ctx), nd.array(w, module.ctx)]).asnumpy()


@pytest.mark.parametrize("H,D", [(8, 64), (8, 16), (3, 5), (1, 64), (2, 130)])
def test_multihead_spmm_matches_closed_form(H, D):
    adj = datasets.config_graph("c4-mini")
    feat = datasets.spmm_operands(adj, (H, D))
    w = datasets.softmax_edge_weights(adj, H)
    out = _run_mh(adj, feat, w)
    assert out.shape == (adj.shape[0], H, D)
    assert np.array_equal(out, ref.spmm_mh(adj.indptr, adj.indices, w, feat))


def test_multihead_spmm_with_one_head_is_the_vanilla_kernel(config_guard):
    adj = datasets.config_graph("c4-mini")
    feat = datasets.spmm_operands(adj, (1, 64))
    vanilla = _run_spmm(adj, feat[:, 0])
    for lpr in (16, 64):
        _lib.config_set("spmm.lpr", lpr)
        assert np.array_equal(_run_mh(adj, feat, adj.data.reshape(-1, 1).copy())[:, 0], vanilla)


@pytest.mark.parametrize("key,values", [("spmm.vec", [1, 2, 4]), ("spmm.lpr", [8, 32, 64]),
                                        ("spmm.pipeline", [0, 1])])
def test_multihead_launch_shapes_give_the_same_bits(config_guard, key, values):
    adj = datasets.config_graph("c4-mini")
    H, D = 8, 32
    feat = datasets.spmm_operands(adj, (H, D))
    w = datasets.softmax_edge_weights(adj, H)
    want = ref.spmm_mh(adj.indptr, adj.indices, w, feat)
    for v in values:
        if key == "spmm.pipeline":
            _lib.config_set("spmm.lpr", 64)
        _lib.config_set(key, v)
        assert np.array_equal(_run_mh(adj, feat, w), want), "%s=%d" % (key, v)


# ---------------------------------------------------------------- seeded random structures, default kernel choice
def _random_csr(rng, n_rows, n_cols, mean_deg, hubs):
    deg = np.minimum(rng.poisson(mean_deg, n_rows), n_cols)
    deg[rng.integers(0, n_rows, hubs)] = np.minimum(rng.integers(n_cols // 2, n_cols + 1, hubs), n_cols)
    deg[rng.random(n_rows) < 0.15] = 0
    indptr = np.zeros(n_rows + 1, dtype=np.int32)
    np.cumsum(deg, out=indptr[1:])
    indices = np.concatenate([np.sort(rng.choice(n_cols, d, replace=False)) for d in deg] + [np.empty(0, np.int64)])
    vals = rng.standard_normal(int(indptr[-1])).astype(np.float32)
    return scipy.sparse.csr_matrix((vals, indices.astype(np.int32), indptr), shape=(n_rows, n_cols))


@pytest.mark.parametrize("seed", range(12))
def test_random_structures_bit_exact_under_random_schedules(config_guard, seed):
    rng = np.random.default_rng(1000 + seed)
    n_rows, n_cols = int(rng.integers(1, 400)), int(rng.integers(1, 3000))
    adj = _random_csr(rng, n_rows, n_cols, float(rng.choice([0.5, 3, 20, 90])), int(rng.integers(0, 4)))
    _lib.config_set("spmm.blocked", int(rng.integers(0, 2)))
    _lib.config_set("spmm.block_cols", int(rng.choice([1, 5, 64, 300, 1 << 20])))
    _lib.config_set("spmm.multi_long", int(rng.choice([0, 4, 64, 700])))
    _lib.config_set("spmm.multi_blocks", int(rng.choice([0, 1, 2])))
    _lib.config_set("spmm.relay", int(seed % 3 != 0))
    module = VanillaSpMMhip(adj)
    for F in rng.choice([1, 3, 4, 5, 8, 12, 16, 24, 30, 32, 48, 64, 65, 67, 100, 128, 129, 192, 250, 260], 7, replace=False):
        feat = rng.standard_normal((n_cols, int(F))).astype(np.float32)
        module.build([placeholder(feat.shape)], {}, {})
        module.out_tvm.tensor.fill_(-1.0)
        out = module.run([nd.array(feat, module.ctx)]).asnumpy()
        assert np.array_equal(out, ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat)), (seed, int(F))


def test_launch_time_keys_may_change_after_the_plan_exists(config_guard):
    """A module built under the defaults keeps giving the same bits when the keys that are read at launch change
    afterwards: only the kernel choice moves."""
    adj = datasets.config_graph("c2-mini")
    feat = datasets.spmm_operands(adj, 64)
    want = _oracle(adj, feat)
    module = VanillaSpMMhip(adj)
    module.build([placeholder(feat.shape)], {}, {})
    x = nd.array(feat, module.ctx)
    seen = set()
    for key, value in (("spmm.multi", 0), ("spmm.blocked", 1), ("spmm.pipeline", 0), ("spmm.sorted", 0),
                       ("spmm.buffer_loads", 0), ("spmm.multi", 1), ("spmm.blocked", 0), ("spmm.unroll", 4)):
        _lib.config_set(key, value)
        seen.add(module.lower_to_ir([placeholder(feat.shape)], {}, {}))
        module.out_tvm.tensor.fill_(2.0)
        assert np.array_equal(module.run([x]).asnumpy(), want), (key, value)
    assert len(seen) >= 4                                  # the description, hence the launch, did change


@pytest.mark.parametrize("interleave", [1, 2])
@pytest.mark.parametrize("F", [128, 192, 256, 260])
def test_tiles_of_one_launch_in_turn_or_one_after_the_other(config_guard, interleave, F):
    """Column-block passes cover every feature tile in one launch; pairs of tiles may alternate workgroup by
    workgroup (even tile counts) or tiles follow one another.  Same bits either way, partial last tile included."""
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 700)
    _lib.config_set("spmm.tile_interleave", interleave)
    adj = datasets.config_graph("c2-mini")
    feat = datasets.spmm_operands(adj, F)
    module = VanillaSpMMhip(adj)
    text = module.lower_to_ir([placeholder(feat.shape)], {}, {})
    n_tiles = F // 64 + (F % 64 > 32)                  # a rest of up to 32 floats runs as a narrower tile of its own
    assert "rows-per-wave" in text and "%d in turn" % (interleave if n_tiles % interleave == 0 else 1) in text
    assert ("the rest of the row as a tile of 16 floats" in text) == (F == 260)
    module.build([placeholder(feat.shape)], {}, {})
    module.out_tvm.tensor.fill_(4.0)
    assert np.array_equal(module.run([nd.array(feat, module.ctx)]).asnumpy(), _oracle(adj, feat))
