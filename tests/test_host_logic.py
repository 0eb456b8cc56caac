"""Host-side behaviour of the module layer that needs no GPU: input normalisation,
argument checking, the stand-in placeholder / array types and the data generators."""
import numpy as np
import pytest
import scipy.sparse
import torch

import featgraph_amd
from featgraph_amd import datasets, placeholder
from featgraph_amd.module import VanillaSDDMMhip, VanillaSpMMhip
from featgraph_amd.module import _common as C
from featgraph_amd.module.sddmm import normalize_coo
from featgraph_amd.module.spmm import normalize_csr


def test_placeholder_defaults_follow_te_placeholder():
    p = placeholder((255, 128))
    assert p.shape == (255, 128) and p.dtype == "float32"


def test_normalize_csr_converts_formats_and_keeps_stored_order():
    coo = scipy.sparse.random(20, 30, density=0.2, format="coo", random_state=np.random.default_rng(0))
    indptr, indices, data, shape = normalize_csr(coo)
    ref = coo.tocsr()
    assert shape == (20, 30) and indptr.dtype == np.int32 and indices.dtype == np.int32 and data.dtype == np.float32
    assert np.array_equal(indptr, ref.indptr) and np.array_equal(indices, ref.indices)
    # unsorted, duplicated columns are passed through untouched (op/vanilla_spmm.py:50-53 just adds them)
    raw = scipy.sparse.csr_matrix((np.ones(3), np.array([2, 0, 2]), np.array([0, 3])), shape=(1, 3))
    _, idx, _, _ = normalize_csr(raw)
    assert np.array_equal(idx, [2, 0, 2])


def test_normalize_csr_narrows_int64_and_rejects_bad_structure():
    m = scipy.sparse.csr_matrix((np.ones(2, np.float64), np.array([0, 1], np.int64), np.array([0, 1, 2], np.int64)),
                                shape=(2, 2))
    indptr, indices, data, _ = normalize_csr(m)
    assert indptr.dtype == np.int32 and indices.dtype == np.int32 and data.dtype == np.float32
    bad = scipy.sparse.csr_matrix((2, 2), dtype=np.float32)
    bad.indices = np.array([0, 5], dtype=np.int32)
    bad.data = np.ones(2, dtype=np.float32)
    bad.indptr = np.array([0, 1, 2], dtype=np.int32)
    with pytest.raises(ValueError):
        normalize_csr(bad)
    bad.indices = np.array([0, 1], dtype=np.int32)
    bad.indptr = np.array([0, 2, 1], dtype=np.int32)
    with pytest.raises(ValueError):
        normalize_csr(bad)
    with pytest.raises(TypeError):
        normalize_csr(np.zeros((2, 2)))


def test_normalize_coo_checks_ranges():
    coo = scipy.sparse.random(10, 12, density=0.3, format="csr", random_state=np.random.default_rng(1))
    row, col, shape = normalize_coo(coo)
    assert row.dtype == np.int32 and shape == (10, 12) and row.shape == col.shape == (coo.nnz,)
    bad = scipy.sparse.coo_matrix((10, 12))
    bad.row, bad.col, bad.data = np.array([10], np.int32), np.array([0], np.int32), np.ones(1)
    with pytest.raises(ValueError):
        normalize_coo(bad)


def test_unknown_argument_keys_raise_type_error_like_kwargs_unpacking():
    assert C.check_known_keys(None, ("a",), "x") == {}
    assert C.check_known_keys({"a": 1}, ("a",), "x") == {"a": 1}
    with pytest.raises(TypeError):
        C.check_known_keys({"num_feat_partition": 2}, ("num_feat_partitions",), "compute_args")


def test_index_dtype_rules():
    with pytest.raises(TypeError):
        C.to_int32_index(np.array([0.5]), "indices")
    with pytest.raises(ValueError):
        C.to_int32_index(np.array([2 ** 31], dtype=np.int64), "indices")


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the behaviour on a machine without a GPU")
def test_operators_refuse_to_run_without_a_gpu():
    adj = scipy.sparse.random(10, 12, density=0.3, format="csr", dtype=np.float32)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        VanillaSpMMhip(adj)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        VanillaSDDMMhip(adj)


def test_partition_counts_are_asserted_like_the_reference():
    from featgraph_amd.module.spmm import SpMMbase
    from featgraph_amd.module.sddmm import SDDMMbase
    adj = scipy.sparse.random(10, 12, density=0.3, format="csr", dtype=np.float32)
    with pytest.raises(AssertionError):
        SpMMbase(adj, num_col_partitions=0)
    with pytest.raises(AssertionError):
        SDDMMbase(adj, num_row_partitions=0)
    with pytest.raises(AssertionError):
        SDDMMbase(adj, num_col_partitions=0)


def test_package_does_not_import_the_checker():
    import sys
    import subprocess
    code = "import featgraph_amd, featgraph_amd.module, featgraph_amd.datasets, sys; " \
           "print(any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules))"
    out = subprocess.run([sys.executable, "-c", code], stdout=subprocess.PIPE, text=True, cwd=featgraph_amd.__path__[0] + "/..")
    assert out.stdout.strip() == "False"


def test_c1_graph_is_the_documented_recipe():
    adj = datasets.config_graph("c1")
    deg = np.diff(adj.indptr)
    assert adj.shape == (4096, 4096) and deg.min() >= 8 and deg.max() <= 24
    assert adj.indices.dtype == np.int32 and adj.data.dtype == np.float32
    assert adj.nnz == 65812 and datasets.structure_checksum(adj) == "ea95c0729a79f6e1"
    for r in (0, 17, 4095):
        cols = adj.indices[adj.indptr[r]:adj.indptr[r + 1]]
        assert np.all(np.diff(cols) > 0)


def test_powerlaw_graph_shape_properties():
    adj = datasets.config_graph("c2-mini")
    again = datasets.config_graph("c2-mini")
    assert datasets.structure_checksum(adj) == datasets.structure_checksum(again)
    n = adj.shape[0]
    deg = np.diff(adj.indptr)
    assert deg.min() >= 1 and deg.max() > 5 * deg.mean()            # heavy tail
    rows = np.repeat(np.arange(n), deg)
    key = rows.astype(np.int64) * n + adj.indices
    assert np.all(np.diff(key) > 0)                                  # sorted, distinct inside every row
    has_self = np.zeros(n, dtype=bool)
    has_self[rows[adj.indices == rows]] = True
    assert has_self.all()                                            # self-loops included
    assert adj.data.min() >= 0 and adj.data.max() < 1


def test_reference_import_paths_resolve_to_this_implementation():
    """`from featgraph.module import ...` / `from featgraph.util import ...` as the reference's callers write them
    (tests/test_module_spmm.py:9, tests/test_module_sddmm.py:9, tests/test_util.py:5)."""
    import featgraph
    from featgraph.module import VanillaSDDMMcuda, VanillaSpMMcuda
    from featgraph.module import VanillaSDDMMhip as S2, VanillaSpMMhip as S1
    from featgraph.util import util_convert_csr_to_dds, util_partition_adj_coo_2d
    assert VanillaSpMMcuda is S1 is VanillaSpMMhip and VanillaSDDMMcuda is S2 is VanillaSDDMMhip
    assert util_convert_csr_to_dds is featgraph_amd.util.util_convert_csr_to_dds
    assert util_partition_adj_coo_2d is featgraph_amd.util.util_partition_adj_coo_2d
    assert featgraph.placeholder is placeholder and featgraph.nd is featgraph_amd.nd


def test_benchmark_commands_take_the_reference_target_spellings():
    """benchmark/bench_vanilla_spmm.py:72-75 passes --target x86 | cuda: cuda is the GPU target here, x86 is refused."""
    from featgraph_amd.benchmark import _common as B
    ap = B.parser("x", "csr")
    for spelling in ("hip", "cuda"):
        assert B.check_target(ap.parse_args(["--synthetic", "c1", "--target", spelling])) == "hip"
    with pytest.raises(SystemExit):
        B.check_target(ap.parse_args(["--synthetic", "c1", "--target", "x86"]))
