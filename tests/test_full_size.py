"""GPU parity at the benchmark's full sizes (the 232,965-vertex / ~114.6M-nonzero graph
and the 2.45M-vertex multi-head graph), against the CPU checker run on the host cores,
plus size-independent properties.  Each test prints what it is about to launch."""
import time

import numpy as np
import pytest

from featgraph_amd import datasets, nd, placeholder
from featgraph_amd.module import MultiHeadSDDMMhip, MultiHeadSpMMhip, VanillaSDDMMhip, VanillaSpMMhip
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-4


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def c2():
    t = time.time()
    adj = datasets.config_graph("c2")
    _say("c2 graph: nnz %d, checksum %s, %.1f s" % (adj.nnz, datasets.structure_checksum(adj), time.time() - t))
    return adj


@pytest.fixture(scope="module")
def c4():
    t = time.time()
    adj = datasets.config_graph("c4")
    _say("c4 graph: nnz %d, checksum %s, %.1f s" % (adj.nnz, datasets.structure_checksum(adj), time.time() - t))
    return adj


def test_generator_gives_the_same_graph_with_and_without_the_gpu_sort():
    cfg = dict(datasets.CONFIGS["c2-mini"])
    cfg.pop("kind")
    a = datasets.powerlaw_csr(use_gpu=True, **cfg)
    b = datasets.powerlaw_csr(use_gpu=False, **cfg)
    assert datasets.structure_checksum(a) == datasets.structure_checksum(b) and np.array_equal(a.data, b.data)


def test_c2_spmm_f64_bit_exact_and_row_coverage(c2):
    adj = c2
    n = adj.shape[0]
    assert n == 232965 and 114.0e6 < adj.nnz < 115.2e6
    _say("SpMM c2 F=64 through VanillaSpMMhip")
    module = VanillaSpMMhip(adj)
    module.build([placeholder((n, 64))], {}, {})
    feat = datasets.spmm_operands(adj, 64)
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    want = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat)
    assert np.array_equal(out, want)                                   # implies rtol 1e-5 / atol 1e-4
    # hub rows against the float64 sum: the float32 sequential sum itself is what limits accuracy there
    exact = ref.spmm_csr_f64(adj.indptr, adj.indices, adj.data, feat)
    deg = np.diff(adj.indptr)
    short = deg <= 2000
    np.testing.assert_allclose(out[short], exact[short], rtol=1e-5, atol=2e-4)
    np.testing.assert_allclose(out, exact, rtol=1e-4, atol=2e-3)
    # property: all-ones values and features turn every output row into its degree, exactly
    ones = VanillaSpMMhip(type(adj)((np.ones(adj.nnz, np.float32), adj.indices, adj.indptr), shape=adj.shape))
    ones.build([placeholder((n, 64))], {}, {})
    got = ones.run([nd.array(np.ones((n, 64), np.float32), ones.ctx)]).asnumpy()
    assert np.array_equal(got, np.repeat(deg.astype(np.float32)[:, None], 64, axis=1))


def test_c2_sddmm_f64_within_tolerance(c2):
    coo = c2.tocoo()
    n = coo.shape[0]
    _say("SDDMM c2 F=64 through VanillaSDDMMhip")
    module = VanillaSDDMMhip(coo)
    module.build([placeholder((n, 64)), placeholder((n, 64))], {}, {})
    src, dst = datasets.sddmm_operands(coo, 64)
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    np.testing.assert_allclose(out, ref.sddmm_f64(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)
    m = 6_000_000   # the strict serial restatement on the head and the tail of the edge list
    for sl in (slice(0, m), slice(coo.nnz - m, coo.nnz)):
        np.testing.assert_allclose(out[sl], ref.sddmm_x86(coo.row[sl], coo.col[sl], src, dst), rtol=RTOL, atol=ATOL)
    # property: unit features make every score equal the feature length
    one = np.ones((n, 64), np.float32)
    got = module.run([nd.array(one, module.ctx), nd.array(one, module.ctx)]).asnumpy()
    assert np.all(got == 64.0)


def test_c4_multihead_sddmm_d16(c4):
    coo = c4.tocoo()
    n = coo.shape[0]
    _say("multi-head SDDMM c4 H=8 D=16 through MultiHeadSDDMMhip")
    module = MultiHeadSDDMMhip(coo)
    module.build([placeholder((n, 8, 16)), placeholder((n, 8, 16))], {}, {})
    src, dst = datasets.sddmm_operands(coo, (8, 16))
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    assert out.shape == (coo.nnz, 8)
    np.testing.assert_allclose(out, ref.sddmm_mh(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


def test_c5_multihead_spmm_d64(c4):
    adj = c4
    n = adj.shape[0]
    _say("multi-head SpMM c5 H=8 D=64 through MultiHeadSpMMhip")
    w = datasets.softmax_edge_weights(adj, 8)
    feat = datasets.spmm_operands(adj, (8, 64))
    module = MultiHeadSpMMhip(adj)
    module.build([placeholder((n, 8, 64)), placeholder(w.shape)], {}, {})
    out = module.run([nd.array(feat, module.ctx), nd.array(w, module.ctx)]).asnumpy()
    want = ref.spmm_mh(adj.indptr, adj.indices, w, feat)
    assert np.array_equal(out, want)


def test_benchmark_commands_run_on_a_small_graph(tmp_path, capsys):
    import scipy.sparse
    from featgraph_amd.benchmark import bench_vanilla_sddmm, bench_vanilla_spmm
    adj = datasets.config_graph("c2-mini")
    path = str(tmp_path / "adj_csr.npz")
    scipy.sparse.save_npz(path, adj)                       # the .npz layout the reference's --dataset flag reads
    args = bench_vanilla_spmm.C.parser("t", "csr").parse_args(["--dataset", path, "--feat-len", "32"])
    loaded = bench_vanilla_spmm.C.load_adjacency(args, "csr")
    assert loaded.format == "csr" and loaded.nnz == adj.nnz
    res = bench_vanilla_spmm.bench_vanilla_spmm_hip(loaded, args.feat_len, 2)
    assert len(res) == 7 * 3 and all(t > 0 for t, _ in res)
    res = bench_vanilla_sddmm.bench_vanilla_sddmm_hip(adj.tocoo(), 32, 2)
    assert len(res) == 7 and all(t > 0 for t, _ in res)
    assert "best:" in capsys.readouterr().out
