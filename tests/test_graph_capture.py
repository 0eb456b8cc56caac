"""The run paths enqueue kernels and nothing else (no allocation, copy, memset or synchronisation), so a caller
may record them into a HIP graph; replays must reproduce the eager results bit for bit, also after the inputs
change and with eager work between the replays."""
import numpy as np
import pytest
import scipy.sparse
import torch

from featgraph_amd import _lib, datasets, placeholder
from featgraph_amd.module import GeneralizedSpMMhip, VanillaSDDMMhip, VanillaSpMMhip
from oracle import ref

pytestmark = pytest.mark.gpu


def test_spmm_and_sddmm_replay_from_a_hip_graph():
    adj = datasets.config_graph("c2-mini")
    coo = adj.tocoo()
    n = adj.shape[0]
    F = 128
    _lib.config_set("spmm.blocked", 1)                 # several launches per call: column-block passes x tiles
    _lib.config_set("spmm.block_cols", 500)
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    try:
        spmm, sddmm = VanillaSpMMhip(adj), VanillaSDDMMhip(coo)
        assert "column blocks" in spmm.lower_to_ir([placeholder((n, F))], {}, {})
        spmm.build([placeholder((n, F))], {}, {})
        sddmm.build([placeholder((n, F)), placeholder((n, F))], {}, {})
        dev = spmm.ctx
        rng = np.random.default_rng(31)
        x = torch.zeros((n, F), dtype=torch.float32, device=dev)
        y = torch.zeros((n, F), dtype=torch.float32, device=dev)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):                  # warm-up outside the capture
            spmm.run([x]); sddmm.run([x, y])
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            spmm.run([x])
            sddmm.run([x, y])
        for step in range(3):
            xn = rng.standard_normal((n, F)).astype(np.float32)
            yn = rng.standard_normal((n, F)).astype(np.float32)
            x.copy_(torch.from_numpy(xn)); y.copy_(torch.from_numpy(yn))
            spmm.out_tvm.tensor.fill_(5.0); sddmm.out_tvm.tensor.fill_(5.0)     # eager work between the replays
            graph.replay()
            torch.cuda.synchronize(dev)
            got_spmm = spmm.out_tvm.asnumpy().copy()
            got_sddmm = sddmm.out_tvm.asnumpy().copy()
            assert np.array_equal(got_spmm, ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, xn)), step
            eager = sddmm.run([x, y]).asnumpy()
            assert np.array_equal(got_sddmm, eager), step
            np.testing.assert_allclose(got_sddmm, ref.sddmm_f64(coo.row, coo.col, xn, yn), rtol=1e-5, atol=1e-4)
    finally:
        for key in ("spmm.blocked", "sddmm.blocked"):
            _lib.config_set(key, -1)
        for key in ("spmm.block_cols", "sddmm.block_cols"):
            _lib.config_set(key, 0)


def test_unsorted_sddmm_and_generalised_spmm_replay_from_a_hip_graph():
    """The SDDMM plan of a shuffled list (row-run kernel over the sorted copy, then the two regrouping kernels with
    128 KB of LDS each) and the generalised SpMM (column-block passes, then the division of the mean)."""
    adj = datasets.config_graph("c2-mini")
    coo = adj.tocoo()
    n = adj.shape[0]
    F = 128
    perm = np.random.default_rng(5).permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    _lib.config_set("spmm.blocked", 1)
    _lib.config_set("spmm.block_cols", 500)
    _lib.config_set("sddmm.blocked", 1)
    _lib.config_set("sddmm.block_cols", 500)
    try:
        spmm, sddmm = GeneralizedSpMMhip(adj, "add", "mean"), VanillaSDDMMhip(shuffled)
        ph = [placeholder((n, F)), placeholder((n, F))]
        assert "rows-per-wave" in spmm.lower_to_ir(ph[:1], {}, {})
        assert "sorted by row and column" in sddmm.lower_to_ir(ph, {}, {})
        spmm.build(ph[:1], {}, {})
        sddmm.build(ph, {}, {})
        dev = spmm.ctx
        rng = np.random.default_rng(32)
        x = torch.zeros((n, F), dtype=torch.float32, device=dev)
        y = torch.zeros((n, F), dtype=torch.float32, device=dev)
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            spmm.run([x]); sddmm.run([x, y])
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            spmm.run([x])
            sddmm.run([x, y])
        for step in range(3):
            xn = rng.standard_normal((n, F)).astype(np.float32)
            yn = rng.standard_normal((n, F)).astype(np.float32)
            x.copy_(torch.from_numpy(xn)); y.copy_(torch.from_numpy(yn))
            spmm.out_tvm.tensor.fill_(5.0); sddmm.out_tvm.tensor.fill_(5.0)
            graph.replay()
            torch.cuda.synchronize(dev)
            got_spmm = spmm.out_tvm.asnumpy().copy()
            got_sddmm = sddmm.out_tvm.asnumpy().copy()
            assert np.array_equal(got_spmm, ref.spmm_general(adj.indptr, adj.indices, adj.data, xn, "add", "mean")), step
            assert np.array_equal(got_sddmm, sddmm.run([x, y]).asnumpy()), step
            np.testing.assert_allclose(got_sddmm, ref.sddmm_f64(shuffled.row, shuffled.col, xn, yn), rtol=1e-5, atol=1e-4)
    finally:
        for key in ("spmm.blocked", "sddmm.blocked"):
            _lib.config_set(key, -1)
        for key in ("spmm.block_cols", "sddmm.block_cols"):
            _lib.config_set(key, 0)
