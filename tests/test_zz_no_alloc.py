"""fg_spmm_csr_noalloc_f32 (the entry point that allocates nothing) against fg_spmm_csr_f32 over a plan, both
called through the C ABI on the same device arrays: identical bits, on two calls in a row of which the second
is smaller (the built-in schedule array still holds the first call's rows then)."""
import ctypes

import numpy as np
import pytest
import torch

from featgraph_amd import _lib, datasets

pytestmark = pytest.mark.gpu


def _both(adj, F, seed):
    L = _lib.lib()
    dev = torch.device("cuda", 0)
    n_rows, n_cols = adj.shape
    indptr = torch.from_numpy(adj.indptr.astype(np.int32)).to(dev)
    indices = torch.from_numpy(adj.indices.astype(np.int32)).to(dev)
    vals = torch.from_numpy(adj.data.astype(np.float32)).to(dev)
    rng = np.random.default_rng(seed)
    feat = torch.from_numpy(rng.standard_normal((n_cols, F), dtype=np.float32)).to(dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    plan = ctypes.c_void_p()
    _lib.check(L.fg_spmm_plan_create(n_rows, n_cols, adj.nnz, indptr.data_ptr(), indices.data_ptr(),
                                     ctypes.byref(plan)))
    want = torch.full((n_rows, F), 7.0, dtype=torch.float32, device=dev)
    _lib.check(L.fg_spmm_csr_f32(plan, feat.data_ptr(), vals.data_ptr(), want.data_ptr(), F, 0, stream))
    got = torch.full((n_rows, F), -3.0, dtype=torch.float32, device=dev)      # stale contents must all be overwritten
    print("fg_spmm_csr_noalloc_f32 rows=%d nnz=%d F=%d" % (n_rows, adj.nnz, F), flush=True)

    def call():
        _lib.check(L.fg_spmm_csr_noalloc_f32(n_rows, n_cols, adj.nnz, indptr.data_ptr(), indices.data_ptr(),
                                             vals.data_ptr(), feat.data_ptr(), got.data_ptr(), F, stream))
        torch.cuda.synchronize(dev)

    call()   # the first call on a device may make the runtime load the library's code object (built-in array included)
    first = got.clone()
    got.fill_(-3.0)
    torch.cuda.synchronize(dev)
    # free device memory as the driver reports it (hipMemGetInfo): it sees a hipMalloc / hipFree inside the library,
    # which torch's own allocator statistics would not
    free_before = torch.cuda.mem_get_info(dev)[0]
    reserved_before = torch.cuda.memory_reserved(dev)
    call()
    assert torch.cuda.memory_reserved(dev) == reserved_before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(first, got)
    L.fg_spmm_plan_destroy(plan)
    return got.cpu().numpy(), want.cpu().numpy()


def test_noalloc_spmm_matches_the_planned_entry_point_twice_in_a_row():
    big = datasets.config_graph("c2-mini")          # 6,000 rows, hub rows of up to 3,000 nonzeros
    got, want = _both(big, 64, 1)
    assert np.array_equal(got, want)
    small = datasets.config_graph("c1")             # 4,096 rows, 8..24 nonzeros each: fewer rows, fewer classes
    got, want = _both(small, 64, 2)
    assert np.array_equal(got, want)
    got, want = _both(small[:1000], 20, 3)          # smaller again, feature length not a multiple of 16
    assert np.array_equal(got, want)


def test_noalloc_spmm_rejects_what_it_cannot_hold():
    L = _lib.lib()
    rc = L.fg_spmm_csr_noalloc_f32((1 << 20) + 1, 8, 0, 8, None, None, None, 8, 4, None)
    assert rc == -4 and b"exceeds" in L.fg_last_error()
    assert L.fg_spmm_csr_noalloc_f32(4, 4, 0, None, None, None, None, 8, 4, None) == -1   # null indptr
    assert L.fg_spmm_csr_noalloc_f32(0, 4, 0, 8, None, None, None, None, 4, None) == 0    # no rows: nothing to do


def test_noalloc_spmm_replays_from_a_hip_graph():
    """The entry point enqueues kernels only (its counters are cleared by a fill kernel, not a memset), so after one
    eager call (which looks up the built-in array's address) it can be recorded into a HIP graph; every replay must
    reproduce the eager result, also after the operands changed and with eager work between the replays."""
    L = _lib.lib()
    dev = torch.device("cuda", 0)
    adj = datasets.config_graph("c2-mini")
    n_rows, n_cols = adj.shape
    F = 64
    indptr = torch.from_numpy(adj.indptr.astype(np.int32)).to(dev)
    indices = torch.from_numpy(adj.indices.astype(np.int32)).to(dev)
    vals = torch.from_numpy(adj.data.astype(np.float32)).to(dev)
    feat = torch.zeros((n_cols, F), dtype=torch.float32, device=dev)
    out = torch.zeros((n_rows, F), dtype=torch.float32, device=dev)

    def call():
        _lib.check(L.fg_spmm_csr_noalloc_f32(n_rows, n_cols, adj.nnz, indptr.data_ptr(), indices.data_ptr(),
                                             vals.data_ptr(), feat.data_ptr(), out.data_ptr(), F,
                                             torch.cuda.current_stream(dev).cuda_stream))

    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        call()                                        # outside the capture: first call on this device
    torch.cuda.current_stream(dev).wait_stream(side)
    torch.cuda.synchronize(dev)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    from oracle import ref
    rng = np.random.default_rng(5)
    for step in range(3):
        x = rng.standard_normal((n_cols, F)).astype(np.float32)
        feat.copy_(torch.from_numpy(x))
        out.fill_(3.0)                                # eager work between the replays
        graph.replay()
        torch.cuda.synchronize(dev)
        assert np.array_equal(out.cpu().numpy(), ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, x)), step
