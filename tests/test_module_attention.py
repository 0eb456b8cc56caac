"""GPU parity of the fused multi-head attention operator (scores + softmax + weighted sum in one kernel), through
the module layer and the C ABI, against the composed CPU checker (oracle/ref.py: attention_mh = multi-head SDDMM,
float64 edge softmax, sequential multi-head SpMM).

The kernel keeps a running softmax in float32 and rescales its weighted sum when the maximum grows, so the bar is a
tolerance: rtol 1e-4 with atol 1e-5 on outputs of magnitude ~1 (weighted means of N(0,1) features)."""
import numpy as np
import pytest
import scipy.sparse

from featgraph_amd import _lib, datasets, nd, placeholder
from featgraph_amd.module import EdgeSoftmaxhip, MultiHeadAttentionhip, MultiHeadSDDMMhip, MultiHeadSpMMhip
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def _operands(adj, H, D, seed=0, scale=0.5):
    rng = np.random.default_rng(seed)
    key = rng.standard_normal((adj.shape[1], H, D), dtype=np.float32) * np.float32(scale)
    query = rng.standard_normal((adj.shape[0], H, D), dtype=np.float32)
    value = rng.standard_normal((adj.shape[1], H, D), dtype=np.float32)
    return key, query, value


def _run(adj, arrays):
    module = MultiHeadAttentionhip(adj)
    ph = [placeholder(a.shape) for a in arrays]
    module.build(ph, {}, {})
    module.out_tvm.tensor.fill_(-7.0)                     # every element must be written, empty rows included
    out = module.run([nd.array(a, module.ctx) for a in arrays]).asnumpy()
    return out, module.lower_to_ir(ph, {}, {})


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("H,D,fused", [(8, 64, True), (8, 32, True), (8, 16, True), (8, 8, True), (4, 64, True),
                                       (16, 4, True), (16, 32, True), (32, 8, True), (4, 16, True),
                                       (4, 128, False), (8, 24, False), (3, 5, False), (1, 64, False)])
def test_attention_matches_the_composed_checker(H, D, fused, shared):
    adj = datasets.config_graph("c4-mini")              # degrees 1 .. 2,000, mean 25
    key, query, value = _operands(adj, H, D, seed=H * 131 + D)
    arrays = [key, query] if shared else [key, query, value]
    out, text = _run(adj, arrays)
    assert ("fused" in text) == fused
    want = ref.attention_mh(adj.indptr, adj.indices, key, query, None if shared else value)
    np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)


def test_attention_rows_of_every_length_around_the_batch_and_id_block_sizes():
    """Row i has i nonzeros, i = 0 .. 200: empty rows, rows shorter than one batch, rows that end on and just past
    a batch, a pair of batches and a block of 64 ids."""
    degs = np.arange(201)
    indptr = np.concatenate([[0], np.cumsum(degs)]).astype(np.int32)
    n_cols = 997
    rng = np.random.default_rng(5)
    indices = np.concatenate([np.sort(rng.choice(n_cols, d, replace=False)) for d in degs]).astype(np.int32)
    adj = scipy.sparse.csr_matrix((np.ones(len(indices), np.float32), indices, indptr), shape=(len(degs), n_cols))
    for H, D in [(8, 64), (8, 32), (8, 16)]:
        key, query, value = _operands(adj, H, D, seed=D)
        for arrays in ([key, query], [key, query, value]):
            out, _ = _run(adj, arrays)
            want = ref.attention_mh(indptr, indices, *arrays)
            np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)
            assert not out[0].any()                       # the row without nonzeros


def test_attention_with_large_scores_stays_finite_and_picks_the_maximum():
    adj = datasets.config_graph("c4-mini")
    key, query, _ = _operands(adj, 8, 32, seed=9, scale=6.0)        # scores of magnitude ~200: exp overflows float32
    out, _ = _run(adj, [key, query])
    assert np.all(np.isfinite(out))
    want = ref.attention_mh(adj.indptr, adj.indices, key, query)
    np.testing.assert_allclose(out, want, rtol=1e-3, atol=1e-4)     # nearly one-hot weights: absolute errors of the scores count


def test_attention_is_a_convex_combination_and_uniform_for_a_zero_query():
    adj = datasets.config_graph("c4-mini")
    key, query, value = _operands(adj, 8, 64, seed=2)
    out, _ = _run(adj, [key, np.zeros_like(query), value])           # all scores 0: the mean of the neighbours' values
    deg = np.diff(adj.indptr)
    row = np.repeat(np.arange(adj.shape[0]), deg)
    mean = np.zeros(out.shape, np.float64)
    np.add.at(mean, row, value[adj.indices].astype(np.float64))
    mean[deg > 0] /= deg[deg > 0, None, None]
    np.testing.assert_allclose(out, mean, rtol=1e-4, atol=1e-5)
    ones = np.ones_like(value)
    out, _ = _run(adj, [key, query, ones])                           # weights sum to one
    np.testing.assert_allclose(out[deg > 0], 1.0, rtol=1e-5)


def test_attention_grid_of_a_few_workgroups_and_errors_through_the_c_abi():
    import torch
    adj = datasets.config_graph("c4-mini")
    key, query, value = _operands(adj, 8, 64, seed=4)
    want = ref.attention_mh(adj.indptr, adj.indices, key, query, value)
    try:
        _lib.config_set("attention.blocks", 3)                       # every wave walks thousands of rows
        out, _ = _run(adj, [key, query, value])
    finally:
        _lib.config_set("attention.blocks", 0)
    np.testing.assert_allclose(out, want, rtol=RTOL, atol=ATOL)
    module = MultiHeadAttentionhip(adj)
    dev = module.ctx
    k = torch.from_numpy(key).to(dev)
    q = torch.from_numpy(query).to(dev)
    o = torch.empty_like(q)
    stream = torch.cuda.current_stream(dev).cuda_stream
    call = _lib.lib().fg_attention_csr_mh_f32                        # -1: bad argument, -4: no kernel for the shape
    assert call(module._plan, k.data_ptr(), q.data_ptr(), k.data_ptr(), o.data_ptr(), 3, 5, stream) == -4
    assert call(module._plan, k.data_ptr(), q.data_ptr(), 0, o.data_ptr(), 8, 64, stream) == -1
    assert call(None, k.data_ptr(), q.data_ptr(), k.data_ptr(), o.data_ptr(), 8, 64, stream) == -1
    assert call(module._plan, k.data_ptr() + 4, q.data_ptr(), k.data_ptr(), o.data_ptr(), 8, 64, stream) == -4
    with pytest.raises(ValueError):
        module.build([placeholder(key.shape), placeholder((query.shape[0] + 1,) + query.shape[1:])], {}, {})
    with pytest.raises(ValueError):
        module.build([placeholder(key.shape), placeholder(query.shape), placeholder((key.shape[0], 8, 32))], {}, {})


@pytest.mark.parametrize("H,D", [(8, 64), (8, 16), (4, 32)])
def test_the_three_operators_one_after_the_other_meet_the_tighter_bar(H, D):
    """Multi-head SDDMM, the standalone edge softmax and multi-head SpMM run one after the other: no running maximum
    is rescaled and every weight is one expf and one division, so the chain meets rtol 1e-5 (atol 1e-5 on outputs of
    magnitude ~1) where the fused kernels are held to 1e-4."""
    adj = datasets.config_graph("c4-mini")
    key, query, _ = _operands(adj, H, D, seed=7 * H + D)
    coo = adj.tocoo()                                     # row-sorted, the CSR order
    scores = MultiHeadSDDMMhip(coo)
    scores.build([placeholder(key.shape), placeholder(query.shape)], {}, {})
    s = scores.run([nd.array(key, scores.ctx), nd.array(query, scores.ctx)])
    softmax = EdgeSoftmaxhip(adj)
    softmax.build([placeholder(tuple(s.shape))], {}, {})
    w = softmax.run([s])
    spmm = MultiHeadSpMMhip(adj)
    spmm.build([placeholder(key.shape), placeholder(tuple(w.shape))], {}, {})
    out = spmm.run([nd.array(key, spmm.ctx), w]).asnumpy()
    want = ref.attention_mh(adj.indptr, adj.indices, key, query, None)
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-5)
