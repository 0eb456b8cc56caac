"""GPU parity of the multi-head backward modules and of the multi-head generalised SpMM, through the module layer
and the C ABI, against the CPU checkers (oracle/featgraph_ref.c: fgref_spmm_mh, fgref_sddmm_mh,
fgref_edge_softmax_backward, fgref_spmm_mh_general) run on the same operands.  Sums of products reproduce the
checker's order bit for bit; dot products and the softmax gradient are float32 against binary64, hence tolerances."""
import ctypes

import numpy as np
import pytest
import scipy.sparse

from featgraph_amd import _lib, datasets, nd, placeholder
from featgraph_amd.module import (EdgeSoftmaxGradhip, MultiHeadAttentionGradhip, MultiHeadAttentionhip,
                                  MultiHeadGeneralizedSpMMhip, MultiHeadSDDMMGradhip, MultiHeadSpMMGradhip)
from featgraph_amd.module.backward import transpose_with_permutation
from oracle import ref

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-4      # dot products (the SDDMM bar)


def _dev(module, arrays):
    return [nd.array(x, module.ctx) for x in arrays]


def _rect_graph(seed=0, shape=(300, 450), density=0.05):
    """Non-square, with rows and columns that have no entries."""
    rng = np.random.default_rng(seed)
    adj = scipy.sparse.random(shape[0], shape[1], density=density, format="lil", random_state=rng, dtype=np.float32)
    adj[7] = 0
    adj[:, 11] = 0
    adj = adj.tocsr()
    adj.sort_indices()
    return adj


def test_transpose_with_permutation_is_scipy_transpose():
    adj = _rect_graph()
    adj.data = np.arange(1, adj.nnz + 1, dtype=np.float32)      # the values name the entries
    t, perm = transpose_with_permutation(adj)
    want = adj.T.tocsr()
    want.sort_indices()
    assert np.array_equal(t.indptr, want.indptr) and np.array_equal(t.indices, want.indices)
    assert np.array_equal(t.data, want.data) and np.array_equal(adj.data[perm], t.data)
    assert np.array_equal(np.sort(perm), np.arange(adj.nnz))


@pytest.mark.parametrize("H", [1, 2, 4, 8, 3, 100])
def test_edge_softmax_backward_matches_the_float64_checker(H):
    adj = datasets.config_graph("c4-mini")
    rng = np.random.default_rng(H)
    weights = ref.edge_softmax(adj.indptr, (rng.standard_normal((adj.nnz, H)) * 3).astype(np.float32))
    grad = rng.standard_normal((adj.nnz, H)).astype(np.float32)
    module = EdgeSoftmaxGradhip(adj)
    module.build([placeholder(weights.shape)], {}, {})
    module.out_tvm.tensor.fill_(9.0)
    out = module.run(_dev(module, [weights, grad])).asnumpy()
    np.testing.assert_allclose(out, ref.edge_softmax_backward(adj.indptr, weights, grad), rtol=1e-4, atol=1e-6)
    rows = np.flatnonzero(np.diff(adj.indptr) > 0)
    np.testing.assert_allclose(np.add.reduceat(out.astype(np.float64), adj.indptr[rows], axis=0), 0.0, atol=1e-5)


def test_edge_softmax_backward_in_place_and_error_codes_through_the_c_abi():
    import torch
    L = _lib.lib()
    adj = datasets.config_graph("c4-mini")
    dev = torch.device("cuda", 0)
    rng = np.random.default_rng(1)
    weights = ref.edge_softmax(adj.indptr, rng.standard_normal((adj.nnz, 8)).astype(np.float32))
    grad = rng.standard_normal((adj.nnz, 8)).astype(np.float32)
    w_d, g_d = torch.from_numpy(weights).to(dev), torch.from_numpy(grad).to(dev)
    indptr = torch.from_numpy(adj.indptr.astype(np.int32)).to(dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    _lib.check(L.fg_edge_softmax_backward_csr_f32(adj.shape[0], indptr.data_ptr(), w_d.data_ptr(), g_d.data_ptr(),
                                                  g_d.data_ptr(), 8, st))
    np.testing.assert_allclose(g_d.cpu().numpy(), ref.edge_softmax_backward(adj.indptr, weights, grad),
                               rtol=1e-4, atol=1e-6)
    assert L.fg_edge_softmax_backward_csr_f32(4, None, w_d.data_ptr(), g_d.data_ptr(), g_d.data_ptr(), 8, st) == -1
    assert L.fg_edge_softmax_backward_csr_f32(-1, indptr.data_ptr(), w_d.data_ptr(), g_d.data_ptr(), g_d.data_ptr(), 8, st) == -1
    assert L.fg_edge_softmax_backward_csr_f32(0, None, None, None, None, 8, st) == 0
    # the two helpers
    perm = torch.from_numpy(np.random.default_rng(2).permutation(1000).astype(np.int32)).to(dev)
    src = torch.arange(3000, dtype=torch.float32, device=dev).reshape(1000, 3)
    out = torch.zeros_like(src)
    _lib.check(L.fg_permute_rows_f32(1000, 3, perm.data_ptr(), src.data_ptr(), out.data_ptr(), st))
    assert torch.equal(out, src[perm.long()])
    assert L.fg_permute_rows_f32(10, 0, perm.data_ptr(), src.data_ptr(), out.data_ptr(), st) == -1
    assert L.fg_permute_rows_f32(10, 3, None, src.data_ptr(), out.data_ptr(), st) == -1
    a, b = torch.rand(5001, device=dev), torch.rand(5001, device=dev)
    want = a + b
    _lib.check(L.fg_add_f32(5001, a.data_ptr(), b.data_ptr(), a.data_ptr(), st))
    assert torch.equal(a, want)
    assert L.fg_add_f32(5, None, b.data_ptr(), a.data_ptr(), st) == -1 and L.fg_add_f32(0, None, None, None, st) == 0


@pytest.mark.parametrize("graph,H,D", [("rect", 4, 8), ("c4-mini", 8, 16), ("c4-mini", 8, 64), ("c2-mini", 2, 5)])
def test_multi_head_spmm_backward(graph, H, D):
    adj = _rect_graph() if graph == "rect" else datasets.config_graph(graph)
    rng = np.random.default_rng(3)
    feat = rng.standard_normal((adj.shape[1], H, D), dtype=np.float32)
    weight = datasets.softmax_edge_weights(adj, H)
    dout = rng.standard_normal((adj.shape[0], H, D), dtype=np.float32)
    module = MultiHeadSpMMGradhip(adj)
    module.build([placeholder(feat.shape), placeholder(weight.shape)], {}, {})
    d_feat, d_weight = module.run(_dev(module, [feat, weight, dout]))
    t, perm = transpose_with_permutation(adj)
    # dFeat: the sequential float32 sum over the transposed matrix, bit for bit
    assert np.array_equal(d_feat.asnumpy(), ref.spmm_mh(t.indptr, t.indices, np.ascontiguousarray(weight[perm]), dout))
    coo = adj.tocoo()
    exact = np.einsum("ehd,ehd->eh", feat[coo.col].astype(np.float64), dout[coo.row].astype(np.float64))
    np.testing.assert_allclose(d_weight.asnumpy(), exact, rtol=RTOL, atol=ATOL)
    # the pair is the gradient of <Out, dOut>: a directional derivative in float64 agrees
    dx = rng.standard_normal(feat.shape)
    dw = rng.standard_normal(weight.shape)
    lhs = (d_feat.asnumpy().astype(np.float64) * dx).sum() + (d_weight.asnumpy().astype(np.float64) * dw).sum()
    def loss(x, w):
        out = np.zeros((adj.shape[0], H, D))
        np.add.at(out, coo.row, w[:, :, None] * x[coo.col])
        return (out * dout).sum()
    rhs = loss(feat + dx, weight.astype(np.float64)) - loss(feat, weight.astype(np.float64)) \
        + loss(feat, weight + dw) - loss(feat, weight.astype(np.float64))      # bilinear: exact first-order parts
    np.testing.assert_allclose(lhs, rhs, rtol=1e-4)


@pytest.mark.parametrize("graph,H,D", [("rect", 4, 8), ("c4-mini", 8, 32), ("c2-mini", 3, 4)])
def test_multi_head_sddmm_backward(graph, H, D):
    adj = _rect_graph(seed=1) if graph == "rect" else datasets.config_graph(graph)
    rng = np.random.default_rng(4)
    src = rng.standard_normal((adj.shape[1], H, D), dtype=np.float32)
    dst = rng.standard_normal((adj.shape[0], H, D), dtype=np.float32)
    dscores = rng.standard_normal((adj.nnz, H)).astype(np.float32)
    module = MultiHeadSDDMMGradhip(adj)
    module.build([placeholder(src.shape), placeholder(dst.shape)], {}, {})
    d_src, d_dst = module.run(_dev(module, [src, dst, dscores]))
    t, perm = transpose_with_permutation(adj)
    assert np.array_equal(d_src.asnumpy(), ref.spmm_mh(t.indptr, t.indices, np.ascontiguousarray(dscores[perm]), dst))
    assert np.array_equal(d_dst.asnumpy(), ref.spmm_mh(adj.indptr, adj.indices, dscores, src))
    assert not d_dst.asnumpy()[np.diff(adj.indptr) == 0].any()


@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("graph,H,D", [("rect", 4, 8), ("c4-mini", 8, 16), ("c4-mini", 8, 64), ("c2-mini", 2, 6)])
def test_attention_backward_matches_the_composed_checker(graph, H, D, shared):
    adj = _rect_graph(seed=2) if graph == "rect" else datasets.config_graph(graph)
    rng = np.random.default_rng(5)
    key = rng.standard_normal((adj.shape[1], H, D), dtype=np.float32) * np.float32(0.3)
    query = rng.standard_normal((adj.shape[0], H, D), dtype=np.float32)
    value = None if shared else rng.standard_normal((adj.shape[1], H, D), dtype=np.float32)
    dout = rng.standard_normal((adj.shape[0], H, D), dtype=np.float32)
    ins = [key, query] + ([] if shared else [value])
    module = MultiHeadAttentionGradhip(adj)
    module.build([placeholder(x.shape) for x in ins], {}, {})
    d_key, d_query, d_value = module.run(_dev(module, ins + [dout]))
    want_key, want_query, want_value = ref.attention_mh_backward(adj.indptr, adj.indices, key, query, value, dout)
    # float32 exp and float32 row sums against the binary64 softmax of the checker, then sums over up to 2,000
    # neighbours: the forward operator's own tolerance, scaled to gradient magnitudes
    np.testing.assert_allclose(d_query.asnumpy(), want_query, rtol=1e-3, atol=2e-4)
    np.testing.assert_allclose(d_key.asnumpy(), want_key, rtol=1e-3, atol=2e-4)
    if shared:
        assert d_value is None
    else:
        np.testing.assert_allclose(d_value.asnumpy(), want_value, rtol=1e-3, atol=2e-4)
    assert np.array_equal(module.run(_dev(module, ins + [dout]))[1].asnumpy(), d_query.asnumpy())   # nothing carried over


def test_attention_backward_against_torch_autograd_of_the_dense_form():
    """Forward and backward modules against torch's autograd of softmax(mask(Q K^T)) V in float64."""
    import torch
    adj = _rect_graph(seed=3, shape=(60, 90), density=0.15)
    rng = np.random.default_rng(6)
    H, D = 8, 16
    key = rng.standard_normal((90, H, D), dtype=np.float32) * np.float32(0.3)
    value = rng.standard_normal((90, H, D), dtype=np.float32)
    query = rng.standard_normal((60, H, D), dtype=np.float32)
    dout = rng.standard_normal((60, H, D), dtype=np.float32)
    k = torch.tensor(key, dtype=torch.float64, requires_grad=True)
    q = torch.tensor(query, dtype=torch.float64, requires_grad=True)
    v = torch.tensor(value, dtype=torch.float64, requires_grad=True)
    mask = torch.tensor(adj.toarray() != 0)
    s = torch.einsum("rhd,chd->hrc", q, k).masked_fill(~mask[None], float("-inf"))
    out = torch.einsum("hrc,chd->rhd", torch.nan_to_num(torch.softmax(s, dim=2)), v)
    out.backward(torch.tensor(dout, dtype=torch.float64))
    fwd = MultiHeadAttentionhip(adj)
    fwd.build([placeholder(key.shape), placeholder(query.shape), placeholder(value.shape)], {}, {})
    np.testing.assert_allclose(fwd.run(_dev(fwd, [key, query, value])).asnumpy(), out.detach().numpy(), rtol=1e-4, atol=1e-5)
    bwd = MultiHeadAttentionGradhip(adj)
    bwd.build([placeholder(key.shape), placeholder(query.shape), placeholder(value.shape)], {}, {})
    d_key, d_query, d_value = bwd.run(_dev(bwd, [key, query, value, dout]))
    np.testing.assert_allclose(d_key.asnumpy(), k.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(d_query.asnumpy(), q.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(d_value.asnumpy(), v.grad.numpy(), rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- multi-head generalised SpMM
@pytest.mark.parametrize("msg", ["mul", "add", "sub", "div", "copy_u"])
@pytest.mark.parametrize("reduce", ["sum", "max", "min", "mean"])
def test_multi_head_generalised_spmm_is_bit_exact(msg, reduce):
    adj = datasets.config_graph("c4-mini")
    H, D = 8, 16
    feat = datasets.spmm_operands(adj, (H, D))
    weight = datasets.softmax_edge_weights(adj, H) + np.float32(0.25)     # away from zero: quotients stay finite
    module = MultiHeadGeneralizedSpMMhip(adj, msg, reduce)
    module.build([placeholder(feat.shape), placeholder(weight.shape)], {}, {})
    module.out_tvm.tensor.fill_(-7.0)
    out = module.run(_dev(module, [feat, weight])).asnumpy()
    assert np.array_equal(out, ref.spmm_mh_general(adj.indptr, adj.indices, weight, feat, msg, reduce))


@pytest.mark.parametrize("graph,H,D", [("c2-mini", 2, 32), ("c2-mini", 3, 5), ("c4-mini", 8, 64), ("c4-mini", 1, 24),
                                       ("rect", 5, 1), ("rect", 16, 12)])
def test_multi_head_generalised_spmm_shapes_hubs_and_column_blocks(graph, H, D):
    adj = _rect_graph(seed=4) if graph == "rect" else datasets.config_graph(graph)
    feat = datasets.spmm_operands(adj, (H, D))
    weight = np.random.default_rng(7).standard_normal((adj.nnz, H)).astype(np.float32)
    for msg, reduce, parts in (("mul", "max", None), ("add", "mean", None), ("sub", "min", 4), ("mul", "sum", 3)):
        module = MultiHeadGeneralizedSpMMhip(adj, msg, reduce, parts)
        module.build([placeholder(feat.shape), placeholder(weight.shape)], {}, {})
        out = module.run(_dev(module, [feat, weight])).asnumpy()
        assert np.array_equal(out, ref.spmm_mh_general(adj.indptr, adj.indices, weight, feat, msg, reduce)), (msg, reduce)
    # (mul, sum) is the multi-head operator of the benchmark's configuration 5
    assert np.array_equal(out, ref.spmm_mh(adj.indptr, adj.indices, weight, feat))


def test_multi_head_generalised_spmm_rejects_bad_arguments():
    adj = _rect_graph()
    with pytest.raises(ValueError):
        MultiHeadGeneralizedSpMMhip(adj, "pow", "sum")
    module = MultiHeadGeneralizedSpMMhip(adj, "mul", "max")
    with pytest.raises(ValueError):
        module.build([placeholder((adj.shape[1], 4, 8)), placeholder((adj.nnz, 3))], {}, {})
    L = _lib.lib()
    assert L.fg_spmm_csr_mh_general_f32(None, 8, 8, 8, 2, 4, 0, 0, None) == -1
    plan = module._plan
    assert L.fg_spmm_csr_mh_general_f32(plan, 8, 8, 8, 2, 4, 9, 0, None) == -1
    assert L.fg_spmm_csr_mh_general_f32(plan, 8, 8, 8, 2, 4, 0, 7, None) == -1
    assert L.fg_spmm_csr_mh_general_f32(plan, None, 8, 8, 2, 4, 0, 0, None) == -1
