"""GPU parity at the benchmark's full sizes (the 232,965-vertex / ~114.6M-nonzero graph
and the 2.45M-vertex multi-head graph), against the CPU checker run on the host cores,
plus size-independent properties.  Each test prints what it is about to launch."""
import time

import numpy as np
import pytest

from featgraph_amd import datasets, nd, placeholder
from featgraph_amd.module import (GeneralizedSDDMMhip, GeneralizedSpMMhip, MultiHeadSDDMMhip, MultiHeadSDDMMSoftmaxhip,
                                  MultiHeadSpMMhip, VanillaSDDMMhip, VanillaSpMMhip)
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


def test_c5_multihead_generalised_spmm_max_and_mean_d16(c4):
    """The per-head message / reduce slots at full size: max of the weighted rows and the mean, bit-exact."""
    from featgraph_amd.module import MultiHeadGeneralizedSpMMhip
    adj = c4
    n = adj.shape[0]
    w = datasets.softmax_edge_weights(adj, 8)
    feat = datasets.spmm_operands(adj, (8, 16))
    for msg, reduce in (("mul", "max"), ("add", "mean")):
        _say("multi-head generalised SpMM c5 H=8 D=16 %s / %s through MultiHeadGeneralizedSpMMhip" % (msg, reduce))
        module = MultiHeadGeneralizedSpMMhip(adj, msg, reduce)
        module.build([placeholder((n, 8, 16)), placeholder(w.shape)], {}, {})
        out = module.run([nd.array(feat, module.ctx), nd.array(w, module.ctx)]).asnumpy()
        want = ref.spmm_mh_general(adj.indptr, adj.indices, w, feat, msg, reduce)
        assert np.array_equal(out, want)


# ---------------------------------------------------------------- every swept feature length at full size
def _device_normal(shape, seed, dev):
    """Seeded N(0,1) float32 operand drawn on the device (seconds faster than numpy at these sizes), plus its host copy."""
    import torch
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    t = torch.randn(shape, dtype=torch.float32, device=dev, generator=g)
    return t, t.cpu().numpy()


@pytest.fixture(scope="module")
def c2_spmm_module(c2):
    return VanillaSpMMhip(c2)


@pytest.fixture(scope="module")
def c3_sddmm_module(c2):
    coo = c2.tocoo()
    return coo, VanillaSDDMMhip(coo)


@pytest.mark.parametrize("F", [32, 128, 256, 512, 30, 65, 100])
def test_c2_spmm_bit_exact_at_every_swept_feature_length(c2, c2_spmm_module, F):
    """Covers what only happens at full size: one launch per column-block pass over every feature tile with carried
    sums, the wider passes of the narrower tiles, more long runs than the workgroup clamp, 100 MB run tables.
    30, 65, 100: lengths beside the sweep, where the row's end cuts a lane's four floats (30), the rest of the row
    runs as a narrower tile in launches of its own (65) and the last tile is a partial one (100)."""
    adj, module = c2, c2_spmm_module
    n = adj.shape[0]
    _say("SpMM c2 F=%d through VanillaSpMMhip: %s" % (F, module.lower_to_ir([placeholder((n, F))], {}, {})))
    module.build([placeholder((n, F))], {}, {})
    feat_dev, feat = _device_normal((n, F), 100 + F, module.ctx)
    module.out_tvm.tensor.fill_(-1.0)
    out = module.run([feat_dev]).asnumpy()
    del feat_dev
    want = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat)
    assert np.array_equal(out, want)


@pytest.mark.parametrize("F", [32, 128, 256, 512, 30, 130])
def test_c3_sddmm_at_every_swept_feature_length(c3_sddmm_module, F):
    coo, module = c3_sddmm_module
    n = coo.shape[0]
    ph = [placeholder((n, F)), placeholder((n, F))]
    _say("SDDMM c3 F=%d through VanillaSDDMMhip: %s" % (F, module.lower_to_ir(ph, {}, {})))
    module.build(ph, {}, {})
    src_dev, src = _device_normal((n, F), 200 + F, module.ctx)
    dst_dev, dst = _device_normal((n, F), 300 + F, module.ctx)
    module.out_tvm.tensor.fill_(-1.0)
    out = module.run([src_dev, dst_dev]).asnumpy()
    del src_dev, dst_dev
    exact = ref.sddmm_f64(coo.row, coo.col, src, dst)
    np.testing.assert_allclose(out, exact, rtol=RTOL, atol=ATOL)
    # the strict serial float32 restatement (op/vanilla_sddmm.py:43-47) on the head and the tail of the list.  Its
    # own rounding grows with the feature length (a 512-term sequential sum of magnitude ~20 is off by up to
    # ~1e-4), so beyond 128 floats the bound is widened by exactly the restatement's distance from the exact value.
    m = 2_000_000
    for sl in (slice(0, m), slice(coo.nnz - m, coo.nnz)):
        serial = ref.sddmm_x86(coo.row[sl], coo.col[sl], src, dst)
        slack = np.abs(serial - exact[sl]) if F > 128 else 0.0
        assert np.all(np.abs(out[sl] - serial) <= ATOL + RTOL * np.abs(serial) + slack)


@pytest.mark.parametrize("F", [64, 256])
def test_c3_sddmm_on_a_shuffled_edge_list(c2, F):
    """The same edges in a seeded random order: not row-sorted, so the plan sorts a copy, the row-run kernel works
    on the copy and a gather brings the results back; they must land at the caller's positions."""
    import scipy.sparse
    coo = c2.tocoo()
    n = coo.shape[0]
    perm = np.random.default_rng(17).permutation(coo.nnz)
    shuffled = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
    module = VanillaSDDMMhip(shuffled)
    ph = [placeholder((n, F)), placeholder((n, F))]
    text = module.lower_to_ir(ph, {}, {})
    _say("SDDMM c3 F=%d, shuffled list: %s" % (F, text))
    assert "sorted by row and column" in text
    module.build(ph, {}, {})
    src, dst = datasets.sddmm_operands(coo, F)
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    np.testing.assert_allclose(out, ref.sddmm_f64(shuffled.row, shuffled.col, src, dst), rtol=RTOL, atol=ATOL)
    # against the sorted list's results, edge by edge: the same kernel over the same runs, so the same bits
    sorted_module = VanillaSDDMMhip(coo)
    sorted_module.build(ph, {}, {})
    base = sorted_module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).asnumpy()
    assert np.array_equal(out, base[perm])


@pytest.mark.parametrize("msg,reduce,F", [("sub", "mean", 32), ("div", "max", 128), ("copy_u", "min", 64)])
def test_c2_generalised_spmm_bit_exact(c2, msg, reduce, F):
    """The several-rows-per-wave kernel with a message and a reducer in place of the multiply-add, at full size:
    tiles of 32 and 64 floats, several tiles, long runs, the division of the mean."""
    adj = c2
    n = adj.shape[0]
    vals = adj.data + np.float32(0.5)                                   # divisors away from zero
    module = GeneralizedSpMMhip(type(adj)((vals, adj.indices, adj.indptr), shape=adj.shape), msg, reduce)
    ph = [placeholder((n, F))]
    text = module.lower_to_ir(ph, {}, {})
    _say("generalised SpMM c2 %s/%s F=%d: %s" % (msg, reduce, F, text))
    assert "rows-per-wave" in text
    module.build(ph, {}, {})
    feat = datasets.spmm_operands(adj, F)
    out = module.run([nd.array(feat, module.ctx)]).asnumpy()
    assert np.array_equal(out, ref.spmm_general(adj.indptr, adj.indices, vals, feat, msg, reduce))


def test_c3_elementwise_edge_function_over_row_runs(c2):
    """Out[e, :] = Src[col[e], :] * Dst[row[e], :] on the full edge list (a 14.7 GB result at 32 floats), checked on
    the first and last two million edges against numpy."""
    coo = c2.tocoo()
    n, F = coo.shape[0], 32
    module = GeneralizedSDDMMhip(coo, "mul")
    ph = [placeholder((n, F)), placeholder((n, F))]
    text = module.lower_to_ir(ph, {}, {})
    _say("elementwise SDDMM c3 mul F=%d: %s" % (F, text))
    assert "row runs" in text
    module.build(ph, {}, {})
    src, dst = datasets.sddmm_operands(coo, F)
    out = module.run([nd.array(src, module.ctx), nd.array(dst, module.ctx)]).tensor
    m = 2_000_000
    for sl in (slice(0, m), slice(coo.nnz - m, coo.nnz)):
        assert np.array_equal(out[sl].cpu().numpy(), src[coo.col[sl]] * dst[coo.row[sl]])


@pytest.mark.parametrize("D", [32, 64])
def test_c4_multihead_sddmm_longer_heads(c4, D):
    """D = 64: 5 GB operands, beyond 32-bit buffer offsets, so the 64-bit addressing variant runs."""
    coo = c4.tocoo()
    n, H = coo.shape[0], 8
    _say("multi-head SDDMM c4 H=8 D=%d through MultiHeadSDDMMhip" % D)
    module = MultiHeadSDDMMhip(coo)
    module.build([placeholder((n, H, D)), placeholder((n, H, D))], {}, {})
    src_dev, src = _device_normal((n, H, D), 400 + D, module.ctx)
    dst_dev, dst = _device_normal((n, H, D), 500 + D, module.ctx)
    out = module.run([src_dev, dst_dev]).asnumpy()
    del src_dev, dst_dev
    assert out.shape == (coo.nnz, H)
    np.testing.assert_allclose(out, ref.sddmm_mh(coo.row, coo.col, src, dst), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("D", [16, 64])
def test_c4_fused_scores_and_softmax(c4, D):
    """The fused score + softmax kernel on the whole 2.45M-vertex graph (hub rows of 20,000 edges included),
    against the CPU checker's scores normalised in float64."""
    adj = c4
    coo = adj.tocoo()
    n, H = adj.shape[0], 8
    _say("fused multi-head scores + softmax c4 H=8 D=%d through MultiHeadSDDMMSoftmaxhip" % D)
    module = MultiHeadSDDMMSoftmaxhip(adj)
    ph = [placeholder((n, H, D)), placeholder((n, H, D))]
    assert "fused" in module.lower_to_ir(ph, {}, {})
    module.build(ph, {}, {})
    src_dev, src = _device_normal((n, H, D), 600 + D, module.ctx)
    dst_dev, dst = _device_normal((n, H, D), 700 + D, module.ctx)
    src_dev *= 0.25
    src *= np.float32(0.25)
    out = module.run([src_dev, dst_dev]).asnumpy()
    del src_dev, dst_dev
    want = ref.edge_softmax(adj.indptr, ref.sddmm_mh(coo.row, coo.col, src, dst))
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-6)
    rows = np.flatnonzero(np.diff(adj.indptr) > 0)
    sums = np.add.reduceat(out.astype(np.float64), adj.indptr[rows].astype(np.int64), axis=0)
    np.testing.assert_allclose(sums, 1.0, atol=1e-4)


@pytest.mark.parametrize("D,shared", [(64, True), (16, True), (64, False)])
def test_c4_fused_attention(c4, D, shared):
    """Scores, softmax and weighted sum in one kernel on the whole 2.45M-vertex graph (hub rows of thousands of
    edges included), against the three CPU checkers run one after the other; then with an all-ones value matrix,
    where every row with an edge must come out as exactly the sum of its weights, 1."""
    from featgraph_amd.module import MultiHeadAttentionhip
    adj = c4
    n, H = adj.shape[0], 8
    _say("fused attention c4 H=8 D=%d %s through MultiHeadAttentionhip" % (D, "key = value" if shared else "key, value"))
    module = MultiHeadAttentionhip(adj)
    ph = [placeholder((n, H, D))] * (2 if shared else 3)
    assert "fused" in module.lower_to_ir(ph, {}, {})
    module.build(ph, {}, {})
    key_dev, key = _device_normal((n, H, D), 800 + D, module.ctx)
    key_dev *= 0.25
    key *= np.float32(0.25)
    query_dev, query = _device_normal((n, H, D), 900 + D, module.ctx)
    ins, value = [key_dev, query_dev], None
    if not shared:
        value_dev, value = _device_normal((n, H, D), 950 + D, module.ctx)
        ins.append(value_dev)
    out = module.run(ins).asnumpy()
    want = ref.attention_mh(adj.indptr, adj.indices, key, query, value)
    np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
    del want, ins
    if not shared:
        value_dev.fill_(1.0)
        out = module.run([key_dev, query_dev, value_dev]).asnumpy()
        has_edges = np.diff(adj.indptr) > 0
        np.testing.assert_allclose(out[has_edges], 1.0, rtol=2e-5)
        assert not out[~has_edges].any()


@pytest.mark.parametrize("D,shared", [(16, True), (32, False)])
def test_c4_attention_backward(c4, D, shared):
    """All three gradients of the attention layer on the whole 2.45M-vertex graph (multi-head SpMM over the
    transposed matrix with permuted weights, softmax gradient, multi-head SDDMM), against the composed CPU checker."""
    from featgraph_amd.module import MultiHeadAttentionGradhip
    adj = c4
    n, H = adj.shape[0], 8
    _say("attention backward c4 H=8 D=%d %s through MultiHeadAttentionGradhip" % (D, "key = value" if shared else "key, value"))
    module = MultiHeadAttentionGradhip(adj)
    module.build([placeholder((n, H, D))] * (2 if shared else 3), {}, {})
    key_dev, key = _device_normal((n, H, D), 1000 + D, module.ctx)
    key_dev *= 0.25
    key *= np.float32(0.25)
    query_dev, query = _device_normal((n, H, D), 1100 + D, module.ctx)
    dout_dev, dout = _device_normal((n, H, D), 1200 + D, module.ctx)
    ins, value = [key_dev, query_dev], None
    if not shared:
        value_dev, value = _device_normal((n, H, D), 1300 + D, module.ctx)
        ins.append(value_dev)
    d_key, d_query, d_value = module.run(ins + [dout_dev])
    want_key, want_query, want_value = ref.attention_mh_backward(adj.indptr, adj.indices, key, query, value, dout)
    # sums of up to thousands of float32 terms whose weights come from a float32 softmax: the forward operator's
    # tolerance scaled to the size of the gradients
    np.testing.assert_allclose(d_query.asnumpy(), want_query, rtol=1e-3, atol=5e-4)
    np.testing.assert_allclose(d_key.asnumpy(), want_key, rtol=1e-3, atol=5e-4)
    if shared:
        assert d_value is None
    else:
        np.testing.assert_allclose(d_value.asnumpy(), want_value, rtol=1e-3, atol=5e-4)


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
