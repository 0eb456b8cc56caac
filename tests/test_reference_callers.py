"""Callers written against the reference's package name: `featgraph.module.VanillaSpMMcuda` /
`VanillaSDDMMcuda` with the launch keys and the matrix family of the reference's GPU tests
(tests/test_module_spmm.py:37-59: threads per block 32 / 128 / unset; tests/test_module_sddmm.py:44-70:
32 / 256 blocks; 127 x 255 at density 0.1, feature length 128, rtol = atol = 1e-4 against scipy / numpy)."""
import numpy as np
import pytest
import scipy.sparse

import featgraph
from featgraph.module import VanillaSDDMMcuda, VanillaSpMMcuda

pytestmark = pytest.mark.gpu
F = 128


def _matrix(fmt, seed):
    return scipy.sparse.random(127, 255, density=0.1, format=fmt, random_state=np.random.default_rng(seed))


@pytest.mark.parametrize("threads", [32, 128, None])
def test_spmm_through_the_reference_names(threads):
    adj = _matrix("csr", 5)
    feat = np.random.default_rng(7).random((adj.shape[1], F)).astype("float32")
    m = VanillaSpMMcuda(adj)
    m.build([featgraph.placeholder(feat.shape)], {}, {"num_threads_per_cuda_block": threads})
    out = m.run([featgraph.nd.array(feat, m.ctx)]).asnumpy()
    np.testing.assert_allclose(adj.dot(feat), out, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("blocks", [32, 256])
def test_sddmm_through_the_reference_names(blocks):
    adj = _matrix("coo", 6).astype("int32")          # edge values are never read; the reference's test casts them too
    rng = np.random.default_rng(8)
    src = rng.random((adj.shape[1], F)).astype("float32")
    dst = rng.random((adj.shape[0], F)).astype("float32")
    m = VanillaSDDMMcuda(adj)
    m.build([featgraph.placeholder(src.shape), featgraph.placeholder(dst.shape)], {}, {"num_cuda_blocks": blocks})
    out = m.run([featgraph.nd.array(src, m.ctx), featgraph.nd.array(dst, m.ctx)]).asnumpy()
    np.testing.assert_allclose((src[adj.col] * dst[adj.row]).sum(axis=-1), out, rtol=1e-4, atol=1e-4)
