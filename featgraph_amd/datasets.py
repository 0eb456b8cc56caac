"""Seeded synthetic adjacency matrices and operands for the SpMM / SDDMM kernels.

The reference benchmarks on the Reddit graph fetched through DGL
(benchmark/download_reddit_dataset.py:9-20: 232,965 vertices, ~114.6M nonzeros,
canonical CSR, float32).  Neither DGL nor a network is available to this
build, so the same shapes are produced by deterministic generators: every
function below is a pure function of its arguments and of numpy's PCG64
stream, so the same call gives the same arrays on every machine.

All index arrays are int32 and all values float32, as scipy produces for
nnz < 2**31 (reference: module/spmm.py:58-66 keeps the scipy dtypes).
"""
import hashlib

import numpy as np
import scipy.sparse

__all__ = [
    "small_uniform_csr", "powerlaw_csr", "config_graph", "spmm_operands",
    "sddmm_operands", "softmax_edge_weights", "structure_checksum", "CONFIGS",
]


def small_uniform_csr(n=4096, deg_lo=8, deg_hi=24, seed=0):
    """Square graph whose rows hold deg_lo..deg_hi distinct sorted columns.

    Draw order (fixed): degrees, then per row the column choice, then values.
    Returns a canonical scipy CSR matrix with float32 values in [0, 1).
    """
    rng = np.random.default_rng(seed)
    deg = rng.integers(deg_lo, deg_hi + 1, n)
    indptr = np.zeros(n + 1, dtype=np.int32)
    np.cumsum(deg, out=indptr[1:])
    indices = np.empty(int(indptr[-1]), dtype=np.int32)
    for r in range(n):
        indices[indptr[r]:indptr[r + 1]] = np.sort(rng.choice(n, int(deg[r]), replace=False))
    vals = rng.random(int(indptr[-1]), dtype=np.float32)
    return scipy.sparse.csr_matrix((vals, indices, indptr), shape=(n, n))


def _sorted_unique_keys(keys, use_gpu=None):
    """Sort int64 keys and drop duplicates.

    Sorting is a function of the values only, so the device used cannot change
    the result; a GPU, when torch sees one, merely makes the 114.6M-key case
    take a fraction of a second instead of tens of seconds.  use_gpu=False
    forces the numpy path.
    """
    try:
        import torch
        if use_gpu is not False and torch.cuda.is_available():
            t = torch.from_numpy(keys).cuda()
            t = torch.unique(t, sorted=True)
            out = t.cpu().numpy()
            del t
            torch.cuda.empty_cache()
            return out
    except ImportError:
        pass
    keys.sort()
    keep = np.empty(keys.shape[0], dtype=bool)
    keep[:1] = True
    np.not_equal(keys[1:], keys[:-1], out=keep[1:])
    return keys[keep]


def powerlaw_csr(n, mean_deg, sigma, max_deg, seed=0, self_loops=True, use_gpu=None):
    """Power-law (lognormal out-degree) graph with uniform random columns.

    Degrees are clip(round(lognormal(mu, sigma)), 1, max_deg) with mu chosen so
    the mean is mean_deg, rescaled once so that their sum is n*mean_deg.
    Columns are drawn with replacement, the first draw of every row is
    replaced by the row's own id (self-loop), and each row is then sorted and
    de-duplicated, so the realised nnz is slightly below the drawn total.
    Values are uniform [0, 1) float32 in CSR order.
    """
    rng = np.random.default_rng(seed)
    mu = np.log(mean_deg) - 0.5 * sigma * sigma
    deg = np.clip(np.rint(rng.lognormal(mu, sigma, n)), 1, max_deg)
    deg = np.clip(np.rint(deg * (n * float(mean_deg) / deg.sum())), 1, max_deg).astype(np.int64)
    total = int(deg.sum())
    rows = np.repeat(np.arange(n, dtype=np.int64), deg)
    cols = rng.integers(0, n, total, dtype=np.int64)
    if self_loops:
        first = np.zeros(n, dtype=np.int64)
        np.cumsum(deg[:-1], out=first[1:])
        cols[first] = np.arange(n, dtype=np.int64)
    rows *= n
    rows += cols
    del cols
    keys = _sorted_unique_keys(rows, use_gpu)
    del rows
    r = keys // n
    indices = (keys - r * n).astype(np.int32)
    del keys
    indptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=indptr[1:])
    del r
    nnz = int(indptr[-1])
    assert nnz < 2 ** 31
    vals = rng.random(nnz, dtype=np.float32)
    m = scipy.sparse.csr_matrix((vals, indices, indptr.astype(np.int32)), shape=(n, n))
    m.has_sorted_indices = True
    return m


# name -> generator arguments.  "c2" is the 232,965-vertex / ~114.6M-nonzero
# graph of the Reddit benchmark's shape; "c4" the 2.45M-vertex multi-head one.
CONFIGS = {
    "c1": dict(kind="uniform", n=4096, deg_lo=8, deg_hi=24, seed=0),
    "c2": dict(kind="powerlaw", n=232965, mean_deg=493.2, sigma=0.967, max_deg=21700, seed=0),
    "c4": dict(kind="powerlaw", n=2449029, mean_deg=25.3, sigma=1.2, max_deg=20000, seed=0),
    # reduced versions of the same families, for parity tests that a CPU finishes in seconds
    "c2-mini": dict(kind="powerlaw", n=6000, mean_deg=120.0, sigma=0.967, max_deg=3000, seed=0),
    "c4-mini": dict(kind="powerlaw", n=20000, mean_deg=25.3, sigma=1.2, max_deg=2000, seed=0),
}
CONFIGS["c3"] = CONFIGS["c2"]
CONFIGS["c5"] = CONFIGS["c4"]


def config_graph(name):
    """Adjacency matrix (canonical CSR) of one named configuration."""
    cfg = dict(CONFIGS[name])
    kind = cfg.pop("kind")
    if kind == "uniform":
        return small_uniform_csr(**cfg)
    return powerlaw_csr(**cfg)


def spmm_operands(adj, feat_shape, seed=1):
    """Standard-normal float32 source features of shape (num_cols, *feat_shape)."""
    rng = np.random.default_rng(seed)
    if isinstance(feat_shape, int):
        feat_shape = (feat_shape,)
    return rng.standard_normal((adj.shape[1],) + tuple(feat_shape), dtype=np.float32)


def sddmm_operands(adj, feat_shape, seed=2):
    """(src, dst): src has num_cols rows, dst num_rows rows; drawn in that order."""
    rng = np.random.default_rng(seed)
    if isinstance(feat_shape, int):
        feat_shape = (feat_shape,)
    src = rng.standard_normal((adj.shape[1],) + tuple(feat_shape), dtype=np.float32)
    dst = rng.standard_normal((adj.shape[0],) + tuple(feat_shape), dtype=np.float32)
    return src, dst


def softmax_edge_weights(adj_csr, num_heads, seed=3):
    """Per-edge per-head weights [nnz, H]: softmax of U[0,1) logits over each row's edges."""
    rng = np.random.default_rng(seed)
    nnz = adj_csr.nnz
    w = np.exp(rng.random((nnz, num_heads), dtype=np.float32).astype(np.float64))
    indptr = adj_csr.indptr.astype(np.int64)
    nonempty = np.flatnonzero(np.diff(indptr) > 0)
    sums = np.add.reduceat(w, indptr[nonempty], axis=0) if nnz else np.zeros((0, num_heads))
    rows = np.repeat(np.arange(nonempty.shape[0]), np.diff(indptr)[nonempty])
    return (w / sums[rows]).astype(np.float32)


def structure_checksum(adj_csr):
    """Short SHA-256 of indptr and indices, quoted in reports to identify the graph."""
    h = hashlib.sha256()
    h.update(np.ascontiguousarray(adj_csr.indptr).tobytes())
    h.update(np.ascontiguousarray(adj_csr.indices).tobytes())
    return h.hexdigest()[:16]
