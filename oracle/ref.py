"""ctypes front end of libfeatgraph_ref.so (oracle/featgraph_ref.c).

TEST INFRASTRUCTURE ONLY: these functions are the checker and the timed CPU
baseline, never a code path of the package.  Arguments are numpy arrays; the
reference lines each function follows are cited in the C source.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfeatgraph_ref.so")
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


def build(force=False):
    """Compile the checker with gcc (see oracle/Makefile)."""
    if force:
        subprocess.check_call(["make", "-s", "-C", _HERE, "clean"])
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        for name in ("fgref_spmm_csr_x86", "fgref_spmm_dds_x86", "fgref_sddmm_x86", "fgref_sddmm_x86_fast",
                     "fgref_spmm_csr_f64", "fgref_sddmm_f64", "fgref_sddmm_mh", "fgref_spmm_mh", "fgref_spmm_general",
                     "fgref_sddmm_general", "fgref_edge_softmax", "fgref_spmm_mh_general", "fgref_edge_softmax_backward"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def num_threads():
    return int(lib().fgref_num_threads())


def _arr(a, dtype):
    a = np.ascontiguousarray(a)
    if a.dtype != np.dtype(dtype):
        raise TypeError("expected %s, got %s" % (np.dtype(dtype), a.dtype))
    return a


def _ptr(a):
    return _p(a.ctypes.data)


def _check(status, what):
    if status != 0:
        raise RuntimeError("%s failed with status %d" % (what, status))


def spmm_csr_x86(indptr, indices, vals, src, num_feat_partitions=1, work=None):
    """Restated x86 CSR SpMM nest (op/vanilla_spmm.py:36-80).  Returns [n_dst, F] float32."""
    indptr, indices, vals = _arr(indptr, np.int32), _arr(indices, np.int32), _arr(vals, np.float32)
    src = _arr(src, np.float32)
    n_dst, (n_src, F) = indptr.shape[0] - 1, src.shape
    out = np.empty((n_dst, F), dtype=np.float32)
    wp = _p(None) if work is None else _ptr(work)
    _check(lib().fgref_spmm_csr_x86(_i64(n_dst), _i64(n_src), _i64(F), _i64(num_feat_partitions), _ptr(indptr),
                                    _ptr(indices), _ptr(vals), _ptr(src), _ptr(out), wp), "fgref_spmm_csr_x86")
    return out


def spmm_dds_x86(s1_pos, s1_idx, vals, src, n_dst, num_col_partitions, num_feat_partitions=1):
    """Restated x86 DDS SpMM nest (op/vanilla_spmm.py:188-246)."""
    s1_pos, s1_idx, vals = _arr(s1_pos, np.int32), _arr(s1_idx, np.int32), _arr(vals, np.float32)
    src = _arr(src, np.float32)
    n_src, F = src.shape
    assert s1_pos.shape[0] == num_col_partitions * (n_dst + 1)
    out = np.empty((n_dst, F), dtype=np.float32)
    _check(lib().fgref_spmm_dds_x86(_i64(n_dst), _i64(n_src), _i64(F), _i64(num_feat_partitions),
                                    _i64(num_col_partitions), _ptr(s1_pos), _ptr(s1_idx), _ptr(vals), _ptr(src),
                                    _ptr(out)), "fgref_spmm_dds_x86")
    return out


def sddmm_x86(row, col, src, dst, num_feat_partitions=1):
    """Restated x86 COO SDDMM nest (op/vanilla_sddmm.py:37-74).  src is indexed by col, dst by row."""
    row, col = _arr(row, np.int32), _arr(col, np.int32)
    src, dst = _arr(src, np.float32), _arr(dst, np.float32)
    nnz, F = row.shape[0], src.shape[1]
    assert col.shape[0] == nnz and dst.shape[1] == F
    out = np.empty(nnz, dtype=np.float32)
    _check(lib().fgref_sddmm_x86(_i64(nnz), _i64(dst.shape[0]), _i64(src.shape[0]), _i64(F),
                                 _i64(num_feat_partitions), _ptr(row), _ptr(col), _ptr(src), _ptr(dst), _ptr(out)),
           "fgref_sddmm_x86")
    return out


def sddmm_x86_fast(row, col, src, dst, parallel=False, out=None):
    """Timing-only SDDMM with a re-associated k reduction (and all cores when parallel)."""
    row, col = _arr(row, np.int32), _arr(col, np.int32)
    src, dst = _arr(src, np.float32), _arr(dst, np.float32)
    nnz, F = row.shape[0], src.shape[1]
    if out is None:
        out = np.empty(nnz, dtype=np.float32)
    _check(lib().fgref_sddmm_x86_fast(_i64(nnz), _i64(F), _ptr(row), _ptr(col), _ptr(src), _ptr(dst), _ptr(out),
                                      ctypes.c_int(1 if parallel else 0)), "fgref_sddmm_x86_fast")
    return out


def spmm_csr_f64(indptr, indices, vals, src):
    """CSR SpMM with binary64 products and sums of the float32 inputs."""
    indptr, indices, vals = _arr(indptr, np.int32), _arr(indices, np.int32), _arr(vals, np.float32)
    src = _arr(src, np.float32)
    n_dst, F = indptr.shape[0] - 1, src.shape[1]
    out = np.empty((n_dst, F), dtype=np.float64)
    _check(lib().fgref_spmm_csr_f64(_i64(n_dst), _i64(F), _ptr(indptr), _ptr(indices), _ptr(vals), _ptr(src),
                                    _ptr(out)), "fgref_spmm_csr_f64")
    return out


def sddmm_f64(row, col, src, dst):
    row, col = _arr(row, np.int32), _arr(col, np.int32)
    src, dst = _arr(src, np.float32), _arr(dst, np.float32)
    nnz = row.shape[0]
    F = int(np.prod(src.shape[1:]))
    out = np.empty(nnz, dtype=np.float64)
    _check(lib().fgref_sddmm_f64(_i64(nnz), _i64(F), _ptr(row), _ptr(col), _ptr(src), _ptr(dst), _ptr(out)),
           "fgref_sddmm_f64")
    return out


def sddmm_mh(row, col, src, dst):
    """Multi-head SDDMM closed form: src/dst [N,H,D] -> out [nnz,H]."""
    row, col = _arr(row, np.int32), _arr(col, np.int32)
    src, dst = _arr(src, np.float32), _arr(dst, np.float32)
    nnz, (_, H, D) = row.shape[0], src.shape
    assert dst.shape[1:] == (H, D)
    out = np.empty((nnz, H), dtype=np.float32)
    _check(lib().fgref_sddmm_mh(_i64(nnz), _i64(H), _i64(D), _ptr(row), _ptr(col), _ptr(src), _ptr(dst), _ptr(out)),
           "fgref_sddmm_mh")
    return out


def spmm_mh(indptr, indices, w, src):
    """Multi-head generalised SpMM closed form: w [nnz,H], src [N,H,D] -> out [n_dst,H,D]."""
    indptr, indices = _arr(indptr, np.int32), _arr(indices, np.int32)
    w, src = _arr(w, np.float32), _arr(src, np.float32)
    n_dst, (_, H, D) = indptr.shape[0] - 1, src.shape
    assert w.shape == (indices.shape[0], H)
    out = np.empty((n_dst, H, D), dtype=np.float32)
    _check(lib().fgref_spmm_mh(_i64(n_dst), _i64(H), _i64(D), _ptr(indptr), _ptr(indices), _ptr(w), _ptr(src),
                               _ptr(out)), "fgref_spmm_mh")
    return out


MSG_OPS = {"mul": 0, "add": 1, "sub": 2, "div": 3, "copy_u": 4}
REDUCE_OPS = {"sum": 0, "max": 1, "min": 2, "mean": 3}
EDGE_OPS = {"dot": 0, "add": 1, "sub": 2, "mul": 3, "div": 4}


def spmm_general(indptr, indices, vals, src, msg="mul", reduce="sum"):
    """Generalised SpMM: fold of msg(src[col], val) over each row in CSR order (see fgref_spmm_general)."""
    indptr, indices, vals = _arr(indptr, np.int32), _arr(indices, np.int32), _arr(vals, np.float32)
    src = _arr(src, np.float32)
    n_dst, F = indptr.shape[0] - 1, src.shape[1]
    out = np.empty((n_dst, F), dtype=np.float32)
    _check(lib().fgref_spmm_general(_i64(n_dst), _i64(F), _ptr(indptr), _ptr(indices), _ptr(vals), _ptr(src),
                                    _ptr(out), ctypes.c_int(MSG_OPS[msg]), ctypes.c_int(REDUCE_OPS[reduce])),
           "fgref_spmm_general")
    return out


def sddmm_general(row, col, src, dst, op):
    """Elementwise edge function: out[e, :] = src[col[e], :] op dst[row[e], :]; 'dot' is sddmm_x86."""
    if op == "dot":
        return sddmm_x86(row, col, src, dst)
    row, col = _arr(row, np.int32), _arr(col, np.int32)
    src, dst = _arr(src, np.float32), _arr(dst, np.float32)
    nnz, F = row.shape[0], src.shape[1]
    out = np.empty((nnz, F), dtype=np.float32)
    _check(lib().fgref_sddmm_general(_i64(nnz), _i64(F), _ptr(row), _ptr(col), _ptr(src), _ptr(dst), _ptr(out),
                                     ctypes.c_int(EDGE_OPS[op])), "fgref_sddmm_general")
    return out


def edge_softmax(indptr, scores):
    """Softmax of scores [nnz, H] over each destination row's edges, per head (binary64 inside)."""
    indptr, scores = _arr(indptr, np.int32), _arr(scores, np.float32)
    n_dst, H = indptr.shape[0] - 1, scores.shape[1]
    out = np.empty_like(scores)
    _check(lib().fgref_edge_softmax(_i64(n_dst), _i64(H), _ptr(indptr), _ptr(scores), _ptr(out)),
           "fgref_edge_softmax")
    return out


def spmm_mh_general(indptr, indices, w, src, msg="mul", reduce="sum"):
    """Multi-head generalised SpMM: w [nnz,H], src [N,H,D] -> fold of msg(src[col,h,:], w[e,h]) per row and head."""
    indptr, indices = _arr(indptr, np.int32), _arr(indices, np.int32)
    w, src = _arr(w, np.float32), _arr(src, np.float32)
    n_dst, (_, H, D) = indptr.shape[0] - 1, src.shape
    assert w.shape == (indices.shape[0], H)
    out = np.empty((n_dst, H, D), dtype=np.float32)
    _check(lib().fgref_spmm_mh_general(_i64(n_dst), _i64(H), _i64(D), _ptr(indptr), _ptr(indices), _ptr(w),
                                       _ptr(src), _ptr(out), ctypes.c_int(MSG_OPS[msg]),
                                       ctypes.c_int(REDUCE_OPS[reduce])), "fgref_spmm_mh_general")
    return out


def edge_softmax_backward(indptr, weights, grad):
    """Gradient for the scores of an edge softmax: weights * (grad - rowsum(weights * grad)), binary64 inside."""
    indptr, weights, grad = _arr(indptr, np.int32), _arr(weights, np.float32), _arr(grad, np.float32)
    assert weights.shape == grad.shape
    n_dst, H = indptr.shape[0] - 1, weights.shape[1]
    out = np.empty_like(weights)
    _check(lib().fgref_edge_softmax_backward(_i64(n_dst), _i64(H), _ptr(indptr), _ptr(weights), _ptr(grad),
                                             _ptr(out)), "fgref_edge_softmax_backward")
    return out


def attention_mh_backward(indptr, indices, key, query, value, dout):
    """Gradients (d_key, d_query, d_value) of attention_mh, composed from the checkers above.

    With A the attention weights, row[e] the destination row of edge e and T the transposed matrix:
      d_value[c] = sum_{e: col=c} A[e] * dout[row[e]]      spmm_mh over T with the weights in T's order
      G[e]       = <dout[row[e]], value[col[e]]>           sddmm_mh
      dS         = edge_softmax_backward(A, G)
      d_query[r] = sum_{e in row r} dS[e] * key[col[e]]    spmm_mh
      d_key[c]   = sum_{e: col=c} dS[e] * query[row[e]]    spmm_mh over T
    value None means key is also the value matrix: then d_key carries both contributions.
    """
    import scipy.sparse
    indptr, indices = _arr(indptr, np.int32), _arr(indices, np.int32)
    n_dst, n_src, nnz = indptr.shape[0] - 1, key.shape[0], indices.shape[0]
    row = np.repeat(np.arange(n_dst, dtype=np.int32), np.diff(indptr))
    weights = edge_softmax(indptr, sddmm_mh(row, indices, key, query))
    # transposed structure; `perm` lists the edges in the transposed matrix's CSR order (stable: by column, then CSR order)
    perm = np.argsort(indices, kind="stable")
    t_indptr = np.zeros(n_src + 1, dtype=np.int32)
    np.cumsum(np.bincount(indices, minlength=n_src), out=t_indptr[1:])
    t_indices = row[perm]
    val = key if value is None else value
    d_value = spmm_mh(t_indptr, t_indices, np.ascontiguousarray(weights[perm]), dout)
    grad_w = sddmm_mh(row, indices, val, dout)
    d_scores = edge_softmax_backward(indptr, weights, grad_w)
    d_query = spmm_mh(indptr, indices, d_scores, key)
    d_key = spmm_mh(t_indptr, t_indices, np.ascontiguousarray(d_scores[perm]), query)
    if value is None:
        return d_key + d_value, d_query, None
    return d_key, d_query, d_value


def attention_mh(indptr, indices, key, query, value=None):
    """out[r, h, :] = sum over row r's nonzeros e of softmax_e(key[indices[e], h] . query[r, h]) * value[indices[e], h, :].

    The three checkers above one after the other: sddmm_mh (scores, float32), edge_softmax (binary64 inside),
    spmm_mh (sequential float32 sum).  value defaults to key.  Rows without nonzeros give zeros.
    """
    indptr, indices = _arr(indptr, np.int32), _arr(indices, np.int32)
    row = np.repeat(np.arange(indptr.shape[0] - 1, dtype=np.int32), np.diff(indptr))
    weights = edge_softmax(indptr, sddmm_mh(row, indices, key, query))
    return spmm_mh(indptr, indices, weights, key if value is None else value)
