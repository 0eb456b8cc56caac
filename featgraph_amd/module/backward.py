"""Backward of the multi-head operators on the HIP target.

Not in the reference, which ships forward kernels only; README.md:6 names generalised SpMM / SDDMM as the
building blocks of GNN layers, and training a GAT-style layer needs the gradients of the three steps multi-head
SDDMM -> edge softmax -> multi-head SpMM.  They are again calls of the same kernels, over the matrix or its
transpose (T = A^T in CSR form, `perm` the position in A's CSR arrays of every entry of T's):

    Out[r,h,:] = sum_e W[e,h] * X[col[e],h,:]      dX[c] = sum_{e: col[e]=c} W[e] * dOut[row[e]]   SpMM over T, weights W[perm]
                                                    dW[e] = <dOut[row[e]], X[col[e]]>               SDDMM (Src = X, Dst = dOut)
    S[e,h]     = <Src[col[e],h], Dst[row[e],h]>    dSrc[c] = sum_{e: col[e]=c} dS[e] * Dst[row[e]]  SpMM over T, weights dS[perm]
                                                    dDst[r] = sum_{e in row r} dS[e] * Src[col[e]]   SpMM over A, weights dS
    A = softmax of S over each row's edges          dS[e] = A[e] * (G[e] - sum_{e' in the row} A[e'] * G[e'])

Every class keeps the reference's module shape: construct with a scipy matrix, build with operand placeholders,
run with device arrays; run returns module-owned arrays that the next run overwrites.
"""
import numpy as np
import torch

from .. import _lib
from ..runtime import NDArray, hip, placeholder
from . import _common as C
from .sddmm import MultiHeadSDDMMhip
from .softmax import MultiHeadSDDMMSoftmaxhip
from .spmm import MultiHeadSpMMhip


def _as_csr(adj_scipy):
    return adj_scipy if getattr(adj_scipy, "format", None) == "csr" else adj_scipy.tocsr()


def transpose_with_permutation(csr):
    """(T, perm): T = csr^T in CSR form with ascending column ids inside each row, perm[i] = position in csr's
    arrays of T's i-th entry (entries of one column of csr keep their order, so the sort is stable)."""
    import scipy.sparse
    n_rows, n_cols = csr.shape
    indices = np.asarray(csr.indices)
    perm = np.argsort(indices, kind="stable").astype(np.int32)
    t_indptr = np.zeros(n_cols + 1, dtype=np.int64)
    np.cumsum(np.bincount(indices, minlength=n_cols), out=t_indptr[1:])
    rows = np.repeat(np.arange(n_rows, dtype=np.int32), np.diff(csr.indptr))
    t = scipy.sparse.csr_matrix((np.asarray(csr.data, dtype=np.float32)[perm], rows[perm], t_indptr.astype(np.int32)),
                                shape=(n_cols, n_rows))
    return t, perm


class _TransposedSpMM:
    """sum over the entries of column c of A of weight[e, :] * feat[row[e], :, :]: multi-head SpMM over A^T with
    the per-edge weights carried into A^T's order first (fg_permute_rows_f32)."""

    def __init__(self, csr, ctx):
        transposed, perm = transpose_with_permutation(csr)
        self._nnz = int(csr.nnz)
        self._ctx = ctx
        self.spmm = MultiHeadSpMMhip(transposed)
        self._perm_dev = torch.from_numpy(perm).to(ctx)
        self._weights_t = None
        self._num_src = csr.shape[0]

    def build(self, H, D):
        self._H = H
        self._weights_t = NDArray(torch.zeros((self._nnz, H), dtype=torch.float32, device=self._ctx))
        self.spmm.build([placeholder((self._num_src, H, D)), placeholder((self._nnz, H))], {}, {})

    def launch(self, feat, weights):
        _lib.check(_lib.lib().fg_permute_rows_f32(self._nnz, self._H, self._perm_dev.data_ptr(), weights.data_ptr(),
                                                  self._weights_t.tensor.data_ptr(), C.current_stream_handle(self._ctx)))
        self.spmm._launch((feat, self._weights_t.tensor))
        return self.spmm.out_tvm


class _GradBase:
    _target = "hip"

    def __init__(self, adj_scipy):
        self._csr = _as_csr(adj_scipy)
        self._num_rows, self._num_cols = self._csr.shape
        self._nnz = int(self._csr.nnz)
        self._ctx = hip(0)
        C.require_device()
        self._built = False

    def _shapes(self, placeholders, expected):
        shapes = [tuple(int(s) for s in p.shape) for p in placeholders]
        for p in placeholders:
            if str(p.dtype) != "float32":
                raise TypeError("operands must be float32, got %s" % p.dtype)
        if len(shapes) != len(expected):
            raise ValueError("expected placeholders for %s" % (expected,))
        return shapes

    def _checked(self, arrays, shapes, names):
        if not self._built:
            raise RuntimeError("call build() before run()")
        if len(arrays) != len(shapes):
            raise ValueError("expected %d input arrays (%s)" % (len(shapes), ", ".join(names)))
        return [C.check_operand(x, s, self._ctx, n) for x, s, n in zip(arrays, shapes, names)]

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        tensors = self._checked(input_tvm_ndarrays, self._run_shapes, self._run_names)
        with torch.cuda.device(self._ctx):
            return C.time_calls(lambda: self._launch(tensors), self._ctx, num_runs)

    def run(self, input_tvm_ndarrays):
        tensors = self._checked(input_tvm_ndarrays, self._run_shapes, self._run_names)
        with torch.cuda.device(self._ctx):
            return self._launch(tensors)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class EdgeSoftmaxGradhip(_GradBase):
    """dScores = Weights * (Grad - rowsum(Weights * Grad)) for the weights of EdgeSoftmaxhip and the gradient that
    arrives for them.  build([placeholder((nnz, H))], ...); run([weights, grad]) returns the [nnz, H] result."""

    _run_names = ("Weights", "Grad")

    def __init__(self, adj_scipy):
        super().__init__(adj_scipy)
        self._indptr_dev = torch.from_numpy(C.to_int32_index(self._csr.indptr, "indptr")).to(self._ctx)
        self.out_tvm = None

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        (shape,) = self._shapes(input_placeholders[:1], ("Weights",))
        if len(shape) != 2 or shape[0] != self._nnz or shape[1] < 1:
            raise ValueError("weights must have shape (nnz, num_heads) = (%d, H), got %s" % (self._nnz, shape))
        self._run_shapes = (shape, shape)
        self.out_tvm = NDArray(torch.zeros(shape, dtype=torch.float32, device=self._ctx))
        self._built = True

    def _launch(self, tensors):
        weights, grad = tensors
        _lib.check(_lib.lib().fg_edge_softmax_backward_csr_f32(
            self._num_rows, self._indptr_dev.data_ptr(), weights.data_ptr(), grad.data_ptr(),
            self.out_tvm.tensor.data_ptr(), self._run_shapes[0][1], C.current_stream_handle(self._ctx)))
        return self.out_tvm


class MultiHeadSpMMGradhip(_GradBase):
    """Backward of MultiHeadSpMMhip.  build([SrcFeat (num_cols, H, D), EdgeWeight (nnz, H)], ...);
    run([feat, weight, dout]) with dout [num_rows, H, D] returns (dFeat [num_cols, H, D], dWeight [nnz, H])."""

    _run_names = ("SrcFeat", "EdgeWeight", "OutGrad")

    def __init__(self, adj_scipy):
        super().__init__(adj_scipy)
        self._over_transpose = _TransposedSpMM(self._csr, self._ctx)
        self._sddmm = MultiHeadSDDMMhip(self._csr.tocoo())     # tocoo() keeps CSR order: dWeight lines up with W

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        feat, weight = self._shapes(input_placeholders, ("SrcFeat", "EdgeWeight"))
        if len(feat) != 3 or feat[0] != self._num_cols:
            raise ValueError("SrcFeat must have shape (%d, H, D), got %s" % (self._num_cols, feat))
        H, D = feat[1], feat[2]
        if weight != (self._nnz, H):
            raise ValueError("EdgeWeight must have shape %s, got %s" % ((self._nnz, H), weight))
        self._run_shapes = (feat, weight, (self._num_rows, H, D))
        self._over_transpose.build(H, D)
        self._sddmm.build([placeholder(feat), placeholder((self._num_rows, H, D))], {}, {})
        self._built = True

    def _launch(self, tensors):
        feat, weight, dout = tensors
        d_feat = self._over_transpose.launch(dout, weight)
        self._sddmm._launch((feat, dout))
        return d_feat, self._sddmm.out_tvm


class MultiHeadSDDMMGradhip(_GradBase):
    """Backward of MultiHeadSDDMMhip over a row-sorted edge list (CSR order).  build([SrcFeat (num_cols, H, D),
    DstFeat (num_rows, H, D)], ...); run([src, dst, dscores]) with dscores [nnz, H] returns (dSrc, dDst)."""

    _run_names = ("SrcFeat", "DstFeat", "ScoreGrad")

    def __init__(self, adj_scipy):
        super().__init__(adj_scipy)
        self._over_transpose = _TransposedSpMM(self._csr, self._ctx)
        self._over_matrix = MultiHeadSpMMhip(self._csr)

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        src, dst = self._shapes(input_placeholders, ("SrcFeat", "DstFeat"))
        if len(src) != 3 or src[0] != self._num_cols:
            raise ValueError("SrcFeat must have shape (%d, H, D), got %s" % (self._num_cols, src))
        H, D = src[1], src[2]
        if dst != (self._num_rows, H, D):
            raise ValueError("DstFeat must have shape %s, got %s" % ((self._num_rows, H, D), dst))
        self._run_shapes = (src, dst, (self._nnz, H))
        self._over_transpose.build(H, D)
        self._over_matrix.build([placeholder(src), placeholder((self._nnz, H))], {}, {})
        self._built = True

    def _launch(self, tensors):
        src, dst, dscores = tensors
        d_src = self._over_transpose.launch(dst, dscores)
        self._over_matrix._launch((src, dscores))
        return d_src, self._over_matrix.out_tvm


class MultiHeadAttentionGradhip(_GradBase):
    """Backward of MultiHeadAttentionhip.  build([Key (num_cols, H, D), Query (num_rows, H, D)], ...) for a layer
    whose key is also its value, build([Key, Query, Value], ...) for a separate value matrix; run([key, query,
    (value,) dout]) returns (dKey, dQuery, dValue) -- dValue None, and its contribution folded into dKey, when the
    key is the value.  The attention weights are recomputed (scores + softmax in one kernel) rather than kept
    from the forward pass; seven kernels run one after the other on the caller's stream."""

    def __init__(self, adj_scipy):
        super().__init__(adj_scipy)
        self._weights = MultiHeadSDDMMSoftmaxhip(self._csr)
        self._weight_grad = MultiHeadSDDMMhip(self._csr.tocoo())
        self._softmax_grad = EdgeSoftmaxGradhip(self._csr)
        self._value_over_transpose = _TransposedSpMM(self._csr, self._ctx)
        self._key_over_transpose = _TransposedSpMM(self._csr, self._ctx)
        self._query_over_matrix = MultiHeadSpMMhip(self._csr)

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        shapes = [tuple(int(s) for s in p.shape) for p in input_placeholders]
        if len(shapes) not in (2, 3):
            raise ValueError("expected placeholders for KeyFeat, QueryFeat and optionally ValueFeat")
        self._shapes(input_placeholders, shapes)
        key, query = shapes[0], shapes[1]
        if len(key) != 3 or key[0] != self._num_cols:
            raise ValueError("KeyFeat must have shape (%d, H, D), got %s" % (self._num_cols, key))
        H, D = key[1], key[2]
        if query != (self._num_rows, H, D):
            raise ValueError("QueryFeat must have shape %s, got %s" % ((self._num_rows, H, D), query))
        if len(shapes) == 3 and shapes[2] != key:
            raise ValueError("ValueFeat must have KeyFeat's shape %s, got %s" % (key, shapes[2]))
        self._shared = len(shapes) == 2
        self._run_shapes = tuple(shapes) + ((self._num_rows, H, D),)
        self._run_names = ("KeyFeat", "QueryFeat") + (() if self._shared else ("ValueFeat",)) + ("OutGrad",)
        scores_ph = placeholder((self._nnz, H))
        self._weights.build([placeholder(key), placeholder(query)], {}, {})
        self._weight_grad.build([placeholder(key), placeholder(query)], {}, {})
        self._softmax_grad.build([scores_ph], {}, {})
        self._value_over_transpose.build(H, D)
        self._key_over_transpose.build(H, D)
        self._query_over_matrix.build([placeholder(key), scores_ph], {}, {})
        self._built = True

    def _launch(self, tensors):
        key, query, dout = tensors[0], tensors[1], tensors[-1]
        value = key if self._shared else tensors[2]
        self._weights._launch((key, query))                                    # A
        weights = self._weights.out_tvm.tensor
        d_value = self._value_over_transpose.launch(dout, weights)              # dValue = T-SpMM(A, dOut)
        self._weight_grad._launch((value, dout))                                # G = <dOut[row], Value[col]>
        d_scores = self._softmax_grad._launch((weights, self._weight_grad.out_tvm.tensor)).tensor
        self._query_over_matrix._launch((key, d_scores))                        # dQuery = SpMM(dS, Key)
        d_key = self._key_over_transpose.launch(query, d_scores)                # dKey = T-SpMM(dS, Query)
        if self._shared:
            _lib.check(_lib.lib().fg_add_f32(d_key.tensor.numel(), d_key.tensor.data_ptr(), d_value.tensor.data_ptr(),
                                             d_key.tensor.data_ptr(), C.current_stream_handle(self._ctx)))
            return d_key, self._query_over_matrix.out_tvm, None
        return d_key, self._query_over_matrix.out_tvm, d_value
