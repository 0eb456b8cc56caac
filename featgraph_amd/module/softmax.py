"""Edge softmax on the HIP target, alone and fused into multi-head SDDMM.

Not in the reference.  In a GAT-style layer the scores of multi-head SDDMM are normalised over each
destination row's edges before multi-head SpMM uses them as weights; EdgeSoftmaxhip is that step on its
own, MultiHeadSDDMMSoftmaxhip computes the scores and normalises them in one kernel.  Both need the
edge list in CSR order (each destination row's edges consecutive), which is what scipy's tocsr() /
tocoo()-of-CSR produce.
"""
import numpy as np
import torch

from .. import _lib
from ..runtime import NDArray, hip
from . import _common as C
from .sddmm import SDDMMbase


def fused_layout(H, D):
    """(lanes per head, floats per load, chunks) of the fused score + softmax kernel for H heads of D floats, or
    None when it has no layout for the shape and the two operators run one after the other.  A vertex row is one
    or two chunks of 64 loads of 1, 2 or 4 floats, and a head spans 4, 8 or 16 lanes of a chunk:
    H = 8 with D in {8, 16, 32, 64}, H = 4 with D in {16, 32, 64}, H = 16 with D in {4, ..., 32}, ..."""
    for w in (4, 2, 1):
        if D % w:
            continue
        c = D // w
        if c not in (4, 8, 16) or H % (64 // c):
            continue
        n = H // (64 // c)
        if n in (1, 2) and c % n == 0:
            return c, w, n
    return None


class EdgeSoftmaxhip:
    """out[e, h] = softmax over the edges of e's destination row of scores[e, h].

    EdgeSoftmaxhip(adj).build([placeholder((nnz, H))], {}, {}); run([scores]) returns the module-owned [nnz, H]
    array.  The edge order is that of adj in CSR form.
    """

    def __init__(self, adj_scipy):
        csr = adj_scipy if getattr(adj_scipy, "format", None) == "csr" else adj_scipy.tocsr()
        self._num_rows, self._nnz = csr.shape[0], int(csr.nnz)
        self._ctx, self._target = hip(0), "hip"
        C.require_device()
        self._indptr_dev = torch.from_numpy(C.to_int32_index(csr.indptr, "indptr")).to(self._ctx)
        self._built = False
        self.out_tvm = None

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        (scores,) = input_placeholders
        shape = tuple(int(s) for s in scores.shape)
        if len(shape) != 2 or shape[0] != self._nnz or shape[1] < 1:
            raise ValueError("scores must have shape (nnz, num_heads) = (%d, H), got %s" % (self._nnz, shape))
        if str(scores.dtype) != "float32":
            raise TypeError("operands must be float32, got %s" % scores.dtype)
        self._shape = shape
        self.out_tvm = NDArray(torch.zeros(shape, dtype=torch.float32, device=self._ctx))
        self._built = True

    def _launch(self, scores):
        _lib.check(_lib.lib().fg_edge_softmax_csr_f32(
            self._num_rows, self._indptr_dev.data_ptr(), scores.data_ptr(), self.out_tvm.tensor.data_ptr(),
            self._shape[1], C.current_stream_handle(self._ctx)))

    def run(self, input_tvm_ndarrays):
        if not self._built:
            raise RuntimeError("call build() before run()")
        (scores,) = input_tvm_ndarrays
        t = C.check_operand(scores, self._shape, self._ctx, "scores")
        with torch.cuda.device(self._ctx):
            self._launch(t)
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        (scores,) = input_tvm_ndarrays
        t = C.check_operand(scores, self._shape, self._ctx, "scores")
        with torch.cuda.device(self._ctx):
            return C.time_calls(lambda: self._launch(t), self._ctx, num_runs)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class MultiHeadSDDMMSoftmaxhip(SDDMMbase):
    """Attention weights of a GAT-style layer in one step:
    Out[e, h] = softmax over the edges of row[e] of sum_d Src[col[e], h, d] * Dst[row[e], h, d].

    Operands [num_vertices, H, D], output [nnz, H]; the adjacency's edge list must be row-sorted (COO derived
    from CSR).  For the shapes fused_layout covers (8 heads of 8 .. 64 floats among them) a single fused kernel
    runs; other shapes run multi-head SDDMM and the edge softmax one after the other.
    """

    def __init__(self, adj_scipy):
        coo = adj_scipy if getattr(adj_scipy, "format", None) == "coo" else adj_scipy.tocsr().tocoo()
        if coo.nnz and np.any(np.diff(coo.row) < 0):
            raise ValueError("edge softmax needs a row-sorted edge list (pass a CSR matrix or a COO list derived from one)")
        super().__init__(coo)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def _heads_and_len(self, feat_shape):
        if len(feat_shape) != 3:
            raise ValueError("features must be 3-D [num_vertices, num_heads, head_len], got %s" % (feat_shape,))
        return int(feat_shape[1]), int(feat_shape[2])

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        _, H, D = self._parse_build(input_placeholders, compute_args, schedule_args)
        layout = fused_layout(H, D)
        return "sddmm_softmax nnz=%d H=%d D=%d | %s" % (
            self._nnz, H, D,
            "kernel=fused scores + softmax, one wave per destination row, %d lanes/head x %d floats, %d chunk(s), "
            "%d neighbours per step, rows by descending degree, 1 launch" % (
                layout[0], layout[1], layout[2], 64 // H) if layout else
            "multi-head SDDMM, then edge softmax in place (2 launches)")

    def _launch(self, tensors):
        src, dst = tensors
        _lib.check(_lib.lib().fg_sddmm_softmax_plan_f32(
            self._plan, src.data_ptr(), dst.data_ptr(), self.out_tvm.tensor.data_ptr(), self._H, self._D,
            C.current_stream_handle(self._ctx)))
