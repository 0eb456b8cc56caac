"""Multi-head attention over a sparse graph on the HIP target: multi-head SDDMM, edge softmax and multi-head
SpMM as one operator.

Not in the reference, which has the two ends as separate operators (the multi-head scores of
op/vanilla_sddmm.py:35-47 and the multi-head SpMM its benchmarks describe).  Run one after the other they
gather every neighbour's feature row twice and write and re-read the [nnz, H] edge weights; the fused kernel
keeps a running softmax per head, uses each gathered row for its score and for the weighted sum while it is in
registers, and never materialises scores or weights.  With one set of vertex features as key and value the whole
layer moves half the bytes.
"""
import torch

from .. import _lib
from ..runtime import NDArray, hip
from . import _common as C
from .softmax import MultiHeadSDDMMSoftmaxhip, fused_layout
from .spmm import MultiHeadSpMMhip, SpMMbase


class MultiHeadAttentionhip(SpMMbase):
    """Out[r, h, :] = sum over row r's nonzeros e of A[e, h] * Value[indices[e], h, :], with
    A[e, h] = softmax over the row's nonzeros of sum_d Key[indices[e], h, d] * Query[r, h, d].

    build([Key (num_cols, H, D), Query (num_rows, H, D)], ...) uses Key as Value too (each neighbour row is
    gathered once); build([Key, Query, Value], ...) takes a separate Value of Key's shape.  run() takes the same
    number of arrays and returns the module-owned [num_rows, H, D] output; rows without nonzeros give zeros.  The
    CSR values of the adjacency matrix are not used.  Shapes that the fused kernel has no layout for (see
    fused_layout) run MultiHeadSDDMMSoftmaxhip and MultiHeadSpMMhip one after the other.
    """

    _input_names = ("KeyFeat", "QueryFeat", "ValueFeat")

    def __init__(self, adj_scipy, num_col_partitions=None):
        super().__init__(adj_scipy, num_col_partitions)
        self._adj = adj_scipy
        self._chain = None

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def _parse_build(self, input_placeholders, compute_args, schedule_args):
        C.check_known_keys(compute_args, (), "compute_args")
        C.check_known_keys(schedule_args, ("num_cuda_blocks", "num_threads_per_cuda_block"), "schedule_args")
        if len(input_placeholders) not in (2, 3):
            raise ValueError("expected placeholders for KeyFeat, QueryFeat and optionally ValueFeat")
        shapes = [tuple(int(s) for s in p.shape) for p in input_placeholders]
        for p in input_placeholders:
            if str(p.dtype) != "float32":
                raise TypeError("operands must be float32, got %s" % p.dtype)
        key, query = shapes[0], shapes[1]
        if len(key) != 3 or min(key[1:]) < 1:
            raise ValueError("KeyFeat must be 3-D [num_src_vertices, num_heads, head_len], got %s" % (key,))
        if key[0] != self._num_cols:
            raise ValueError("KeyFeat has %d rows, the adjacency matrix %d columns" % (key[0], self._num_cols))
        if query != (self._num_rows,) + key[1:]:
            raise ValueError("QueryFeat must have shape %s, got %s" % ((self._num_rows,) + key[1:], query))
        if len(shapes) == 3 and shapes[2] != key:
            raise ValueError("ValueFeat must have KeyFeat's shape %s, got %s" % (key, shapes[2]))
        return shapes, key[1], key[2], 0

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        shapes, H, D, _ = self._parse_build(input_placeholders, compute_args, schedule_args)
        self._input_shapes = shapes
        self._H, self._D = H, D
        self.out_tvm = NDArray(torch.zeros((self._num_rows, H, D), dtype=torch.float32, device=self._ctx))
        self._chain = None
        if fused_layout(H, D) is None:
            scores = MultiHeadSDDMMSoftmaxhip(self._adj)
            scores.build(input_placeholders[:2], {}, {})
            spmm = MultiHeadSpMMhip(self._adj)
            spmm.build([input_placeholders[0], scores.out_tvm], {}, {})
            self._chain = (scores, spmm)
            self.out_tvm = spmm.out_tvm
        self._built = True

    def lower_to_ir(self, input_placeholders, compute_args=None, schedule_args=None):
        shapes, H, D, _ = self._parse_build(input_placeholders, compute_args, schedule_args)
        layout = fused_layout(H, D)
        if layout is None:
            return "attention nnz=%d H=%d D=%d | multi-head SDDMM + softmax, then multi-head SpMM" % (self._nnz, H, D)
        per_batch = min(8, 32 // (layout[1] * layout[2])) // (1 if len(shapes) == 2 else 2)
        return ("attention nnz=%d H=%d D=%d | kernel=fused scores + softmax + weighted sum, one wave per destination "
                "row, %d lanes/head x %d floats, %d chunk(s), two batches of %d neighbours in flight, %s, rows by "
                "descending degree, 1 launch" % (
                    self._nnz, H, D, layout[0], layout[1], layout[2], per_batch,
                    "one gather per neighbour (value is key)" if len(shapes) == 2 else "key and value gathered"))

    def _launch(self, tensors):
        key, query = tensors[0], tensors[1]
        value = tensors[2] if len(tensors) == 3 else key
        if self._chain is not None:
            scores, spmm = self._chain
            scores._launch((key, query))
            spmm._launch((value, scores.out_tvm.tensor))
            return
        _lib.check(_lib.lib().fg_attention_csr_mh_f32(
            self._plan, key.data_ptr(), query.data_ptr(), value.data_ptr(), self.out_tvm.tensor.data_ptr(),
            self._H, self._D, C.current_stream_handle(self._ctx)))
