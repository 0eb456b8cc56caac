"""Generalised SpMM / SDDMM modules and the backward of vanilla SpMM on the HIP target.

The reference builds its operators around two slots, a message function folded by a reducer
(op/vanilla_spmm.py:46-53) and an edge function (op/vanilla_sddmm.py:43-47), and ships one instance of
each (multiply + sum, dot product) under the name "generalized SpMM / SDDMM" (README.md:6).  The classes
here fill the slots with the other operators; the call surface is that of the vanilla modules.
"""
import re

import torch

from .. import _lib
from ..runtime import NDArray, hip
from . import _common as C
from .sddmm import SDDMMbase, VanillaSDDMMhip
from .spmm import SpMMbase, VanillaSpMMhip

MSG_OPS = {"mul": 0, "add": 1, "sub": 2, "div": 3, "copy_u": 4}       # FG_MSG_* of include/featgraph_hip.h
REDUCE_OPS = {"sum": 0, "max": 1, "min": 2, "mean": 3}                # FG_REDUCE_*
EDGE_OPS = {"dot": 0, "add": 1, "sub": 2, "mul": 3, "div": 4}         # FG_EDGE_*


class GeneralizedSpMMhip(SpMMbase):
    """Out[r, :] = reduce over the row's nonzeros e of msg(SrcFeat[indices[e], :], vals[e]).

    msg in {'mul', 'add', 'sub', 'div', 'copy_u'} (u = gathered feature, e = edge value), reduce in
    {'sum', 'max', 'min', 'mean'}; rows without nonzeros give 0.  ('mul', 'sum') is VanillaSpMMhip bit for bit.
    """

    def __init__(self, adj_scipy, msg="mul", reduce="sum", num_col_partitions=None):
        if msg not in MSG_OPS:
            raise ValueError("msg must be one of %s, got %r" % (sorted(MSG_OPS), msg))
        if reduce not in REDUCE_OPS:
            raise ValueError("reduce must be one of %s, got %r" % (sorted(REDUCE_OPS), reduce))
        self._msg, self._reduce = msg, reduce
        super().__init__(adj_scipy, num_col_partitions)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        _, H, D, _ = self._parse_build(input_placeholders, compute_args, schedule_args)
        # the plan's own description tells which kernel the plain operator would take and whether (and into how
        # many) column blocks the matrix is cut
        plan_text = super().lower_to_ir(input_placeholders, compute_args, schedule_args)
        head = "spmm_csr_general rows=%d cols=%d nnz=%d D=%d | msg=%s reduce=%s | " % (
            self._num_rows, self._num_cols, self._nnz, D, self._msg, self._reduce)
        # the several-rows-per-wave kernel takes the call where it takes the plain one
        if "rows-per-wave" in plan_text and _lib.config_get("spmm.general_multi") != 0:
            return head + ("kernel=rows-per-wave with the message and the reducer in place of the multiply-add%s | %s" % (
                ", then one division per element" if self._reduce == "mean" else "", plan_text.split(" | ")[-1]))
        found = re.search(r"(\d+) column blocks of (\d+)", plan_text)
        passes = ("%s column blocks of %s, one launch per block, the fold carried in the output" % found.groups()
                  if found else "whole rows, 1 launch")
        return head + "kernel=row-slot, %s, rows=by-descending-degree, tile=64 floats x %d tiles" % (passes, (D + 63) // 64)

    def _launch(self, tensors):
        feat = tensors[0]
        _lib.check(_lib.lib().fg_spmm_csr_general_f32(
            self._plan, feat.data_ptr(), self._adj_vals_dev.data_ptr(), self.out_tvm.tensor.data_ptr(), self._D,
            MSG_OPS[self._msg], REDUCE_OPS[self._reduce], C.current_stream_handle(self._ctx)))


class MultiHeadGeneralizedSpMMhip(SpMMbase):
    """Out[r, h, :] = reduce over the row's nonzeros e of msg(SrcFeat[indices[e], h, :], EdgeWeight[e, h]): the
    generalised operator with per-edge per-head values (max / mean aggregation of a multi-head layer).

    build([SrcFeat (num_cols, H, D), EdgeWeight (nnz, H)], ...), run([feat, weight]); msg / reduce as for
    GeneralizedSpMMhip.  ('mul', 'sum') is MultiHeadSpMMhip bit for bit.  The CSR values of the matrix are not used.
    """

    _input_names = ("SrcFeat", "EdgeWeight")

    def __init__(self, adj_scipy, msg="mul", reduce="sum", num_col_partitions=None):
        if msg not in MSG_OPS:
            raise ValueError("msg must be one of %s, got %r" % (sorted(MSG_OPS), msg))
        if reduce not in REDUCE_OPS:
            raise ValueError("reduce must be one of %s, got %r" % (sorted(REDUCE_OPS), reduce))
        self._msg, self._reduce = msg, reduce
        super().__init__(adj_scipy, num_col_partitions)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def _heads_and_len(self, feat_shape):
        if len(feat_shape) != 3:
            raise ValueError("SrcFeat must be 3-D [num_src_vertices, num_heads, head_len], got %s" % (feat_shape,))
        return int(feat_shape[1]), int(feat_shape[2])

    def _parse_build(self, input_placeholders, compute_args, schedule_args):
        shapes, H, D, tiles = super()._parse_build(input_placeholders, compute_args, schedule_args)
        if shapes[1] != (self._nnz, H):
            raise ValueError("EdgeWeight must have shape (nnz, num_heads) = %s, got %s" % ((self._nnz, H), shapes[1]))
        return shapes, H, D, tiles

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        _, H, D, _ = self._parse_build(input_placeholders, compute_args, schedule_args)
        return ("spmm_csr_mh_general rows=%d cols=%d nnz=%d H=%d D=%d | msg=%s reduce=%s | kernel=row-slot, "
                "rows=by-descending-degree, %d floats/lane, tile=64 floats x %d tiles" % (
                    self._num_rows, self._num_cols, self._nnz, H, D, self._msg, self._reduce,
                    4 if D % 4 == 0 else 1, (H * D + 63) // 64))

    def _launch(self, tensors):
        feat, weight = tensors
        _lib.check(_lib.lib().fg_spmm_csr_mh_general_f32(
            self._plan, feat.data_ptr(), weight.data_ptr(), self.out_tvm.tensor.data_ptr(), self._H, self._D,
            MSG_OPS[self._msg], REDUCE_OPS[self._reduce], C.current_stream_handle(self._ctx)))


class GeneralizedSDDMMhip(SDDMMbase):
    """Out[e] = <SrcFeat[col[e]], DstFeat[row[e]]> for op 'dot' (VanillaSDDMMhip), otherwise the elementwise
    edge function Out[e, :] = SrcFeat[col[e], :] op DstFeat[row[e], :] with op in {'add', 'sub', 'mul', 'div'}
    and an output of shape [nnz, feat_len]."""

    def __init__(self, adj_scipy, op="dot", num_row_partitions=None, num_col_partitions=None):
        if op not in EDGE_OPS:
            raise ValueError("op must be one of %s, got %r" % (sorted(EDGE_OPS), op))
        self._op = op
        super().__init__(adj_scipy, num_row_partitions, num_col_partitions)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def build(self, input_placeholders, compute_args, schedule_args):
        super().build(input_placeholders, compute_args, schedule_args)
        if self._op != "dot":
            self.out_tvm = NDArray(torch.zeros((self._nnz, self._D), dtype=torch.float32, device=self._ctx))

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        if self._op == "dot":
            return super().lower_to_ir(input_placeholders, compute_args, schedule_args)
        _, _, D = self._parse_build(input_placeholders, compute_args, schedule_args)
        # the elementwise operators share the dot product's row-run schedule when the plan has one for the
        # caller's own list (a sorted copy would leave the [nnz, D] result in the copy's order)
        plan_text = super().lower_to_ir(input_placeholders, compute_args, schedule_args)
        if "row runs (row-sorted edge list)" in plan_text and D % 4 == 0:
            found = re.search(r"(\d+) column blocks of (\d+)", plan_text)
            return ("sddmm_coo_general nnz=%d D=%d | op=%s | kernel=row runs, Dst tile in registers, one store per "
                    "gathered Src tile, %s column blocks" % (self._nnz, D, self._op, found.group(1) if found else "?"))
        return "sddmm_coo_general nnz=%d D=%d | op=%s | kernel=thread per (edge, 4 floats), 1 launch" % (
            self._nnz, D, self._op)

    def _launch(self, tensors):
        if self._op == "dot":
            return super()._launch(tensors)
        src, dst = tensors
        _lib.check(_lib.lib().fg_sddmm_coo_general_plan_f32(
            self._plan, src.data_ptr(), dst.data_ptr(), self.out_tvm.tensor.data_ptr(), self._D, EDGE_OPS[self._op],
            C.current_stream_handle(self._ctx)))


class VanillaSpMMGradhip:
    """Backward of Out = A . X (VanillaSpMMhip) from the two vanilla kernels:

        dX    = A^T . dOut                         SpMM over the transposed matrix (the CSC arrays of A)
        dA[e] = <dOut[row[e]], X[col[e]]>          SDDMM over A's edge list: SrcFeat = X, DstFeat = dOut

    build([X placeholder (num_cols, F)], ...) fixes the feature length; run([x, dout]) returns (dX, dA) as the
    two module-owned arrays, dA in the order of A's CSR values.
    """

    def __init__(self, adj_scipy):
        csr = adj_scipy if getattr(adj_scipy, "format", None) == "csr" else adj_scipy.tocsr()
        self._shape = csr.shape
        transposed = csr.T.tocsr()           # canonical CSR of A^T: rows are A's columns, column ids ascend
        self.spmm_transposed = VanillaSpMMhip(transposed)
        self.sddmm = VanillaSDDMMhip(csr.tocoo())   # tocoo() keeps CSR order, so dA lines up with csr.data
        self._ctx = self.spmm_transposed.ctx

    def build(self, input_placeholders, compute_args=None, schedule_args=None):
        num_rows, num_cols = self._shape
        (x,) = input_placeholders
        F = int(x.shape[1])
        if int(x.shape[0]) != num_cols:
            raise ValueError("X has %d rows, the adjacency matrix %d columns" % (x.shape[0], num_cols))
        from ..runtime import placeholder
        self.spmm_transposed.build([placeholder((num_rows, F))], compute_args or {}, schedule_args or {})
        self.sddmm.build([placeholder((num_cols, F)), placeholder((num_rows, F))], {}, {})

    def run(self, input_tvm_ndarrays):
        x, dout = input_tvm_ndarrays
        return self.spmm_transposed.run([dout]), self.sddmm.run([x, dout])

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return "hip"
