"""SDDMM module classes on the HIP target.

Same call surface as the reference's featgraph.module.sddmm (SDDMMbase
module/sddmm.py:11-165, VanillaSDDMMcuda :179-187).  Operand naming follows the
reference's tests, not its docstring: SrcFeat has one row per COLUMN of the
adjacency matrix and DstFeat one per ROW (tests/test_module_sddmm.py:18-19,
op/vanilla_sddmm.py:47).
"""
import ctypes

import numpy as np
import torch

from .. import _lib
from ..runtime import NDArray, hip
from . import _common as C


def normalize_coo(adj_scipy):
    """COO view of the input with int32 row / col arrays (host side); module/sddmm.py:28-33, :51-52.
    Edge values are never read.  Returns (row, col, shape)."""
    if not hasattr(adj_scipy, "format"):
        raise TypeError("adjacency must be a scipy sparse matrix, got %s" % type(adj_scipy).__name__)
    coo = adj_scipy if adj_scipy.format == "coo" else adj_scipy.tocoo()
    num_rows, num_cols = coo.shape
    row = C.to_int32_index(coo.row, "row")
    col = C.to_int32_index(coo.col, "col")
    if row.shape[0] != col.shape[0]:
        raise ValueError("row and col differ in length")  # op/vanilla_sddmm.py:40
    C.check_index_range(row, num_rows, "row")
    C.check_index_range(col, num_cols, "col")
    return row, col, (num_rows, num_cols)


class SDDMMbase:
    """Base class of the SDDMM-like modules (reference: module/sddmm.py:11-165)."""

    def __init__(self, adj_scipy, num_row_partitions=None, num_col_partitions=None):
        """Partition counts as in the reference (module/sddmm.py:13-26).  On this target cache blocking is by
        column blocks only (the row dimension is already local in a row-sorted edge list): num_col_partitions
        None lets the library decide, 1 turns blocking off, P > 1 asks for P blocks; num_row_partitions is
        checked and otherwise unused.  Outputs always come in the caller's edge order."""
        if num_row_partitions is not None:
            assert num_row_partitions >= 1, "num_row_partitions should be larger than or equal to 1"
        if num_col_partitions is not None:
            assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
        row, col, (self._num_rows, self._num_cols) = normalize_coo(adj_scipy)
        self._num_row_partitions = num_row_partitions or 1
        self._num_col_partitions = num_col_partitions or 1
        self._nnz = int(row.shape[0])
        self._target = None
        self._ctx = None
        self._register()
        C.require_device()
        self._adj_row_dev = torch.from_numpy(row).to(self._ctx)  # one upload per module (module/sddmm.py:59-60)
        self._adj_col_dev = torch.from_numpy(col).to(self._ctx)
        # the cache-blocking step that the reference's constructor runs as 2-D partitioning on the host
        # (module/sddmm.py:45-49) is a column-block plan on the device here; outputs stay in edge order
        self._plan = ctypes.c_void_p()
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_sddmm_plan_create_partitioned(
                self._nnz, self._num_rows, self._num_cols, self._adj_row_dev.data_ptr(),
                self._adj_col_dev.data_ptr(), int(num_col_partitions or 0), ctypes.byref(self._plan)))
        self._built = False
        self.out_tvm = None

    def __del__(self):
        plan = getattr(self, "_plan", None)
        if plan:
            try:
                _lib.lib().fg_sddmm_plan_destroy(plan)
            except Exception:
                pass
            self._plan = None

    def _register(self):
        raise NotImplementedError("Please register target and ctx.")

    def _heads_and_len(self, feat_shape):
        if len(feat_shape) != 2:
            raise ValueError("features must be 2-D [num_vertices, feat_len], got %s" % (feat_shape,))
        return 1, int(feat_shape[1])

    def _parse_build(self, input_placeholders, compute_args, schedule_args):
        compute_args = C.check_known_keys(compute_args, ("num_feat_partitions",), "compute_args")
        schedule_args = C.check_known_keys(
            schedule_args, ("num_feat_partitions", "num_cuda_blocks", "num_threads_per_cuda_block"), "schedule_args")
        # num_feat_partitions (op/vanilla_sddmm.py:49, tests/test_module_sddmm.py:21-22): the x86 operator splits
        # the reduction axis into P tiles; the reference's CUDA schedules refuse that (op/vanilla_sddmm.py:79-80)
        # because their tiles would need a reduction across workgroups.  The kernels here tile long feature rows
        # themselves (64 floats per tile, partial sums added tile by tile in one stream), so any P that divides the
        # feature length is accepted; it does not change the tile width.
        tiles = [int(args.get("num_feat_partitions") or 1) for args in (compute_args, schedule_args)]
        if min(tiles) < 1:
            raise ValueError("num_feat_partitions must be positive")
        if len(input_placeholders) != 2:
            raise ValueError("expected placeholders [SrcFeat, DstFeat]")
        for p in input_placeholders:
            if str(p.dtype) != "float32":
                raise TypeError("operands must be float32, got %s" % p.dtype)
        src_shape, dst_shape = (tuple(int(s) for s in p.shape) for p in input_placeholders)
        assert src_shape[1:] == dst_shape[1:], "dimension mismatch"  # op/vanilla_sddmm.py:38
        if src_shape[0] != self._num_cols:
            raise ValueError("SrcFeat has %d rows, the adjacency matrix %d columns" % (src_shape[0], self._num_cols))
        if dst_shape[0] != self._num_rows:
            raise ValueError("DstFeat has %d rows, the adjacency matrix %d rows" % (dst_shape[0], self._num_rows))
        H, D = self._heads_and_len(src_shape)
        if H * D < 1:
            raise ValueError("feature length must be positive")
        for P in tiles:
            if (H * D) % P != 0:
                # the reference assumes this silently (op/vanilla_sddmm.py:49)
                raise ValueError("feat_len %d is not a multiple of num_feat_partitions %d" % (H * D, P))
        return [src_shape, dst_shape], H, D

    def build(self, input_placeholders, compute_args, schedule_args):
        """Fix operand shapes and allocate the (zero-filled, reused) output: module/sddmm.py:72-92.
        The reference's CUDA launch keys in schedule_args are accepted and ignored; num_feat_partitions in either
        dict must divide the feature length and is otherwise informational (see _parse_build)."""
        shapes, H, D = self._parse_build(input_placeholders, compute_args, schedule_args)
        self._input_shapes = shapes
        self._H, self._D = H, D
        out_shape = (self._nnz,) if len(shapes[0]) == 2 else (self._nnz, H)
        self.out_tvm = NDArray(torch.zeros(out_shape, dtype=torch.float32, device=self._ctx))
        self._padded = None
        pitch = self._row_pitch(shapes, H, D)
        if pitch:
            self._padded = (torch.zeros((self._num_cols, pitch), dtype=torch.float32, device=self._ctx),
                            torch.zeros((self._num_rows, pitch), dtype=torch.float32, device=self._ctx))
        self._built = True

    _pads_rows = False

    def _describe(self, H, D):
        buf = ctypes.create_string_buffer(1024)
        _lib.check(_lib.lib().fg_sddmm_plan_describe(self._plan, H, D, buf, len(buf)))
        return buf.value.decode()

    def _row_pitch(self, shapes, H, D):
        """Floats per row of the padded copies of both feature matrices that a run gathers from, or 0 for none: rows
        beyond 64 floats whose length is not a multiple of 32 floats (a 128-byte cache line) are copied at every run
        to rows that are, as VanillaSpMMhip does.  Only the row-run kernel reads rows at a pitch."""
        if (not self._pads_rows or len(shapes[0]) != 2 or H != 1 or D <= 64 or D % 32 == 0
                or _lib.config_get("spmm.pad_rows") == 0):
            return 0
        if D % 32 < 4 or 96 < D < 128:
            # measured on the 114.6M-edge graph: where the row's last four floats would lie across a line in every
            # padded row (65 / 130 floats: 5.1 / 6.7 against 3.5 / 5.1 ms) and where one partly filled 128-float tile
            # takes the row anyway (100 floats: 3.4 against 3.2) the two copies cost more than they save
            return 0
        return (D + 31) // 32 * 32 if "row runs" in self._describe(H, D) else 0

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        """Description of the launch (module/sddmm.py:94-113 returns TVM IR)."""
        shapes, H, D = self._parse_build(input_placeholders, compute_args, schedule_args)
        pitch = self._row_pitch(shapes, H, D)
        return self._describe(H, D) + (" | feature rows copied to a pitch of %d floats at every run" % pitch if pitch else "")

    def _launch(self, tensors):
        src, dst = tensors
        stream = C.current_stream_handle(self._ctx)
        if self._padded is not None:
            src_p, dst_p = self._padded
            pitch = src_p.shape[1]
            _lib.check(_lib.lib().fg_pad_rows_f32(self._num_cols, self._D, pitch, src.data_ptr(), src_p.data_ptr(), stream))
            _lib.check(_lib.lib().fg_pad_rows_f32(self._num_rows, self._D, pitch, dst.data_ptr(), dst_p.data_ptr(), stream))
            status = _lib.lib().fg_sddmm_coo_plan_pitched_f32(
                self._plan, src_p.data_ptr(), dst_p.data_ptr(), pitch, self.out_tvm.tensor.data_ptr(), self._D, stream)
            if status != _lib.FG_EUNSUPPORTED:        # a tuning key switched the kernel off after build: the plain call
                _lib.check(status)
                return
        _lib.check(_lib.lib().fg_sddmm_coo_plan_f32(
            self._plan, src.data_ptr(), dst.data_ptr(), self.out_tvm.tensor.data_ptr(), self._H, self._D, stream))

    def _checked_inputs(self, input_ndarrays):
        if not self._built:
            raise RuntimeError("call build() before run()")
        if len(input_ndarrays) != 2:
            raise ValueError("expected input arrays [src_feat, dst_feat]")
        return [C.check_operand(x, s, self._ctx, n)
                for x, s, n in zip(input_ndarrays, self._input_shapes, ("SrcFeat", "DstFeat"))]

    def run(self, input_tvm_ndarrays):
        """Enqueue the kernel and return the module-owned output (one float per edge,
        in the order of the adjacency's row / col arrays): module/sddmm.py:115-129."""
        tensors = self._checked_inputs(input_tvm_ndarrays)
        with torch.cuda.device(self._ctx):
            self._launch(tensors)
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        """Average seconds per run over num_runs runs after one warm-up (module/sddmm.py:131-150)."""
        tensors = self._checked_inputs(input_tvm_ndarrays)
        with torch.cuda.device(self._ctx):
            return C.time_calls(lambda: self._launch(tensors), self._ctx, num_runs)

    @property
    def edge_mapping(self):
        """Permutation that puts run() results back into the caller's edge order (module/sddmm.py:152-157,
        tests/test_module_sddmm.py:31-32).  Results here are already in that order, so it is the identity;
        like the reference it exists only when partitioning was asked for."""
        assert self._num_row_partitions > 1 or self._num_col_partitions > 1, \
            "no graph partitioning, no edge_mapping"
        return np.arange(self._nnz)

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class VanillaSDDMMhip(SDDMMbase):
    """COO SDDMM on the GPU.  VanillaSDDMMhip(adj) is the call of VanillaSDDMMcuda (module/sddmm.py:179-181);
    the optional partition counts are the arguments of VanillaSDDMMx86 (:169)."""

    _pads_rows = True

    def __init__(self, adj_scipy, num_row_partitions=None, num_col_partitions=None):
        super().__init__(adj_scipy, num_row_partitions, num_col_partitions)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)


class MultiHeadSDDMMhip(SDDMMbase):
    """Per-head dot products (GAT attention scores): Out[e,h] = sum_d Src[col[e],h,d] * Dst[row[e],h,d].

    Not in the reference; operands are [num_vertices, H, D], the output [nnz, H].
    """

    def __init__(self, adj_scipy):
        super().__init__(adj_scipy)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)

    def _heads_and_len(self, feat_shape):
        if len(feat_shape) != 3:
            raise ValueError("features must be 3-D [num_vertices, num_heads, head_len], got %s" % (feat_shape,))
        return int(feat_shape[1]), int(feat_shape[2])
