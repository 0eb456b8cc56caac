"""SpMM module classes on the HIP target.

Same call surface as the reference's featgraph.module.spmm (module/spmm.py:
SpMMbase :12-195, VanillaSpMMcuda :212-220): construct with a scipy matrix,
`build` with operand placeholders and two argument dicts, `run` /
`measure_average_time` with device arrays.  What the reference delegates to
TVM (code generation, module/spmm.py:105-109) is a prebuilt HIP library here,
so `build` only fixes shapes, picks the feature tiling and allocates the
output once; the adjacency arrays are uploaded once in the constructor.
"""
import ctypes

import numpy as np
import torch

from .. import _lib
from ..runtime import NDArray, hip
from . import _common as C


def normalize_csr(adj_scipy):
    """CSR view of the input with int32 index arrays and float32 values (host side).

    Follows module/spmm.py:26-31: non-CSR input is converted with .tocsr(); the
    arrays are otherwise taken as they are (no sorting, no merging of
    duplicate columns).  Returns (indptr, indices, data, shape).
    """
    if not hasattr(adj_scipy, "format"):
        raise TypeError("adjacency must be a scipy sparse matrix, got %s" % type(adj_scipy).__name__)
    csr = adj_scipy if adj_scipy.format == "csr" else adj_scipy.tocsr()
    num_rows, num_cols = csr.shape
    indptr = C.to_int32_index(csr.indptr, "indptr")
    indices = C.to_int32_index(csr.indices, "indices")
    data = np.ascontiguousarray(csr.data, dtype=np.float32)
    if indptr.shape[0] != num_rows + 1:
        raise ValueError("indptr has %d entries for %d rows" % (indptr.shape[0], num_rows))
    if indices.shape[0] != data.shape[0]:
        raise ValueError("indices and data differ in length")  # op/vanilla_spmm.py:36
    if indptr[0] != 0 or indptr[-1] != indices.shape[0] or np.any(np.diff(indptr) < 0):
        raise ValueError("indptr is not a non-decreasing sequence from 0 to nnz")
    C.check_index_range(indices, num_cols, "indices")
    return indptr, indices, data, (num_rows, num_cols)


class SpMMbase:
    """Base class of the SpMM-like modules (reference: module/spmm.py:12-195)."""

    _input_names = ("SrcFeat",)

    def __init__(self, adj_scipy, num_col_partitions=None):
        """num_col_partitions: the reference's 1-D source-vertex partitioning (module/spmm.py:14-24).  On this
        target it selects the number of column blocks of the L2-blocked passes: None lets the library decide
        from the matrix, 1 turns blocking off, P > 1 asks for P blocks.  It never changes a result bit."""
        if num_col_partitions is not None:
            assert num_col_partitions >= 1, "num_col_partitions should be larger than or equal to 1"
        indptr, indices, data, (self._num_rows, self._num_cols) = normalize_csr(adj_scipy)
        self._num_col_partitions = num_col_partitions
        self._nnz = int(indices.shape[0])
        self._target = None
        self._ctx = None
        self._register()
        C.require_device()
        # one upload per module; every run reuses the device copies (module/spmm.py:67-69)
        self._adj_indptr_dev = torch.from_numpy(indptr).to(self._ctx)
        self._adj_indices_dev = torch.from_numpy(indices).to(self._ctx)
        self._adj_vals_dev = torch.from_numpy(data).to(self._ctx)
        self._plan = ctypes.c_void_p()
        with torch.cuda.device(self._ctx):
            _lib.check(_lib.lib().fg_spmm_plan_create_partitioned(
                self._num_rows, self._num_cols, self._nnz, self._adj_indptr_dev.data_ptr(),
                self._adj_indices_dev.data_ptr(), int(num_col_partitions or 0), ctypes.byref(self._plan)))
        self._feat_shape = None
        self._feat_tiles = 0
        self._built = False
        self.out_tvm = None

    def __del__(self):
        plan = getattr(self, "_plan", None)
        if plan:
            try:
                _lib.lib().fg_spmm_plan_destroy(plan)
            except Exception:
                pass
            self._plan = None

    def _register(self):
        raise NotImplementedError("Please register target and ctx.")

    # -- shapes -----------------------------------------------------------
    def _heads_and_len(self, feat_shape):
        """(H, D) of a feature placeholder shape; vanilla modules have H = 1."""
        if len(feat_shape) != 2:
            raise ValueError("SrcFeat must be 2-D [num_src_vertices, feat_len], got %s" % (feat_shape,))
        return 1, int(feat_shape[1])

    def _parse_build(self, input_placeholders, compute_args, schedule_args):
        compute_args = C.check_known_keys(compute_args, ("num_feat_partitions",), "compute_args")
        C.check_known_keys(schedule_args, ("num_cuda_blocks", "num_threads_per_cuda_block", "num_feat_partitions"),
                           "schedule_args")
        if len(input_placeholders) != len(self._input_names):
            raise ValueError("expected placeholders for %s" % (self._input_names,))
        shapes = [tuple(int(s) for s in p.shape) for p in input_placeholders]
        for p in input_placeholders:
            if str(p.dtype) != "float32":
                raise TypeError("operands must be float32, got %s" % p.dtype)
        feat_shape = shapes[0]
        if feat_shape[0] != self._num_cols:
            raise ValueError("SrcFeat has %d rows, the adjacency matrix %d columns" % (feat_shape[0], self._num_cols))
        H, D = self._heads_and_len(feat_shape)
        if H * D < 1:
            raise ValueError("feature length must be positive")
        tiles = int(compute_args.get("num_feat_partitions", 0) or 0)
        if tiles < 0:
            raise ValueError("num_feat_partitions must be positive")
        if tiles > 1 and (H * D) % tiles != 0:
            # the reference assumes this silently (op/vanilla_spmm.py:41)
            raise ValueError("feat_len %d is not a multiple of num_feat_partitions %d" % (H * D, tiles))
        return shapes, H, D, tiles

    # -- reference call surface ------------------------------------------
    def build(self, input_placeholders, compute_args, schedule_args):
        """Fix operand shapes and allocate the (zero-filled, reused) output: module/spmm.py:81-111.

        compute_args : {'num_feat_partitions': P} asks for feature tiles of F/P floats
            (op/vanilla_spmm.py:41); absent or 0 lets the library choose.
        schedule_args : the reference's CUDA launch keys ('num_cuda_blocks',
            'num_threads_per_cuda_block') are accepted and ignored: the launch
            shape follows the row plan.
        """
        shapes, H, D, tiles = self._parse_build(input_placeholders, compute_args, schedule_args)
        self._input_shapes = shapes
        self._H, self._D, self._feat_tiles = H, D, tiles
        out_shape = (self._num_rows,) + tuple(shapes[0][1:])
        self.out_tvm = NDArray(torch.zeros(out_shape, dtype=torch.float32, device=self._ctx))
        self._padded = None
        pitch = self._row_pitch(H, D, tiles)
        if pitch:
            self._padded = torch.zeros((self._num_cols, pitch), dtype=torch.float32, device=self._ctx)
        self._built = True

    _pads_rows = False

    def _describe(self, H, D, tiles):
        buf = ctypes.create_string_buffer(1024)
        _lib.check(_lib.lib().fg_spmm_describe(self._plan, H, D, tiles, buf, len(buf)))
        return buf.value.decode()

    def _row_pitch(self, H, D, tiles):
        """Floats per row of the padded copy of the features that a run gathers from, or 0 for none.  A feature row
        whose byte length is not a multiple of the 128-byte cache line makes every 256-byte piece that is gathered
        lie across three lines instead of two; for rows beyond 64 floats a copy with rows padded to a multiple of 32
        floats, made at every run, costs far less than that (232,965 x 100 / 250 floats: 3.6 against 4.7 ms / 7.4
        against 12.3; up to 64 floats the copy costs what it saves).  Only the
        several-rows-per-wave kernel reads rows at a pitch."""
        if not self._pads_rows or H != 1 or tiles or D <= 64 or D % 32 == 0 or _lib.config_get("spmm.pad_rows") == 0:
            return 0
        if D < 128 and D % 32 < 4:
            # the row's last four floats, which the lane that the row's end cuts reads, would lie across a line in
            # every padded row; with a single whole tile before them that costs more than the copy saves (65 floats:
            # 4.4 against 3.9 ms on the 114.6M-nonzero graph; 130 floats: 6.3 against 7.5)
            return 0
        return (D + 31) // 32 * 32 if "rows-per-wave" in self._describe(H, D, tiles) else 0

    def lower_to_ir(self, input_placeholders, compute_args, schedule_args):
        """Description of the launch that `build` with these arguments would use (module/spmm.py:113-140
        returns TVM IR; the kernels here are prebuilt, so the plan is what there is to inspect)."""
        _, H, D, tiles = self._parse_build(input_placeholders, compute_args, schedule_args)
        text = self._describe(H, D, tiles)
        pitch = self._row_pitch(H, D, tiles)
        return text + (" | feature rows copied to a pitch of %d floats at every run" % pitch if pitch else "")

    def _launch(self, tensors):
        feat = tensors[0]
        stream = C.current_stream_handle(self._ctx)
        if self._padded is not None:
            pitch = self._padded.shape[1]
            _lib.check(_lib.lib().fg_pad_rows_f32(self._num_cols, self._D, pitch, feat.data_ptr(),
                                                  self._padded.data_ptr(), stream))
            status = _lib.lib().fg_spmm_csr_pitched_f32(
                self._plan, self._padded.data_ptr(), pitch, self._adj_vals_dev.data_ptr(),
                self.out_tvm.tensor.data_ptr(), self._D, stream)
            if status != _lib.FG_EUNSUPPORTED:        # a tuning key switched the kernel off after build: the plain call
                _lib.check(status)
                return
        _lib.check(_lib.lib().fg_spmm_csr_f32(
            self._plan, feat.data_ptr(), self._adj_vals_dev.data_ptr(), self.out_tvm.tensor.data_ptr(),
            self._D, self._feat_tiles, stream))

    def _checked_inputs(self, input_ndarrays):
        if not self._built:
            raise RuntimeError("call build() before run()")
        if len(input_ndarrays) != len(self._input_shapes):
            raise ValueError("expected %d input arrays" % len(self._input_shapes))
        return [C.check_operand(x, s, self._ctx, n)
                for x, s, n in zip(input_ndarrays, self._input_shapes, self._input_names)]

    def run(self, input_tvm_ndarrays):
        """Enqueue the kernel on torch's current stream and return the module-owned
        output array, which the next run overwrites (module/spmm.py:142-161)."""
        tensors = self._checked_inputs(input_tvm_ndarrays)
        with torch.cuda.device(self._ctx):
            self._launch(tensors)
        return self.out_tvm

    def measure_average_time(self, input_tvm_ndarrays, num_runs):
        """Average seconds per run over num_runs runs after one warm-up (module/spmm.py:163-186)."""
        tensors = self._checked_inputs(input_tvm_ndarrays)
        with torch.cuda.device(self._ctx):
            return C.time_calls(lambda: self._launch(tensors), self._ctx, num_runs)

    def row_order(self):
        """The plan's row visiting order (int32 host array) and the largest row degree."""
        order = np.empty(self._num_rows, dtype=np.int32)
        max_deg = ctypes.c_int32(0)
        _lib.check(_lib.lib().fg_spmm_plan_row_order(self._plan, order.ctypes.data, ctypes.byref(max_deg)))
        return order, max_deg.value

    @property
    def ctx(self):
        return self._ctx

    @property
    def target(self):
        return self._target


class VanillaSpMMhip(SpMMbase):
    """CSR SpMM on the GPU.  VanillaSpMMhip(adj) is the call of VanillaSpMMcuda (module/spmm.py:212-214);
    the optional num_col_partitions is the argument of VanillaSpMMx86 (:198)."""

    _pads_rows = True

    def __init__(self, adj_scipy, num_col_partitions=None):
        super().__init__(adj_scipy, num_col_partitions)

    def _register(self):
        self._target = "hip"
        self._ctx = hip(0)


class MultiHeadSpMMhip(SpMMbase):
    """Generalised SpMM with per-edge per-head weights (GAT aggregation):
    Out[r,h,:] = sum_e W[e,h] * SrcFeat[indices[e],h,:].

    Not in the reference; same surface as VanillaSpMMhip with two operands:
    build([SrcFeat (num_cols,H,D), EdgeWeight (nnz,H)], ...), run([feat, weight]).
    The CSR values of the adjacency matrix are not used.
    """

    _input_names = ("SrcFeat", "EdgeWeight")

    def __init__(self, adj_scipy, num_col_partitions=None):
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

    def _launch(self, tensors):
        feat, weight = tensors
        _lib.check(_lib.lib().fg_spmm_csr_mh_f32(
            self._plan, feat.data_ptr(), weight.data_ptr(), self.out_tvm.tensor.data_ptr(),
            self._H, self._D, self._feat_tiles, C.current_stream_handle(self._ctx)))
