"""Host-side checks and helpers shared by the SpMM and SDDMM module classes."""
import numpy as np
import torch

from .. import _lib
from ..runtime import as_tensor

INT32_MAX = 2 ** 31 - 1


def to_int32_index(a, what):
    """Index array as contiguous int32.  scipy hands out int32 whenever the
    values fit (the reference keeps that dtype, module/spmm.py:61-64); int64
    input is narrowed when it fits and rejected otherwise."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.int32:
        return a
    if not np.issubdtype(a.dtype, np.integer):
        raise TypeError("%s must be an integer array, got %s" % (what, a.dtype))
    if a.size and (a.max() > INT32_MAX or a.min() < -INT32_MAX - 1):
        raise ValueError("%s holds values beyond int32, which the kernels index with" % what)
    return a.astype(np.int32)


def check_index_range(a, bound, what):
    """Ids must lie in [0, bound): the kernels gather through them unchecked."""
    if a.size and (int(a.min()) < 0 or int(a.max()) >= bound):
        raise ValueError("%s holds ids outside [0, %d)" % (what, bound))


def require_device():
    """The HIP library and a GPU, or an exception: there is no other code path."""
    _lib.lib()
    if not torch.cuda.is_available():
        raise RuntimeError("featgraph_amd needs a ROCm GPU (torch.cuda.is_available() is False); "
                           "there is no CPU fallback")


def check_known_keys(args, allowed, what):
    """The reference unpacks these dicts into keyword arguments, so a misspelt key raises TypeError there too."""
    if args is None:
        return {}
    unknown = sorted(set(args) - set(allowed))
    if unknown:
        raise TypeError("%s got unexpected keys %s (accepted: %s)" % (what, unknown, sorted(allowed)))
    return dict(args)


def check_operand(x, shape, device, what):
    """Device tensor of the built shape, float32, dense row-major."""
    t = as_tensor(x)
    if t.device != device:
        raise ValueError("%s lives on %s, the module on %s" % (what, t.device, device))
    if t.dtype != torch.float32:
        raise TypeError("%s must be float32, got %s" % (what, t.dtype))
    if tuple(t.shape) != tuple(shape):
        raise ValueError("%s has shape %s, the module was built for %s" % (what, tuple(t.shape), tuple(shape)))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous (row-major)" % what)
    return t


def current_stream_handle(device):
    """hipStream_t of torch's current stream on `device`, as an integer."""
    return torch.cuda.current_stream(device).cuda_stream


def time_calls(fn, device, num_runs):
    """Mean seconds per call: one untimed warm-up, then num_runs back-to-back
    calls between two events on the launch stream (the protocol of TVM's
    time_evaluator as the reference uses it, module/spmm.py:179-186)."""
    if num_runs < 1:
        raise ValueError("num_runs must be at least 1")
    fn()
    torch.cuda.synchronize(device)
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record(torch.cuda.current_stream(device))
    for _ in range(num_runs):
        fn()
    stop.record(torch.cuda.current_stream(device))
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / num_runs
