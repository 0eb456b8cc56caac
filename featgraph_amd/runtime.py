"""Light stand-ins for the few TVM objects that the reference's call surface uses.

The reference describes operands with te.placeholder and carries data in
tvm.nd.array objects (tests/test_module_spmm.py:18, :25).  With TVM gone a
placeholder is a (shape, dtype) record and an array is a torch tensor on the
ROCm device behind the two methods callers use (`asnumpy`, `shape`).
"""
import numpy as np
import torch

__all__ = ["Placeholder", "placeholder", "NDArray", "array", "hip", "device_available"]


class Placeholder:
    """Shape and dtype of an operand, as te.placeholder((rows, feat_len)) gives."""

    def __init__(self, shape, dtype="float32", name="placeholder"):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = str(dtype)
        self.name = name

    def __repr__(self):
        return "Placeholder(%s, shape=%s, dtype=%s)" % (self.name, self.shape, self.dtype)


def placeholder(shape, dtype="float32", name="placeholder"):
    return Placeholder(shape, dtype, name)


def hip(dev_id=0):
    """The context object of the HIP target: a torch device (ROCm devices are named 'cuda' in torch)."""
    return torch.device("cuda", dev_id)


def device_available():
    return torch.cuda.is_available()


class NDArray:
    """A device-resident array: a torch tensor with the accessors of tvm.nd.NDArray that callers use."""

    __slots__ = ("tensor",)

    def __init__(self, tensor):
        self.tensor = tensor

    @property
    def shape(self):
        return tuple(self.tensor.shape)

    @property
    def dtype(self):
        return str(self.tensor.dtype).replace("torch.", "")

    @property
    def ctx(self):
        return self.tensor.device

    def asnumpy(self):
        """Copy to the host (synchronises with the device)."""
        return self.tensor.detach().cpu().numpy()

    def __repr__(self):
        return "NDArray(shape=%s, dtype=%s, ctx=%s)" % (self.shape, self.dtype, self.ctx)


def array(data, ctx=None):
    """Upload a numpy array (or adopt a torch tensor) to the device `ctx`; counterpart of tvm.nd.array."""
    if isinstance(data, NDArray):
        data = data.tensor
    if isinstance(data, torch.Tensor):
        t = data if ctx is None else data.to(ctx)
    else:
        t = torch.from_numpy(np.ascontiguousarray(data))
        t = t.to(hip(0) if ctx is None else ctx)
    return NDArray(t.contiguous())


def as_tensor(x):
    """torch tensor behind an NDArray or tensor argument."""
    if isinstance(x, NDArray):
        return x.tensor
    if isinstance(x, torch.Tensor):
        return x
    raise TypeError("expected a featgraph_amd NDArray or a torch.Tensor on the device, got %s" % type(x).__name__)
