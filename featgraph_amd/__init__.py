"""FeatGraph's sparse kernels (CSR SpMM, COO SDDMM) as hand-written HIP kernels for MI355X (gfx950).

    from featgraph_amd import placeholder, nd
    from featgraph_amd.module import VanillaSpMMhip, VanillaSDDMMhip

The operators run only through libfeatgraph_hip.so on a ROCm GPU; importing the
package needs neither, using an operator needs both.
"""
from . import runtime as nd
from .runtime import placeholder, hip
from . import util

__version__ = "0.1.0"
__all__ = ["nd", "placeholder", "hip", "util", "module", "datasets"]
