"""Module classes under the reference's import path (python/featgraph/module/__init__.py:1-2).

The reference exports Vanilla{SpMM,SDDMM}{x86,cuda}.  Here the GPU classes are the HIP ones;
`VanillaSpMMcuda` / `VanillaSDDMMcuda` are bound to them so that a caller of the reference's
GPU target (tests/test_module_spmm.py:37-59, tests/test_module_sddmm.py:44-70) runs unchanged.
The x86 classes are a CPU target and are not provided; their partition arguments are accepted
by the HIP classes.
"""
from featgraph_amd.module import (MultiHeadSDDMMhip, MultiHeadSpMMhip, VanillaSDDMMhip,  # noqa: F401
                                  VanillaSpMMhip)

VanillaSpMMcuda = VanillaSpMMhip
VanillaSDDMMcuda = VanillaSDDMMhip

__all__ = ["VanillaSpMMhip", "VanillaSDDMMhip", "VanillaSpMMcuda", "VanillaSDDMMcuda", "MultiHeadSpMMhip",
           "MultiHeadSDDMMhip"]
