"""`featgraph`: the reference's package name, bound to the MI355X implementation in `featgraph_amd`.

Callers written against the reference import `featgraph.module` and `featgraph.util`
(python/featgraph/module/__init__.py:1-2, python/featgraph/util/__init__.py:1,
tests/test_module_spmm.py:9, tests/test_util.py:5); those imports work here unchanged.
`placeholder` and `nd` stand in for `tvm.te.placeholder` and `tvm.nd`, which the same
callers take from TVM.  The reference's `featgraph.op` holds TVM tensor expressions and
has no counterpart: the kernels are prebuilt.
"""
from featgraph_amd import nd, placeholder, hip, datasets  # noqa: F401
from . import module, util  # noqa: F401

__all__ = ["module", "util", "nd", "placeholder", "hip", "datasets"]
