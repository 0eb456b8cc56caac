"""Writes the numeric fixtures under tests/golden/ for the C1 configuration.

The reference holds no stored numeric vectors for the kernels (its tests draw
unseeded inputs and compare with scipy / numpy formulas), and it cannot run
here (it needs TVM).  These fixtures are therefore produced by the CPU
restatement in oracle/, after tests/test_oracle.py has pinned it; they freeze
its answers so that later changes to the oracle or the generators show up.
Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from featgraph_amd import datasets  # noqa: E402
from oracle import ref  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    adj = datasets.config_graph("c1")
    feat = datasets.spmm_operands(adj, 64)
    out = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat)
    rows = np.arange(0, 4096, 64, dtype=np.int64)
    np.savez(os.path.join(HERE, "c1_spmm.npz"), sha256=hashlib.sha256(out.tobytes()).hexdigest(), rows=rows,
             out_rows=out[rows], graph=datasets.structure_checksum(adj))
    coo = adj.tocoo()
    src, dst = datasets.sddmm_operands(coo, 64)
    edges = np.arange(0, coo.nnz, 97, dtype=np.int64)
    sd = ref.sddmm_f64(coo.row, coo.col, src, dst)
    np.savez(os.path.join(HERE, "c1_sddmm_f64.npz"), edges=edges, out_edges=sd[edges],
             graph=datasets.structure_checksum(adj))
    print("wrote fixtures for graph", datasets.structure_checksum(adj))


if __name__ == "__main__":
    main()
