"""Times vanilla CSR SpMM on the GPU:  python -m featgraph_amd.benchmark.bench_vanilla_spmm --dataset reddit_csr.npz --feat-len 64

Same flags and timing protocol as the reference's benchmark/bench_vanilla_spmm.py:71-84 (--dataset, --feat-len,
--target; mean of 5 runs after one warm-up, :32-33).  Where the reference sweeps CUDA launch shapes
(:63-68), which this target derives from its row plan, the sweep here is over what is tunable: the number
of column partitions (the x86 sweep's first axis, :36) and of feature partitions (its second, :37).
"""
from .. import placeholder
from ..module import VanillaSpMMhip
from . import _common as C


def bench_vanilla_spmm_hip(adj_scipy_csr, feat_len, num_runs=5):
    num_rows, num_cols = adj_scipy_csr.shape
    nnz = adj_scipy_csr.nnz
    flops = 2.0 * nnz * feat_len
    alg_bytes = nnz * (8 + 4 * feat_len) + num_rows * (4 + 4 * feat_len)
    results = []
    for num_col_partitions in [None] + C.exp_range(1, 32, 2):
        module = VanillaSpMMhip(adj_scipy_csr, num_col_partitions)
        src_feat = C.random_features((num_cols, feat_len), module.ctx)
        for num_feat_partitions in [0] + C.exp_range(1, max(1, feat_len // 16), 2):
            module.build([placeholder((num_cols, feat_len))], {"num_feat_partitions": num_feat_partitions}, {})
            tcost = module.measure_average_time([src_feat], num_runs)
            label = "num_col_partitions=%s num_feat_partitions=%s" % (
                "auto" if num_col_partitions is None else num_col_partitions, num_feat_partitions or "auto")
            C.report(label, tcost, flops, alg_bytes)
            results.append((tcost, label))
    print("best:", min(results)[1])
    return results


if __name__ == "__main__":
    args = C.parser("Vanilla CSR SpMM timing", "csr").parse_args()
    bench_vanilla_spmm_hip(C.load_adjacency(args, "csr"), args.feat_len, args.num_runs)
