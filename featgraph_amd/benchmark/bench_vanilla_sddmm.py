"""Times vanilla COO SDDMM on the GPU:  python -m featgraph_amd.benchmark.bench_vanilla_sddmm --dataset reddit_coo.npz --feat-len 64

Same flags and timing protocol as the reference's benchmark/bench_vanilla_sddmm.py:77-90 (mean of 5 runs after
one warm-up, :35-36).  The sweep is over the number of column partitions (the x86 sweep's axis, :39-40); the
reference's CUDA sweep over block counts (:71) has no counterpart because the launch shape follows the edge list.
"""
from .. import placeholder
from ..module import VanillaSDDMMhip
from . import _common as C


def bench_vanilla_sddmm_hip(adj_scipy_coo, feat_len, num_runs=5):
    num_rows, num_cols = adj_scipy_coo.shape
    nnz = adj_scipy_coo.nnz
    flops = 2.0 * nnz * feat_len
    alg_bytes = nnz * (12 + 8 * feat_len)
    results = []
    for num_col_partitions in [None] + C.exp_range(1, 32, 2):
        module = VanillaSDDMMhip(adj_scipy_coo, None, num_col_partitions)
        module.build([placeholder((num_cols, feat_len)), placeholder((num_rows, feat_len))], {}, {})
        src_feat = C.random_features((num_cols, feat_len), module.ctx)
        dst_feat = C.random_features((num_rows, feat_len), module.ctx)
        tcost = module.measure_average_time([src_feat, dst_feat], num_runs)
        label = "num_col_partitions=%s" % ("auto" if num_col_partitions is None else num_col_partitions)
        C.report(label, tcost, flops, alg_bytes)
        results.append((tcost, label))
    print("best:", min(results)[1])
    return results


if __name__ == "__main__":
    args = C.parser("Vanilla COO SDDMM timing", "coo").parse_args()
    bench_vanilla_sddmm_hip(C.load_adjacency(args, "coo"), args.feat_len, args.num_runs)
