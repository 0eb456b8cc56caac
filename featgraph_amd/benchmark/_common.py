"""Shared pieces of the two benchmark commands."""
import argparse

import numpy as np
import scipy.sparse


def parser(description, matrix_format):
    ap = argparse.ArgumentParser(description=description)
    src = ap.add_mutually_exclusive_group(required=True)
    src.add_argument("--dataset", type=str,
                     help="adjacency matrix in %s format stored as a scipy .npz file" % matrix_format)
    src.add_argument("--synthetic", type=str, help="name of a seeded synthetic graph (c1, c2, c4, c2-mini, c4-mini)")
    ap.add_argument("--feat-len", type=int, default=128, help="the feature length")
    ap.add_argument("--target", type=str, default="hip", choices=["hip", "cuda", "x86"],
                    help="hip, or cuda (the reference's spelling of the GPU target, benchmark/bench_vanilla_spmm.py:"
                         "72-75; same as hip here, as featgraph.module.VanillaSpMMcuda is VanillaSpMMhip); x86 is "
                         "refused: this package has no CPU path")
    ap.add_argument("--num-runs", type=int, default=5, help="timed runs after one warm-up")
    return ap


def check_target(args):
    """The reference's --target spellings: cuda runs the HIP target; x86 has no counterpart and says so."""
    if args.target == "x86":
        raise SystemExit("--target x86: this package has only the GPU path (use --target hip or cuda)")
    return "hip"


def load_adjacency(args, matrix_format):
    check_target(args)
    if args.dataset:
        adj = scipy.sparse.load_npz(args.dataset)
        assert adj.format == matrix_format, "expected a %s matrix, got %s" % (matrix_format, adj.format)
        return adj
    from .. import datasets
    adj = datasets.config_graph(args.synthetic)
    return adj if matrix_format == "csr" else adj.tocoo()


def exp_range(start, end, mul):
    """start, start*mul, ... up to end (the grids of the reference's sweeps)."""
    out = []
    while start <= end:
        out.append(start)
        start *= mul
    return out


def report(label, seconds, flops, alg_bytes):
    print("%-44s average time of runs: %9.3f ms   %8.1f GFLOP/s   %8.1f GB/s (gather model)" % (
        label, seconds * 1e3, flops / seconds / 1e9, alg_bytes / seconds / 1e9))


def random_features(shape, ctx):
    from .. import nd
    return nd.array(np.random.random(shape).astype("float32"), ctx)
