#!/usr/bin/env python3
"""Benchmark of the SpMM / SDDMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: the 232,965-vertex / ~114.6M-nonzero power-law graph ("c2", the shape
of the Reddit graph that the reference's benchmark scripts load,
benchmark/bench_vanilla_spmm.py:77-79), float32, synthetic and seeded.  One
"step" is one vanilla CSR SpMM at feature length 64 with every operand already
resident in device memory.  W warm-up steps, then exactly K steps are timed
between two events on the launch stream; the printed JSON line carries

  value        SpMM GFLOP/s (2*nnz*F flops per step)
  roofline     algorithmic gather-model bytes / measured launch time against the
               8 TB/s HBM peak (bytes = nnz*(8+4F) + rows*(4+4F)); `traffic` is
               the measured L2<->memory byte count per launch, read from the
               committed counter summary under profiles/ when there is one
  cpu_baseline the CPU restatement of the reference's x86 loop nest on the host
               cores of this machine (same graph, same operands)
  sweep        both operators at feature lengths 32..512, timed with the
               reference's protocol (one warm-up, mean of five runs)

Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
FEAT_LENS = (32, 64, 128, 256, 512)


def spmm_alg_bytes(nnz, n_rows, F):
    """Gather model: per nonzero a column id, a value and one gathered row; per row a pointer and the output row."""
    return nnz * (8 + 4 * F) + n_rows * (4 + 4 * F)


def sddmm_alg_bytes(nnz, F):
    """Gather model: per edge two ids, two gathered rows and one output float."""
    return nnz * (12 + 8 * F)


def committed_traffic(op, F):
    """Bytes per launch between L2 and memory from the counter summary in profiles/, or None."""
    path = os.path.join(ROOT, "profiles", "%s_c2_counters.txt" % op)
    if not os.path.exists(path):
        return None
    m = re.search(r"^traffic_bytes_per_launch F=%d:\s*([0-9.eE+]+)" % F, open(path).read(), flags=re.M)
    return float(m.group(1)) if m else None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--feat-len", type=int, default=64, help="feature length of the timed step")
    ap.add_argument("--graph", default="c2", help="named synthetic configuration (featgraph_amd.datasets.CONFIGS)")
    ap.add_argument("--only", choices=["all", "spmm", "sddmm", "copy", "mh_sddmm", "mh_spmm"], default="all",
                    help="spmm / sddmm / copy: run just that kernel (for profiler runs), no sweep, no CPU leg; "
                         "mh_sddmm / mh_spmm: the multi-head operators (8 heads of --feat-len floats, use --graph c4)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the feature-length sweep")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py drives one GPU: both kernels are single-device and nothing here uses a second one "
                 "(got --gpus %d)" % args.gpus)

    import numpy as np
    import torch
    from featgraph_amd import _lib, datasets, nd, placeholder
    from featgraph_amd.module import MultiHeadSDDMMhip, MultiHeadSpMMhip, VanillaSDDMMhip, VanillaSpMMhip

    _lib.lib()  # fail now if the HIP library is missing
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a ROCm GPU")
    dev = torch.device("cuda", 0)
    stream = torch.cuda.current_stream(dev)

    def timed(fn, steps, warmup):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize(dev)
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record(stream)
        for _ in range(steps):
            fn()
        t1.record(stream)
        torch.cuda.synchronize(dev)
        return t0.elapsed_time(t1) / steps  # ms per launch

    if args.only == "copy":
        # plain device copy of known size: the yardstick the byte counters are scaled with
        n = 1 << 28
        a = torch.empty(n, dtype=torch.float32, device=dev).normal_()
        b = torch.empty_like(a)
        ms = timed(lambda: b.copy_(a), args.steps, args.warmup)
        print(json.dumps({"kernel": "copy", "bytes_read": 4 * n, "bytes_written": 4 * n, "ms": ms,
                          "GBps": 8 * n / ms / 1e6}))
        return

    t = time.time()
    adj = datasets.config_graph(args.graph)
    n_rows, n_cols, nnz = adj.shape[0], adj.shape[1], adj.nnz
    log("graph %s: %d x %d, nnz %d, max degree %d, checksum %s (%.1f s)" % (
        args.graph, n_rows, n_cols, nnz, int(np.diff(adj.indptr).max()), datasets.structure_checksum(adj),
        time.time() - t))
    F = args.feat_len
    out = {}

    if args.only in ("mh_sddmm", "mh_spmm"):
        # per-head forms of the two operators: [N, H, D] features, [nnz, H] edge weights / results
        H, D = 8, F
        if args.only == "mh_sddmm":
            op = MultiHeadSDDMMhip(adj.tocoo())
            ins = [nd.array(torch.randn((n_cols, H, D), dtype=torch.float32, device=dev)),
                   nd.array(torch.randn((n_rows, H, D), dtype=torch.float32, device=dev))]
            op.build([placeholder((n_cols, H, D)), placeholder((n_rows, H, D))], {}, {})
            b = nnz * (8 + 8 * H * D + 4 * H)
        else:
            op = MultiHeadSpMMhip(adj)
            ins = [nd.array(torch.randn((n_cols, H, D), dtype=torch.float32, device=dev)),
                   nd.array(torch.rand((nnz, H), dtype=torch.float32, device=dev))]
            op.build([placeholder((n_cols, H, D)), placeholder((nnz, H))], {}, {})
            b = nnz * (4 + 4 * H + 4 * H * D) + n_rows * (4 + 4 * H * D)
        ms = timed(lambda: op.run(ins), args.steps, args.warmup)
        print(json.dumps({"kernel": args.only, "graph": args.graph, "H": H, "D": D, "ms": ms,
                          "GFLOPs": 2.0 * nnz * H * D / ms / 1e6, "algorithmic_bytes": b, "alg_GBps": b / ms / 1e6,
                          "frac": b / ms / 1e6 / HBM_PEAK_GBPS}))
        return

    spmm = sddmm = None
    if args.only in ("all", "spmm"):
        spmm = VanillaSpMMhip(adj)
    if args.only in ("all", "sddmm"):
        sddmm = VanillaSDDMMhip(adj.tocoo())

    def spmm_case(F, feat_np=None):
        feat = nd.array(feat_np, dev) if feat_np is not None else nd.array(
            torch.randn((n_cols, F), dtype=torch.float32, device=dev))
        spmm.build([placeholder((n_cols, F))], {}, {})
        return feat

    def sddmm_case(F):
        src = nd.array(torch.randn((n_cols, F), dtype=torch.float32, device=dev))
        dst = nd.array(torch.randn((n_rows, F), dtype=torch.float32, device=dev))
        sddmm.build([placeholder((n_cols, F)), placeholder((n_rows, F))], {}, {})
        return [src, dst]

    if args.only == "sddmm":
        ins = sddmm_case(F)
        ms = timed(lambda: sddmm.run(ins), args.steps, args.warmup)
        b = sddmm_alg_bytes(nnz, F)
        print(json.dumps({"kernel": "sddmm", "F": F, "ms": ms, "alg_GBps": b / ms / 1e6,
                          "frac": b / ms / 1e6 / HBM_PEAK_GBPS}))
        return

    # ---- the timed step: CSR SpMM, feature length F --------------------------------
    feat_np = datasets.spmm_operands(adj, F)
    feat = spmm_case(F, feat_np)
    ms = timed(lambda: spmm.run([feat]), args.steps, args.warmup)
    flops = 2.0 * nnz * F
    alg = spmm_alg_bytes(nnz, n_rows, F)
    achieved = alg / ms / 1e6
    gpu_out = spmm.out_tvm.asnumpy() if args.only == "all" else None
    result = {
        "metric": "SpMM GFLOP/s (vanilla CSR, fp32, feat-len %d) with achieved algorithmic GB/s vs HBM roofline" % F,
        "value": flops / ms / 1e6, "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic (seeded power-law graph, N(0,1) features)",
        "config": {"workload": "%s: vanilla CSR SpMM, %d vertices, %d nonzeros, feat-len %d" % (
            args.graph, n_rows, nnz, F), "graph_checksum": datasets.structure_checksum(adj)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": committed_traffic("spmm", F),
                     "algorithmic_bytes": alg, "kernel": "spmm (CSR, feat-len %d)" % F, "launch_ms": ms,
                     "note": "one operator launch may be several dispatches of the same kernel (one per column "
                             "block and feature tile, see `launch`); bytes, time and traffic are per operator launch"},
        "launch": spmm.lower_to_ir([placeholder((n_cols, F))], {}, {}),
    }
    if args.only == "spmm":
        print(json.dumps(result))
        return

    # ---- the same step for a caller that starts from host memory (never `value`): pinned upload of the
    # features, the kernel, pinned download of the result
    host_in = torch.from_numpy(feat_np).pin_memory()
    host_out = torch.empty((n_rows, F), dtype=torch.float32).pin_memory()

    def from_host():
        feat.tensor.copy_(host_in, non_blocking=True)
        spmm.run([feat])
        host_out.copy_(spmm.out_tvm.tensor, non_blocking=True)

    ms_host = timed(from_host, max(3, args.steps // 4), 1)
    result["pcie_inclusive"] = {"ms_per_step": ms_host, "GFLOPs": flops / ms_host / 1e6,
                                "note": "features uploaded and result downloaded every step (pinned host memory)"}
    del host_in, host_out

    # ---- sweep, reference protocol: one warm-up, mean of five (bench_vanilla_spmm.py:32-33) ------
    if not args.no_sweep:
        sweep = []
        for f in FEAT_LENS:
            x = spmm_case(f)
            sec = spmm.measure_average_time([x], 5)
            b = spmm_alg_bytes(nnz, n_rows, f)
            sweep.append({"op": "spmm", "F": f, "ms": sec * 1e3, "GFLOPs": 2.0 * nnz * f / sec / 1e9,
                          "alg_GBps": b / sec / 1e9, "frac": b / sec / 1e9 / HBM_PEAK_GBPS,
                          "traffic": committed_traffic("spmm", f)})
            del x
            ins = sddmm_case(f)
            sec = sddmm.measure_average_time(ins, 5)
            b = sddmm_alg_bytes(nnz, f)
            sweep.append({"op": "sddmm", "F": f, "ms": sec * 1e3, "GFLOPs": 2.0 * nnz * f / sec / 1e9,
                          "alg_GBps": b / sec / 1e9, "frac": b / sec / 1e9 / HBM_PEAK_GBPS,
                          "traffic": committed_traffic("sddmm", f)})
            del ins
            torch.cuda.empty_cache()
            log("sweep F=%d: spmm %.3f ms (%.2f of roofline), sddmm %.3f ms (%.2f)" % (
                f, sweep[-2]["ms"], sweep[-2]["frac"], sweep[-1]["ms"], sweep[-1]["frac"]))
        result["sweep"] = sweep

    # ---- CPU baseline: the restated x86 nest on this machine's cores ----------------------------
    if not args.no_cpu:
        from oracle import ref
        cores = ref.num_threads()
        work = np.empty((n_cols + n_rows) * F, dtype=np.float32)
        t0 = time.time()
        cpu_out = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat_np, 1, work)   # warm-up, kept for parity
        first = time.time() - t0
        runs = int(max(1, min(20, 10.0 / max(first, 1e-3))))   # about ten seconds of CPU work
        if first > 10.0:
            runs, cpu_s = 1, first
        else:
            t0 = time.time()
            for _ in range(runs):
                ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat_np, 1, work)
            cpu_s = (time.time() - t0) / runs
        result["cpu_baseline"] = {
            "value": flops / cpu_s / 1e9, "unit": "GFLOP/s", "cores": cores, "kind": "port",
            "seconds": cpu_s,
            "sample": "the whole workload (%s, feat-len %d): restated TVM x86 nest with both layout transforms, "
                      "num_feat_partitions=1, OpenMP static rows, mean of %d run(s) after one warm-up" % (
                          args.graph, F, runs)}
        result["parity"] = {"spmm_bit_exact_vs_cpu_restatement": bool(np.array_equal(gpu_out, cpu_out)),
                            "spmm_max_abs_diff": float(np.max(np.abs(gpu_out - cpu_out)))}
        # SDDMM: the reference schedule is serial, so a bounded sample of the edge list on one core
        coo = adj.tocoo()
        m = min(nnz, 4_000_000)
        rng = np.random.default_rng(2)
        src = rng.standard_normal((n_cols, F), dtype=np.float32)
        dst = rng.standard_normal((n_rows, F), dtype=np.float32)
        buf = np.empty(m, dtype=np.float32)
        ref.sddmm_x86_fast(coo.row[:m], coo.col[:m], src, dst, False, buf)
        t0 = time.time()
        ref.sddmm_x86_fast(coo.row[:m], coo.col[:m], src, dst, False, buf)
        sd_s = time.time() - t0
        result["cpu_baseline_sddmm"] = {"value": 2.0 * m * F / sd_s / 1e9, "unit": "GFLOP/s", "cores": 1,
                                        "kind": "port",
                                        "sample": "first %d edges of the row-sorted COO list, feat-len %d, "
                                                  "serial edge loop (the reference schedule has no parallel axis)" % (m, F)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
