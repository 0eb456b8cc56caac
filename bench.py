#!/usr/bin/env python3
"""Benchmark of the SpMM / SDDMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: the 232,965-vertex / ~114.6M-nonzero power-law graph ("c2", the shape
of the Reddit graph that the reference's benchmark scripts load,
benchmark/bench_vanilla_spmm.py:77-79), float32, synthetic and seeded.  One
"step" is one vanilla CSR SpMM at feature length 64 with every operand already
resident in device memory.  W warm-up steps, then exactly K steps are timed
between two events on the launch stream.  The LAST line of stdout is one short
JSON object (under 1.5 KB: metric, value, roofline, cpu_baseline, parity); every
other row (feature-length sweep, multi-head operators, probes, per-setting CPU
timings) is printed earlier, one compact JSON object per line on stderr, and
the whole record is also written to bench_detail.json in the directory that FEATGRAPH_BENCH_OUT names
(default: bench_out/ beside this file).  The record carries

  value        SpMM GFLOP/s (2*nnz*F flops per step)
  roofline     `achieved` / `frac`: algorithmic gather-model bytes (nnz*(8+4F) + rows*(4+4F)) over the measured
               launch time against the 8 TB/s HBM peak.  The model credits no cache reuse, so on this graph
               (59.6 MB of features, 492 gathers per row) it exceeds what reaches HBM and `frac` can pass 1.
               Three fractions that cannot are reported beside it:
                 hbm_frac_compulsory     every array touched once (8*nnz + 4(N+1) + 8*N*F bytes) / time / peak
                 l2_fabric_frac          bytes that crossed the L2 boundary per launch (`traffic`, from the
                                         committed rocprofv3 counter summary named in `traffic_source`) / time / peak
                 frac_of_gather_ceiling  time of the bare gather probe (same rows-per-instruction, same band
                                         width, same number of gathers; nothing else) / time of the operator,
                                         measured in this run
  cpu_baseline the CPU restatement of the reference's x86 loop nest on the host cores of this machine
               (same graph, same operands), num_feat_partitions swept as the reference's script does
  sweep        both operators at feature lengths 32..512 (one warm-up, mean of five runs: the reference's
               protocol), each row with its parity check against the CPU checker, the shuffled edge list,
               and the multi-head operators on the 2.45M-vertex graph

Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import ctypes
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
MH_HEADS = 8
MH_HEAD_LENS = (16, 32, 64)
RTOL, ATOL = 1e-5, 1e-4


def spmm_alg_bytes(nnz, n_rows, F):
    """Gather model: per nonzero a column id, a value and one gathered row; per row a pointer and the output row."""
    return nnz * (8 + 4 * F) + n_rows * (4 + 4 * F)


def spmm_min_bytes(nnz, n_rows, n_cols, F):
    """Every array touched exactly once: ids + values, row pointer, features read, output written."""
    return 8 * nnz + 4 * (n_rows + 1) + 4 * F * (n_rows + n_cols)


def sddmm_alg_bytes(nnz, F):
    """Gather model: per edge two ids, two gathered rows and one output float."""
    return nnz * (12 + 8 * F)


def sddmm_min_bytes(nnz, n_rows, n_cols, F):
    return 12 * nnz + 4 * F * (n_rows + n_cols)


def mh_sddmm_alg_bytes(nnz, H, D):
    return nnz * (8 + 8 * H * D + 4 * H)


def mh_spmm_alg_bytes(nnz, n_rows, H, D):
    return nnz * (4 + 4 * H + 4 * H * D) + n_rows * (4 + 4 * H * D)


def mh_attention_alg_bytes(nnz, n_rows, H, D, shared):
    """Gather model of the fused attention operator: per nonzero the id and one (key = value) or two gathered rows,
    per destination row its bounds, the query and the result."""
    return nnz * (4 + (1 if shared else 2) * 4 * H * D) + n_rows * (8 + 8 * H * D)


def committed_traffic(op, graph, F):
    """(bytes per launch across the L2 boundary, source file) from the counter summary in profiles/, or (None, None)."""
    rel = os.path.join("profiles", "%s_%s_counters.txt" % (op, graph))
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return None, None
    m = re.search(r"^traffic_bytes_per_launch F=%d:\s*([0-9.eE+]+)" % F, open(path).read(), flags=re.M)
    return (float(m.group(1)), rel) if m else (None, None)


def committed_hit_rate(op, graph, F):
    """(L2 hit rate of the operator's kernels as a fraction, source file) from the same summary, or (None, None)."""
    rel = os.path.join("profiles", "%s_%s_counters.txt" % (op, graph))
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return None, None
    m = re.search(r"^feat-len %d .*?L2 hit rate ([0-9.]+) %%" % F, open(path).read(), flags=re.M | re.S)
    return (float(m.group(1)) / 100.0, rel) if m else (None, None)


def committed_traffic_mh(kind, D):
    """The same for a multi-head operator on the 2.45M-vertex graph."""
    rel = os.path.join("profiles", "multihead_c4_counters.txt")
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return None, None
    m = re.search(r"^traffic_bytes_per_launch %s D=%d:\s*([0-9.eE+]+)" % (kind, D), open(path).read(), flags=re.M)
    return (float(m.group(1)), rel) if m else (None, None)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def _sig(x, digits=5):
    """Floats shortened to `digits` significant digits (the short line only; the detail record keeps full precision)."""
    if isinstance(x, float):
        return float("%.*g" % (digits, x))
    if isinstance(x, dict):
        return {k: _sig(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_sig(v, digits) for v in x]
    return x


HEADLINE_LIMIT = 1500


def headline(result, detail_path=None):
    """The short record that ends stdout: what a harness reads, nothing else.  Built from the detail record."""
    r = result["roofline"]
    roof = {k: r.get(k) for k in ("bound", "achieved", "peak", "unit", "frac", "frac_bounded", "traffic",
                                  "traffic_source", "algorithmic_bytes", "kernel", "dispatches_per_launch",
                                  "hbm_frac_compulsory", "frac_of_gather_ceiling")}
    # the bare gather pattern at the operator's own L2 hit rate with an index-like stream beside it / operator time
    roof["frac_of_gather_and_stream_ceiling"] = r.get("frac_of_gather_and_stream_at_the_operators_l2_hit_rate")
    line = {k: result.get(k) for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                       "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config")}
    line["roofline"] = roof
    if result.get("roofline_hbm_bound_config"):
        line["roofline_hbm_bound_config"] = result["roofline_hbm_bound_config"]
    c = result.get("cpu_baseline")
    if c:
        line["cpu_baseline"] = {k: c.get(k) for k in ("value", "unit", "cores", "kind", "seconds", "cpu_model",
                                                      "best_num_feat_partitions", "sample")}
    p = result.get("parity")
    if p is not None:
        line["parity"] = all(v for v in p.values() if isinstance(v, bool))
    if detail_path:
        line["detail"] = detail_path
    return _sig(line)


def headline_line(result, detail_path=None):
    line = json.dumps(headline(result, detail_path), separators=(",", ":"))
    if len(line) >= HEADLINE_LIMIT:
        raise RuntimeError("the headline line grew to %d characters (limit %d)" % (len(line), HEADLINE_LIMIT))
    return line


def emit(result):
    """Detail rows to stderr (one compact JSON object per line), the whole record to a file, the headline last on stdout."""
    def row(tag, obj):
        print(json.dumps({"detail": tag, **_sig(obj, 6)}, separators=(",", ":")), file=sys.stderr)

    for r in result.get("sweep", []):
        row("sweep", r)
    for r in result.get("multi_head", {}).get("rows", []):
        row("multi_head", r)
    for key in ("pcie_inclusive", "small_graph", "cpu_baseline", "cpu_baseline_sddmm", "parity", "plan_seconds"):
        if key in result:
            row(key, result[key] if isinstance(result[key], dict) else {"value": result[key]})
    row("roofline", result["roofline"])
    row("launch", {"text": result.get("launch")})
    detail_path = None
    try:
        out_name = os.environ.get("FEATGRAPH_BENCH_OUT", "bench_out")
        out_dir = out_name if os.path.isabs(out_name) else os.path.join(ROOT, out_name)
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "bench_detail.json"), "w") as f:
            json.dump(result, f, indent=1)
        detail_path = os.path.join(out_name, "bench_detail.json")
    except OSError:
        pass
    sys.stderr.flush()
    print(headline_line(result, detail_path), flush=True)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--feat-len", type=int, default=64, help="feature length of the timed step")
    ap.add_argument("--graph", default="c2", help="named synthetic configuration (featgraph_amd.datasets.CONFIGS)")
    ap.add_argument("--only", choices=["all", "spmm", "sddmm", "sddmm_shuffled", "copy", "mh_sddmm", "mh_spmm", "mh_sddmm_softmax",
                                       "mh_attention", "mh_attention_kv", "mh_attention_grad", "gather_probe", "gather_store_probe", "gather_stream_probe"],
                    default="all",
                    help="spmm / sddmm / copy / gather_probe: run just that kernel (for profiler runs), no sweep, no "
                         "CPU leg; mh_sddmm / mh_spmm: the multi-head operators (8 heads of --feat-len floats, use "
                         "--graph c4)")
    ap.add_argument("--band-rows", type=int, default=0,
                    help="with --only gather_probe: rows per band (default 16384 rows of a 64-float tile)")
    ap.add_argument("--fold-cols", type=int, default=0,
                    help="with --only spmm / sddmm: column ids taken modulo this (the same rows and nonzeros over a "
                         "feature matrix of so many rows; 8192 rows of 64 floats fit one L2, so every gather hits)")
    ap.add_argument("--squeeze-cols", default="",
                    help="with --only spmm / sddmm: W:K maps the column ids of every band of W columns onto the band's "
                         "first K columns, ascending order kept (same passes, same runs, a smaller gather target per "
                         "pass: W = the pass width that lower_to_ir reports, K = 8192 rows of 64 floats fit one L2)")
    ap.add_argument("--degree-cap", type=int, default=0,
                    help="with --only spmm / sddmm: every row cut to at most so many nonzeros (takes the hub rows out)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg and the parity checks")
    ap.add_argument("--no-sweep", action="store_true", help="skip the feature-length sweep")
    ap.add_argument("--no-mh", action="store_true", help="skip the multi-head operators on the 2.45M-vertex graph")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py drives one GPU: both kernels are single-device and nothing here uses a second one "
                 "(got --gpus %d)" % args.gpus)

    import numpy as np
    import torch
    from featgraph_amd import _lib, datasets, nd, placeholder
    from featgraph_amd.module import (EdgeSoftmaxhip, GeneralizedSpMMhip, MultiHeadAttentionGradhip,
                                      MultiHeadAttentionhip, MultiHeadSDDMMhip, MultiHeadSDDMMSoftmaxhip,
                                      MultiHeadSpMMhip, VanillaSDDMMhip, VanillaSpMMhip)

    L = _lib.lib()  # fail now if the HIP library is missing
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

    def device_normal(shape, seed):
        g = torch.Generator(device=dev)
        g.manual_seed(seed)
        return torch.randn(shape, dtype=torch.float32, device=dev, generator=g)

    sink = torch.zeros(64, dtype=torch.float32, device=dev)

    def gather_probe(feat_t, n_gathers, steps=5, warmup=3, band=None):
        """Milliseconds that the bare gather pattern takes for n_gathers row gathers per tile, with the tile width of
        the operators and a band of `band` rows (default: a 4 MB band, 16384 rows of a 64-float tile, which an L2
        holds: nearly every gather hits)."""
        n, F = feat_t.shape
        tile = 64 if F >= 64 else (32 if F >= 32 else 16)
        if F % tile != 0 or n * F * 4 >= 2 ** 32:
            return None
        band = int(band) if band else 16384 * (64 // tile)
        issued = L.fg_probe_gather_count(n, tile, band, n_gathers)
        ms = timed(lambda: _lib.check(L.fg_probe_gather_f32(feat_t.data_ptr(), n, F, tile, band, n_gathers,
                                                            sink.data_ptr(), stream.cuda_stream)), steps, warmup)
        return {"ms": ms * n_gathers / issued, "tile": tile, "band_rows": band, "gathers_per_tile": n_gathers,
                "row_TBps": n_gathers * F * 4 / (ms * n_gathers / issued) / 1e9}

    def gather_probe_at_hit_rate(feat_t, n_gathers, op, F):
        """The same probe with its band widened until its own L2 hit rate is the operator's: gathers that fall
        uniformly on a band of b L2 sizes hit at 1 / b (measured: profiles/gather_probe_c2_f64_bands.txt), so the
        band is 16384 / hit_rate rows of a 64-float tile.  What the memory system does for this gather stream at
        the hit rate the operator reaches, with no ids, values, sums or results beside it."""
        hit, src_file = committed_hit_rate(op, args.graph, F)
        if not hit:
            return None
        tile = 64 if F >= 64 else (32 if F >= 32 else 16)
        p = gather_probe(feat_t, n_gathers, band=min(feat_t.shape[0], round(16384 * (64 // tile) / hit)))
        if p:
            p.update({"l2_hit_rate_of_the_operator": hit, "hit_rate_source": src_file})
        return p

    def gather_and_stream_probe_at_hit_rate(feat_t, n_gathers, op, F):
        """The 64-float gather pattern at the operator's own L2 hit rate (band widened as above) WITH an index-like
        stream of 8 bytes per gather read from HBM by the gathering waves beside it (fg_probe_gather_stream_f32): what
        the memory system does for the operator's mix of traffic and nothing else."""
        hit, src_file = committed_hit_rate(op, args.graph, F)
        if not hit or F != 64 or feat_t.shape[1] != 64:
            return None
        band = int(min(feat_t.shape[0], round(16384 / hit)))
        stream_dw = 1 << 28
        buf = torch.zeros(stream_dw, dtype=torch.int32, device=dev)

        def go():
            return L.fg_probe_gather_stream_f32(feat_t.data_ptr(), band, n_gathers, buf.data_ptr(), stream_dw, stream_dw, 1,
                                                sink.data_ptr(), stream.cuda_stream)
        issued = go()
        if issued <= 0:
            return None
        ms = timed(go, 5, 2) * n_gathers / issued
        del buf
        return {"ms": ms, "band_rows": band, "stream_bytes_per_gather": 8, "l2_hit_rate_of_the_operator": hit,
                "hit_rate_source": src_file}

    def rows_probe(feat_t, n_gathers, steps=3):
        """Milliseconds that n_gathers random whole-row gathers from feat_t take (rows of 128 .. 1024 floats)."""
        n, row_floats = feat_t.shape[0], int(feat_t[0].numel())
        issued = L.fg_probe_gather_rows_count(row_floats, n_gathers)
        if issued <= 0:
            return None
        ms = timed(lambda: _lib.check(L.fg_probe_gather_rows_f32(feat_t.data_ptr(), n, row_floats, n_gathers,
                                                                 sink.data_ptr(), stream.cuda_stream)), steps, 1)
        ms = ms * n_gathers / issued
        return {"ms": ms, "row_bytes": row_floats * 4, "gathers": n_gathers,
                "row_TBps": n_gathers * row_floats * 4 / ms / 1e9}

    def rows_write_probe(feat_t, out_t, n_gathers, n_writes, read_only_ms, steps=3):
        """Milliseconds for n_gathers random whole-row gathers from feat_t plus n_writes whole-row stores into out_t:
        the read-only probe's rate for the gathers and, for the stores, the extra time per stored row that the
        gather + store probe shows at (about) the same mix."""
        n, row_floats = feat_t.shape[0], int(feat_t[0].numel())
        g, w = ctypes.c_int64(0), ctypes.c_int64(0)
        per = max(1, int(round(n_gathers / max(n_writes, 1))))
        if L.fg_probe_gather_write_rows_count(row_floats, n_gathers, per, ctypes.byref(g), ctypes.byref(w)) != 0:
            return None
        ms = timed(lambda: _lib.check(L.fg_probe_gather_write_rows_f32(
            feat_t.data_ptr(), n, row_floats, n_gathers, per, out_t.data_ptr(), out_t.shape[0], sink.data_ptr(),
            stream.cuda_stream)), steps, 1)
        per_gather = read_only_ms / n_gathers
        per_write = max(0.0, (ms - g.value * per_gather) / max(w.value, 1))
        return {"ms": n_gathers * per_gather + n_writes * per_write, "probe_ms": ms, "probe_gathers": g.value,
                "probe_row_writes": w.value, "ms_per_million_row_writes": per_write * 1e6}

    if args.only == "copy":
        # plain device copy of known size: the yardstick the byte counters are scaled with
        n = 1 << 28
        a = torch.empty(n, dtype=torch.float32, device=dev).normal_()
        b = torch.empty_like(a)
        ms = timed(lambda: b.copy_(a), args.steps, args.warmup)
        fill_ms = timed(lambda: b.fill_(1.0), args.steps, args.warmup)  # stores alone
        print(json.dumps({"kernel": "copy", "bytes_read": 4 * n, "bytes_written": 4 * n, "ms": ms,
                          "GBps": 8 * n / ms / 1e6, "fill_ms": fill_ms, "fill_GBps": 4 * n / fill_ms / 1e6}))
        return

    t = time.time()
    adj = datasets.config_graph(args.graph)
    n_rows, n_cols, nnz = adj.shape[0], adj.shape[1], adj.nnz
    log("graph %s: %d x %d, nnz %d, max degree %d, checksum %s (%.1f s)" % (
        args.graph, n_rows, n_cols, nnz, int(np.diff(adj.indptr).max()), datasets.structure_checksum(adj),
        time.time() - t))
    F = args.feat_len
    if args.only in ("spmm", "sddmm") and (args.fold_cols or args.degree_cap or args.squeeze_cols):
        # diagnostic variants of the graph: what bounds the kernels when the cache misses or the hub rows are taken away
        import scipy.sparse
        if args.degree_cap:
            deg = np.diff(adj.indptr)
            keep_deg = np.minimum(deg, args.degree_cap)
            keep = (np.arange(nnz) - np.repeat(adj.indptr[:-1], deg)) < np.repeat(keep_deg, deg)
            indptr = np.zeros(n_rows + 1, np.int32)
            np.cumsum(keep_deg, out=indptr[1:])
            adj = scipy.sparse.csr_matrix((adj.data[keep], adj.indices[keep], indptr), shape=adj.shape)
        if args.fold_cols:
            adj = scipy.sparse.csr_matrix((adj.data, (adj.indices % args.fold_cols).astype(np.int32), adj.indptr),
                                          shape=(n_rows, args.fold_cols))
        if args.squeeze_cols:
            width, kept = (int(x) for x in args.squeeze_cols.split(":"))
            band, inside = np.divmod(adj.indices.astype(np.int64), width)
            adj = scipy.sparse.csr_matrix((adj.data, (band * width + inside * kept // width).astype(np.int32), adj.indptr),
                                          shape=adj.shape)
        n_rows, n_cols, nnz = adj.shape[0], adj.shape[1], adj.nnz
        log("variant: %d x %d, nnz %d, max degree %d" % (n_rows, n_cols, nnz, int(np.diff(adj.indptr).max())))

    if args.only == "gather_probe":
        feat_t = device_normal((n_cols, F), 1)
        p = gather_probe(feat_t, nnz, args.steps, band=args.band_rows or None)
        print(json.dumps({"kernel": "gather_probe", "F": F, **(p or {})}))
        return

    if args.only == "gather_stream_probe":
        # bare gathers of 64-float rows from a 4 MB band, with an index-like stream of 8 bytes per gather beside them
        band = 16384
        feat_t = device_normal((band, 64), 1)
        stream_dw = 1 << 28                                  # 1 GiB of zeros
        buf = torch.zeros(stream_dw, dtype=torch.int32, device=dev)
        rows = []
        for what, mode, window in (("gathers only", 0, 65536),
                                   ("stream from HBM, read by every wave", 1, stream_dw),
                                   ("stream from a 64 MB window, read by every wave", 1, 1 << 24),
                                   ("stream from a 256 KB window, read by every wave", 1, 1 << 16),
                                   ("stream from HBM, read by one wave of four", 2, stream_dw),
                                   ("stream from a 256 KB window, read by one wave of four", 2, 1 << 16),
                                   ("stream from HBM through the scalar cache", 3, stream_dw),
                                   ("stream from a 256 KB window through the scalar cache", 3, 1 << 16)):
            def go():
                return L.fg_probe_gather_stream_f32(feat_t.data_ptr(), band, nnz, buf.data_ptr(), stream_dw, window, mode,
                                                    sink.data_ptr(), stream.cuda_stream)
            issued = go()
            if issued <= 0:
                raise RuntimeError(L.fg_last_error().decode("utf-8", "replace"))
            ms = timed(go, args.steps, 2) * nnz / issued
            rows.append({"variant": what, "ms_per_%d_gathers" % nnz: round(ms, 4)})
            log("%-56s %.3f ms" % (what, ms))
        print(json.dumps({"kernel": "gather_stream_probe", "band_rows": band, "row_floats": 64, "rows": rows}))
        return

    if args.only == "gather_store_probe":
        # whole rows of 8 x F floats from anywhere in an [N, 8, F] matrix: nnz gathers alone, then with one
        # whole-row store per destination row beside them (the mix of multi-head SpMM and of the fused attention)
        feat_t = device_normal((n_cols, MH_HEADS, F), 1)
        out_t = torch.zeros((n_rows, MH_HEADS, F), dtype=torch.float32, device=dev)
        p = rows_probe(feat_t, nnz, args.steps)
        pw = rows_write_probe(feat_t, out_t, nnz, n_rows, p["ms"], args.steps) if p else None
        rf = MH_HEADS * F

        def stores_only():
            return L.fg_probe_store_rows_f32(out_t.data_ptr(), n_rows, rf, n_rows, stream.cuda_stream)

        def one_after_the_other():
            _lib.check(L.fg_probe_gather_rows_f32(feat_t.data_ptr(), n_cols, rf, nnz, sink.data_ptr(),
                                                  stream.cuda_stream))
            stores_only()

        stored = stores_only()
        alone = {"ms": timed(stores_only, args.steps, 1), "row_stores": stored} if stored > 0 else None
        after = {"ms": timed(one_after_the_other, args.steps, 1)} if stored > 0 and p else None
        print(json.dumps({"kernel": "gather_store_probe", "graph": args.graph, "row_floats": rf,
                          "gathers": nnz, "row_stores": n_rows, "read_only": p, "with_stores": pw,
                          "stores_only": alone, "gathers_then_stores": after}))
        return

    def mh_case(kind, graph_adj, D, steps, warmup, check):
        """One multi-head operator: [N, 8, D] features, [nnz, 8] edge weights / results."""
        H = MH_HEADS
        n_r, n_c, e = graph_adj.shape[0], graph_adj.shape[1], graph_adj.nnz
        row = {"op": kind, "H": H, "D": D}
        if kind in ("mh_sddmm", "mh_sddmm_softmax"):
            coo = graph_adj.tocoo()
            op = MultiHeadSDDMMhip(coo) if kind == "mh_sddmm" else MultiHeadSDDMMSoftmaxhip(coo)
            src, dst = device_normal((n_c, H, D), 11 + D), device_normal((n_r, H, D), 12 + D)
            if kind == "mh_sddmm_softmax":
                src *= 0.25                      # scores of magnitude ~ sqrt(D) / 4: weights that are not one-hot
            op.build([placeholder((n_c, H, D)), placeholder((n_r, H, D))], {}, {})
            ins = [src, dst]
            b, b_min = mh_sddmm_alg_bytes(e, H, D), 8 * e + 4 * H * e + 4 * H * D * (n_r + n_c)
        elif kind == "mh_attention_grad":
            # backward of the layer whose key is its value: scores + softmax recomputed, then the softmax gradient,
            # two multi-head SpMMs over the transposed matrix, one over the matrix and one multi-head SDDMM
            op = MultiHeadAttentionGradhip(graph_adj)
            src, dst = device_normal((n_c, H, D), 11 + D), device_normal((n_r, H, D), 12 + D)
            src *= 0.25
            ins = [src, dst, device_normal((n_r, H, D), 15 + D)]
            op.build([placeholder((n_c, H, D)), placeholder((n_r, H, D))], {}, {})
            b = (2 * mh_sddmm_alg_bytes(e, H, D) + 2 * mh_spmm_alg_bytes(e, n_c, H, D) + mh_spmm_alg_bytes(e, n_r, H, D)
                 + e * (3 * 4 * H) + 2 * e * (4 + 8 * H) + 3 * 4 * H * D * n_c)
            b_min = 8 * e + 4 * H * D * (3 * n_r + 3 * n_c)
        elif kind in ("mh_attention", "mh_attention_kv"):
            # scores, softmax and weighted sum in one kernel; "mh_attention": the vertex features are key and value
            shared = kind == "mh_attention"
            op = MultiHeadAttentionhip(graph_adj)
            src, dst = device_normal((n_c, H, D), 11 + D), device_normal((n_r, H, D), 12 + D)
            src *= 0.25
            ins = [src, dst] if shared else [src, dst, device_normal((n_c, H, D), 14 + D)]
            op.build([placeholder(tuple(x.shape)) for x in ins], {}, {})
            b = mh_attention_alg_bytes(e, n_r, H, D, shared)
            b_min = 4 * e + 8 * n_r + 4 * H * D * (2 * n_r + (1 if shared else 2) * n_c)
        else:
            op = MultiHeadSpMMhip(graph_adj)
            src = device_normal((n_c, H, D), 13 + D)
            # softmax of uniform logits over each destination row's edges, per head
            g = torch.Generator(device=dev)
            g.manual_seed(3)
            w = torch.rand((e, H), dtype=torch.float32, device=dev, generator=g).exp_()
            rows_of = torch.repeat_interleave(torch.arange(n_r, device=dev),
                                              torch.from_numpy(np.diff(graph_adj.indptr)).to(dev))
            sums = torch.zeros((n_r, H), dtype=torch.float32, device=dev).index_add_(0, rows_of, w)
            w /= sums[rows_of]
            del rows_of, sums
            op.build([placeholder((n_c, H, D)), placeholder((e, H))], {}, {})
            ins = [src, w]
            b, b_min = mh_spmm_alg_bytes(e, n_r, H, D), 4 * e + 4 * H * e + 4 * (n_r + 1) + 4 * H * D * (n_r + n_c)
        ms = timed(lambda: op.run(ins), steps, warmup)
        p = rows_probe(src, e)
        if p and kind == "mh_attention_kv":      # two gathered rows per edge
            p = dict(p, ms=2 * p["ms"], gathers=2 * e)
        if p and kind == "mh_attention_grad":    # five operators that each gather one row per edge
            p = dict(p, ms=5 * p["ms"], gathers=5 * e)
        if kind == "mh_attention_grad":
            row["flops_note"] = "10 * E * H * D: five gather-and-multiply operators"
        if p:
            row.update({"gather_ceiling_ms": p["ms"], "gather_ceiling_row_TBps": p["row_TBps"],
                        "frac_of_gather_ceiling": p["ms"] / ms})
        tr, tr_src = committed_traffic_mh(kind, D) if graph_adj.shape[0] == 2449029 else (None, None)
        if tr:
            row.update({"traffic": tr, "traffic_source": tr_src, "hbm_frac_traffic": tr / ms / 1e6 / HBM_PEAK_GBPS})
        row.update({"ms": ms, "GFLOPs": (10.0 if kind == "mh_attention_grad" else 2.0) * e * H * D / ms / 1e6,
                    "alg_GBps": b / ms / 1e6,
                    "frac": b / ms / 1e6 / HBM_PEAK_GBPS, "hbm_frac_compulsory": b_min / ms / 1e6 / HBM_PEAK_GBPS,
                    "algorithmic_bytes": b, "compulsory_bytes": b_min})
        if check and kind != "mh_attention_grad":   # (its parity runs at full size in tests/test_full_size.py)
            from oracle import ref
            out = op.out_tvm.asnumpy()
            if kind == "mh_sddmm":
                m = min(e, 3_000_000)
                s_h, d_h = src.cpu().numpy(), dst.cpu().numpy()
                ok = True
                for sl in (slice(0, m), slice(e - m, e)):
                    want = ref.sddmm_mh(coo.row[sl], coo.col[sl], s_h, d_h)
                    ok = ok and bool(np.all(np.abs(out[sl] - want) <= ATOL + RTOL * np.abs(want)))
                row["parity"] = {"within_rtol1e-5_atol1e-4_of_cpu_checker": ok, "edges_checked": 2 * m}
            elif kind == "mh_sddmm_softmax":
                # the first rows' edges: scores by the CPU checker, softmax in float64, against the fused kernel
                n_check = int(np.searchsorted(graph_adj.indptr, 3_000_000))
                m = int(graph_adj.indptr[n_check])
                scores = ref.sddmm_mh(coo.row[:m], coo.col[:m], src.cpu().numpy(), dst.cpu().numpy())
                want = ref.edge_softmax(graph_adj.indptr[:n_check + 1], scores)
                ok = bool(np.all(np.abs(out[:m] - want) <= 1e-6 + 1e-4 * np.abs(want)))
                row["parity"] = {"within_rtol1e-4_atol1e-6_of_cpu_checker": ok, "edges_checked": m}
            elif kind in ("mh_attention", "mh_attention_kv"):
                # the first rows (the three CPU checkers one after the other on their sub-matrix) against the kernel
                n_check = int(np.searchsorted(graph_adj.indptr, 1_500_000))
                m = int(graph_adj.indptr[n_check])
                hosts = [x.cpu().numpy() for x in ins]
                want = ref.attention_mh(graph_adj.indptr[:n_check + 1], graph_adj.indices[:m], hosts[0],
                                        hosts[1][:n_check], hosts[2] if len(hosts) == 3 else None)
                ok = bool(np.all(np.abs(out[:n_check] - want) <= 1e-5 + 1e-4 * np.abs(want)))
                row["parity"] = {"within_rtol1e-4_atol1e-5_of_cpu_checker": ok, "rows_checked": n_check,
                                 "edges_checked": m}
            else:
                want = ref.spmm_mh(graph_adj.indptr, graph_adj.indices, w.cpu().numpy(), src.cpu().numpy())
                row["parity"] = {"bit_exact_vs_cpu_checker": bool(np.array_equal(out, want))}
        if p and kind in ("mh_spmm", "mh_attention", "mh_attention_kv"):
            # these store one result row per destination row; the probe with stores in the same proportion (it
            # overwrites the result, hence after the parity check) gives a ceiling that such an operator can reach
            gathers = e * (2 if kind == "mh_attention_kv" else 1)
            pw = rows_write_probe(src, op.out_tvm.tensor, gathers, n_r, p["ms"])
            if pw:
                row.update({"gather_store_ceiling_ms": pw["ms"], "frac_of_gather_store_ceiling": pw["ms"] / ms,
                            "gather_store_probe": pw})
        return row

    if args.only in ("mh_sddmm", "mh_spmm", "mh_sddmm_softmax", "mh_attention", "mh_attention_kv", "mh_attention_grad"):
        row = mh_case(args.only, adj, F, args.steps, args.warmup, False)
        row.update({"kernel": args.only, "graph": args.graph})
        print(json.dumps(row))
        return

    # module construction = upload of the adjacency + plan creation: once per graph, outside every timed region
    spmm = sddmm = None
    plan_seconds = {}
    if args.only in ("all", "spmm"):
        torch.cuda.synchronize(dev)
        t = time.time()
        spmm = VanillaSpMMhip(adj)
        torch.cuda.synchronize(dev)
        plan_seconds["spmm"] = time.time() - t
    if args.only in ("all", "sddmm", "sddmm_shuffled"):
        coo = adj.tocoo()
        if args.only == "sddmm_shuffled":  # the same edges in a seeded random order (the sweep's shuffled row)
            import scipy.sparse
            perm = np.random.default_rng(17).permutation(nnz)
            coo = scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])), shape=coo.shape)
            del perm
        torch.cuda.synchronize(dev)
        t = time.time()
        sddmm = VanillaSDDMMhip(coo)
        torch.cuda.synchronize(dev)
        plan_seconds["sddmm"] = time.time() - t

    def spmm_case(F, feat_np=None, seed=21):
        feat = nd.array(feat_np, dev) if feat_np is not None else nd.array(device_normal((n_cols, F), seed + F))
        spmm.build([placeholder((n_cols, F))], {}, {})
        return feat

    def sddmm_case(module, F):
        src = nd.array(device_normal((n_cols, F), 31 + F))
        dst = nd.array(device_normal((n_rows, F), 41 + F))
        module.build([placeholder((n_cols, F)), placeholder((n_rows, F))], {}, {})
        return [src, dst]

    if args.only in ("sddmm", "sddmm_shuffled"):
        ins = sddmm_case(sddmm, F)
        ms = timed(lambda: sddmm.run(ins), args.steps, args.warmup)
        b = sddmm_alg_bytes(nnz, F)
        print(json.dumps({"kernel": args.only, "F": F, "nnz": nnz, "n_cols": n_cols, "ms": ms, "alg_GBps": b / ms / 1e6,
                          "frac": b / ms / 1e6 / HBM_PEAK_GBPS, "plan_seconds": plan_seconds["sddmm"]}))
        return

    # ---- the timed step: CSR SpMM, feature length F --------------------------------
    feat_np = datasets.spmm_operands(adj, F)
    feat = spmm_case(F, feat_np)
    ms = timed(lambda: spmm.run([feat]), args.steps, args.warmup)
    flops = 2.0 * nnz * F
    alg = spmm_alg_bytes(nnz, n_rows, F)
    b_min = spmm_min_bytes(nnz, n_rows, n_cols, F)
    achieved = alg / ms / 1e6
    gpu_out = spmm.out_tvm.asnumpy() if args.only == "all" else None
    traffic, traffic_source = committed_traffic("spmm", args.graph, F)
    probe = gather_probe(feat.tensor, nnz) if args.only == "all" else None
    probe_hit = gather_probe_at_hit_rate(feat.tensor, nnz, "spmm", F) if args.only == "all" else None
    probe_mix = gather_and_stream_probe_at_hit_rate(feat.tensor, nnz, "spmm", F) if args.only == "all" else None
    launch_text = spmm.lower_to_ir([placeholder((n_cols, F))], {}, {})
    m_pass = re.search(r"(\d+) launch", launch_text)
    launch_dispatches = int(m_pass.group(1)) if m_pass else None
    roofline = {
        "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
        "traffic": traffic, "traffic_source": traffic_source,
        "algorithmic_bytes": alg, "kernel": "spmm_multi_kernel<%d,true,true,-1,0>" % (4 if F <= 16 else 8 if F <= 32 else 16),
        "launch_ms": ms,
        "compulsory_bytes": b_min, "hbm_frac_compulsory": b_min / ms / 1e6 / HBM_PEAK_GBPS,
        "l2_fabric_frac": (traffic / ms / 1e6 / HBM_PEAK_GBPS) if traffic else None,
        "frac_bounded": (traffic / ms / 1e6 / HBM_PEAK_GBPS) if traffic else None,
        "dispatches_per_launch": launch_dispatches,
        "gather_ceiling": probe, "frac_of_gather_ceiling": (probe["ms"] / ms) if probe else None,
        "gather_at_the_operators_l2_hit_rate": probe_hit,
        "frac_of_gather_at_the_operators_l2_hit_rate": (probe_hit["ms"] / ms) if probe_hit else None,
        "gather_and_stream_at_the_operators_l2_hit_rate": probe_mix,
        "frac_of_gather_and_stream_at_the_operators_l2_hit_rate": (probe_mix["ms"] / ms) if probe_mix else None,
        "note": "`achieved` is the gather model (no cache reuse credited): most of those bytes are served by L2 / "
                "Infinity Cache and never reach HBM, so `frac` is not bounded by 1 on this graph; "
                "hbm_frac_compulsory, l2_fabric_frac and the two frac_of_gather_* are (the bare gather stream with "
                "nearly every gather hitting L2, and with the band widened until the probe's hit rate is the "
                "operator's). One operator launch is one "
                "dispatch per column-block pass and feature tile (see `launch`); bytes, time and traffic are per "
                "operator launch. `traffic` is read from the committed profile named in traffic_source, not "
                "measured in this run."}
    result = {
        "metric": "SpMM GFLOP/s (vanilla CSR, fp32, feat-len %d)" % F,
        "value": flops / ms / 1e6, "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s: vanilla CSR SpMM, %d vertices, %d nonzeros, feat-len %d" % (
            args.graph, n_rows, nnz, F), "graph_checksum": datasets.structure_checksum(adj)},
        "roofline": roofline,
        "launch": launch_text,
        "plan_seconds": plan_seconds,
    }
    if args.only == "spmm":
        print(headline_line(result))
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

    check = not args.no_cpu
    if check:
        from oracle import ref
        cores = ref.num_threads()

    # ---- sweep, reference protocol: one warm-up, mean of five (bench_vanilla_spmm.py:32-33) ------
    if not args.no_sweep:
        sweep = []
        m = min(nnz, 4_000_000)
        def ramp(fn):
            # untimed launches that bring the clocks back up after host-side work (operand generation, the CPU
            # checker); the measurement itself stays one warm-up + five timed runs
            for _ in range(10):
                fn()
            torch.cuda.synchronize(dev)

        for f in FEAT_LENS:
            x = spmm_case(f)
            ramp(lambda: spmm.run([x]))
            sec = spmm.measure_average_time([x], 5)
            b = spmm_alg_bytes(nnz, n_rows, f)
            tr, src_file = committed_traffic("spmm", args.graph, f)
            p = gather_probe(x.tensor, nnz)
            ph = gather_probe_at_hit_rate(x.tensor, nnz, "spmm", f)
            ph_sddmm = gather_probe_at_hit_rate(x.tensor, nnz, "sddmm", f)  # same gathers, SDDMM's hit rate
            row = {"op": "spmm", "F": f, "ms": sec * 1e3, "GFLOPs": 2.0 * nnz * f / sec / 1e9,
                   "alg_GBps": b / sec / 1e9, "frac": b / sec / 1e9 / HBM_PEAK_GBPS,
                   "hbm_frac_compulsory": spmm_min_bytes(nnz, n_rows, n_cols, f) / sec / 1e9 / HBM_PEAK_GBPS,
                   "traffic": tr, "traffic_source": src_file,
                   "gather_ceiling_ms": p["ms"] if p else None,
                   "frac_of_gather_ceiling": p["ms"] / (sec * 1e3) if p else None,
                   "gather_at_the_operators_l2_hit_rate": ph,
                   "frac_of_gather_at_the_operators_l2_hit_rate": ph["ms"] / (sec * 1e3) if ph else None}
            if check:
                t0 = time.time()
                want = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, x.tensor.cpu().numpy())
                row["parity"] = {"bit_exact_vs_cpu_restatement": bool(np.array_equal(spmm.out_tvm.asnumpy(), want)),
                                 "cpu_seconds": time.time() - t0}
                del want
            sweep.append(row)
            del x
            ins = sddmm_case(sddmm, f)
            ramp(lambda: sddmm.run(ins))
            sec = sddmm.measure_average_time(ins, 5)
            b = sddmm_alg_bytes(nnz, f)
            tr, src_file = committed_traffic("sddmm", args.graph, f)
            row = {"op": "sddmm", "F": f, "ms": sec * 1e3, "GFLOPs": 2.0 * nnz * f / sec / 1e9,
                   "alg_GBps": b / sec / 1e9, "frac": b / sec / 1e9 / HBM_PEAK_GBPS,
                   "hbm_frac_compulsory": sddmm_min_bytes(nnz, n_rows, n_cols, f) / sec / 1e9 / HBM_PEAK_GBPS,
                   "traffic": tr, "traffic_source": src_file,
                   "gather_ceiling_ms": p["ms"] if p else None,
                   "frac_of_gather_ceiling": p["ms"] / (sec * 1e3) if p else None,
                   "gather_at_the_operators_l2_hit_rate": ph_sddmm,
                   "frac_of_gather_at_the_operators_l2_hit_rate": ph_sddmm["ms"] / (sec * 1e3) if ph_sddmm else None}
            pm = gather_and_stream_probe_at_hit_rate(ins[0].tensor, nnz, "sddmm", f)   # 64 floats only
            if pm:
                row["gather_and_stream_at_the_operators_l2_hit_rate"] = pm
                row["frac_of_gather_and_stream_at_the_operators_l2_hit_rate"] = pm["ms"] / (sec * 1e3)
            if check:
                out = sddmm.out_tvm.asnumpy()
                s_h, d_h = ins[0].tensor.cpu().numpy(), ins[1].tensor.cpu().numpy()
                ok = True
                for sl in (slice(0, m), slice(nnz - m, nnz)):
                    exact = ref.sddmm_f64(coo.row[sl], coo.col[sl], s_h, d_h)
                    ok = ok and bool(np.all(np.abs(out[sl] - exact) <= ATOL + RTOL * np.abs(exact)))
                row["parity"] = {"within_rtol1e-5_atol1e-4_of_float64": ok, "edges_checked": 2 * m}
                del out, s_h, d_h
            sweep.append(row)
            del ins
            torch.cuda.empty_cache()
            log("sweep F=%d: spmm %.3f ms (%.2f of the gather ceiling), sddmm %.3f ms (%.2f)" % (
                f, sweep[-2]["ms"], sweep[-2]["frac_of_gather_ceiling"] or 0, sweep[-1]["ms"],
                sweep[-1]["frac_of_gather_ceiling"] or 0))

        # the same edge list in a seeded random order: not row-sorted, so the plan works on a sorted copy and
        # gathers the results back to the caller's order
        import scipy.sparse
        perm = np.random.default_rng(17).permutation(nnz)
        shuffled = VanillaSDDMMhip(scipy.sparse.coo_matrix((coo.data[perm], (coo.row[perm], coo.col[perm])),
                                                           shape=coo.shape))
        ins = sddmm_case(shuffled, F)
        ramp(lambda: shuffled.run(ins))
        sec = shuffled.measure_average_time(ins, 5)
        b = sddmm_alg_bytes(nnz, F)
        row = {"op": "sddmm", "F": F, "edge_order": "shuffled (seeded permutation of the c2 list)",
               "ms": sec * 1e3, "GFLOPs": 2.0 * nnz * F / sec / 1e9, "alg_GBps": b / sec / 1e9,
               "frac": b / sec / 1e9 / HBM_PEAK_GBPS}
        if check:
            out = shuffled.out_tvm.asnumpy()[:m]
            exact = ref.sddmm_f64(coo.row[perm[:m]], coo.col[perm[:m]], ins[0].tensor.cpu().numpy(),
                                  ins[1].tensor.cpu().numpy())
            row["parity"] = {"within_rtol1e-5_atol1e-4_of_float64":
                             bool(np.all(np.abs(out - exact) <= ATOL + RTOL * np.abs(exact))), "edges_checked": m}
            del out, exact
        sweep.append(row)
        log("sddmm on the shuffled list, F=%d: %.3f ms" % (F, sec * 1e3))
        del shuffled, ins, perm
        torch.cuda.empty_cache()

        # the generalised aggregation (message x reducer) at the headline length: same gathers as the vanilla
        # operator, one more operand per nonzero when the message uses the edge value
        x = spmm_case(F)
        for msg, reduce in (("mul", "sum"), ("copy_u", "max"), ("add", "min"), ("mul", "mean")):
            general = GeneralizedSpMMhip(adj, msg, reduce)
            general.build([placeholder((n_cols, F))], {}, {})
            ramp(lambda: general.run([x]))
            sec = general.measure_average_time([x], 5)
            b = spmm_alg_bytes(nnz, n_rows, F)
            row = {"op": "spmm_general", "msg": msg, "reduce": reduce, "F": F, "ms": sec * 1e3,
                   "alg_GBps": b / sec / 1e9, "frac": b / sec / 1e9 / HBM_PEAK_GBPS}
            if check:
                want = ref.spmm_general(adj.indptr, adj.indices, adj.data, x.tensor.cpu().numpy(), msg, reduce)
                row["parity"] = {"bit_exact_vs_cpu_restatement":
                                 bool(np.array_equal(general.out_tvm.asnumpy(), want, equal_nan=True))}
                del want
            sweep.append(row)
            log("spmm_general %s/%s F=%d: %.3f ms" % (msg, reduce, F, sec * 1e3))
            del general
        del x
        torch.cuda.empty_cache()
        result["sweep"] = sweep

    # ---- multi-head operators on the 2.45M-vertex graph (features far beyond the caches: HBM-bound) ----
    if not args.no_mh:
        sddmm = None
        torch.cuda.empty_cache()
        t = time.time()
        big = datasets.config_graph("c4")
        log("graph c4: %d vertices, nnz %d, checksum %s (%.1f s)" % (
            big.shape[0], big.nnz, datasets.structure_checksum(big), time.time() - t))
        mh = []
        for D in MH_HEAD_LENS:
            mh.append(mh_case("mh_sddmm", big, D, 5, 1, check))
            torch.cuda.empty_cache()
            log("mh_sddmm D=%d: %.3f ms (%.2f of the HBM roofline by algorithmic bytes)" % (
                D, mh[-1]["ms"], mh[-1]["frac"]))
        # the GAT chain between them: scores + edge softmax in one kernel, against the two operators run
        # one after the other (multi-head SDDMM, then the softmax over its [nnz, 8] output)
        for D in MH_HEAD_LENS:
            mh.append(mh_case("mh_sddmm_softmax", big, D, 5, 1, check))
            torch.cuda.empty_cache()
            log("mh_sddmm_softmax (fused) D=%d: %.3f ms" % (D, mh[-1]["ms"]))
        soft = EdgeSoftmaxhip(big)
        soft.build([placeholder((big.nnz, MH_HEADS))], {}, {})
        scores = device_normal((big.nnz, MH_HEADS), 5)
        soft_ms = timed(lambda: soft.run([scores]), 5, 1)
        mh.append({"op": "edge_softmax", "H": MH_HEADS, "ms": soft_ms,
                   "note": "standalone pass over [nnz, 8] scores: what the fused operator saves on top of the "
                           "scores' round trip"})
        del soft, scores
        torch.cuda.empty_cache()
        mh.append(mh_case("mh_spmm", big, 64, 5, 1, check))
        log("mh_spmm D=64: %.3f ms (%.2f of the HBM roofline by algorithmic bytes)" % (mh[-1]["ms"], mh[-1]["frac"]))
        torch.cuda.empty_cache()
        # the whole layer in one kernel: scores, softmax and weighted sum, with the vertex features as key and value
        # (one gather per neighbour) and with a separate value matrix (two)
        chain_ms = {r["D"]: r["ms"] for r in mh if r["op"] == "mh_sddmm_softmax"}
        spmm_ms = mh[-1]["ms"]
        for kind in ("mh_attention", "mh_attention_kv"):
            mh.append(mh_case(kind, big, 64, 5, 1, check))
            mh[-1]["chain_ms"] = chain_ms[64] + spmm_ms
            mh[-1]["speedup_over_chain"] = mh[-1]["chain_ms"] / mh[-1]["ms"]
            torch.cuda.empty_cache()
            log("%s D=64: %.3f ms (scores + softmax, then multi-head SpMM: %.3f ms)" % (
                kind, mh[-1]["ms"], mh[-1]["chain_ms"]))
        hb = next(r for r in mh if r["op"] == "mh_spmm")
        result["roofline_hbm_bound_config"] = {
            "workload": "c5: multi-head CSR SpMM, %d vertices, %d edges, H=8, D=64" % (big.shape[0], big.nnz),
            "ms": hb["ms"], "algorithmic_bytes": hb["algorithmic_bytes"], "achieved": hb["alg_GBps"],
            "frac": hb["frac"], "traffic": hb.get("traffic"), "frac_traffic": hb.get("hbm_frac_traffic"),
            "parity": (hb.get("parity") or {}).get("bit_exact_vs_cpu_checker")}
        mh.append(mh_case("mh_attention_grad", big, 64, 3, 1, False))
        torch.cuda.empty_cache()
        log("mh_attention_grad D=64 (value = key): %.3f ms" % mh[-1]["ms"])
        result["multi_head"] = {"graph": "c4: %d vertices, %d edges" % (big.shape[0], big.nnz), "rows": mh,
                                "note": "1.25 - 5 GB of features and mean degree 25: nearly every neighbour gather "
                                        "goes to HBM.  `frac` is algorithmic bytes / time / 8 TB/s (above 1 for SDDMM "
                                        "because consecutive edges share their Dst row, which caches serve); "
                                        "hbm_frac_traffic is the committed rocprofv3 byte count of the operator / time "
                                        "/ 8 TB/s; frac_of_gather_ceiling is the time of the same number of random "
                                        "whole-row gathers and nothing else (fg_probe_gather_rows_f32) / time"}
        del big
        torch.cuda.empty_cache()

    # ---- the reference's own CPU-sized case (c1: 4096 vertices): launch-bound, eager against a HIP graph ----
    if args.only == "all" and not args.no_sweep:
        small = datasets.config_graph("c1")
        ns = small.shape[0]
        s_spmm, s_sddmm = VanillaSpMMhip(small), VanillaSDDMMhip(small.tocoo())
        s_spmm.build([placeholder((ns, 64))], {}, {})
        s_sddmm.build([placeholder((ns, 64)), placeholder((ns, 64))], {}, {})
        xs, ys = device_normal((ns, 64), 51), device_normal((ns, 64), 52)

        def pair():
            s_spmm.run([xs])
            s_sddmm.run([xs, ys])

        eager_us = timed(pair, 200, 20) * 1e3
        eager_out = s_sddmm.out_tvm.tensor.clone()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            pair()
        stream.wait_stream(side)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(10):
                pair()
        s_sddmm.out_tvm.tensor.zero_()
        graph_us = timed(graph.replay, 20, 3) * 1e3 / 10
        result["small_graph"] = {
            "graph": "c1: %d vertices, %d nonzeros, feat-len 64" % (ns, small.nnz),
            "us_per_spmm_plus_sddmm_eager": eager_us, "us_per_spmm_plus_sddmm_in_hip_graph": graph_us,
            "graph_replay_matches_eager": bool(torch.equal(s_sddmm.out_tvm.tensor, eager_out)),
            "note": "one SpMM and one SDDMM call per step; the run paths only enqueue kernels, so ten steps "
                    "recorded into one HIP graph replay without the per-launch host cost"}
        log("c1 (4096 vertices): SpMM + SDDMM %.1f us eager, %.1f us per step inside a HIP graph" % (eager_us, graph_us))
        del s_spmm, s_sddmm, graph

    # ---- CPU baseline: the restated x86 nest on this machine's cores ----------------------------
    if check:
        work = np.empty((n_cols + n_rows) * F, dtype=np.float32)
        per_p = {}
        cpu_out = None
        for P in [p for p in (1, 2, 4, 8, 16, 32) if p <= max(1, F // 16)]:   # bench_vanilla_spmm.py:37
            t0 = time.time()
            o = ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat_np, P, work)   # warm-up
            first = time.time() - t0
            if P == 1:
                cpu_out = o
            runs = int(max(1, min(10, 5.0 / max(first, 1e-3))))   # about five seconds of CPU work per setting
            t0 = time.time()
            for _ in range(runs):
                ref.spmm_csr_x86(adj.indptr, adj.indices, adj.data, feat_np, P, work)
            per_p[P] = {"seconds": (time.time() - t0) / runs, "runs": runs}
        best = min(per_p, key=lambda p: per_p[p]["seconds"])
        cpu_s = per_p[best]["seconds"]
        result["cpu_baseline"] = {
            "value": flops / cpu_s / 1e9, "unit": "GFLOP/s", "cores": cores, "kind": "port", "seconds": cpu_s,
            "cpu_model": cpu_model(), "best_num_feat_partitions": best,
            "value_at_num_feat_partitions_1": flops / per_p[1]["seconds"] / 1e9,
            "per_num_feat_partitions": {str(p): v for p, v in per_p.items()},
            "sample": "whole workload, restated x86 nest, num_feat_partitions in %s, mean of %d run(s)" % (
                sorted(per_p), per_p[best]["runs"])}
        result["parity"] = {"spmm_bit_exact_vs_cpu_restatement": bool(np.array_equal(gpu_out, cpu_out)),
                            "spmm_max_abs_diff": float(np.max(np.abs(gpu_out - cpu_out)))}
        # distance of the float32 result (the reference's summation order) from the exact sum, by row degree
        exact = ref.spmm_csr_f64(adj.indptr, adj.indices, adj.data, feat_np)
        err = np.abs(gpu_out.astype(np.float64) - exact).max(axis=1)
        mag = np.abs(exact).max(axis=1)
        deg = np.diff(adj.indptr)
        bins = []
        for lo_d, hi_d in ((0, 64), (64, 512), (512, 4096), (4096, 1 << 30)):
            sel = (deg >= lo_d) & (deg < hi_d)
            if sel.any():
                bins.append({"degree": "%d..%s" % (lo_d, hi_d - 1 if hi_d < (1 << 30) else "max"),
                             "rows": int(sel.sum()), "max_abs_err": float(err[sel].max()),
                             "max_err_over_row_magnitude": float((err[sel] / np.maximum(mag[sel], 1e-30)).max())})
        result["parity"]["spmm_float32_vs_exact_sum_by_row_degree"] = bins
        del exact, err, mag
        if "sweep" in result:
            result["parity"]["every_sweep_row_passes"] = all(
                all(v for k, v in r["parity"].items() if isinstance(v, bool)) for r in result["sweep"] if "parity" in r)
        # SDDMM: the reference's x86 schedule is serial, so a bounded sample of the edge list on one core
        m = min(nnz, 4_000_000)
        rng = np.random.default_rng(2)
        src = rng.standard_normal((n_cols, F), dtype=np.float32)
        dst = rng.standard_normal((n_rows, F), dtype=np.float32)
        ref.sddmm_x86(coo.row[:m], coo.col[:m], src, dst)
        t0 = time.time()
        ref.sddmm_x86(coo.row[:m], coo.col[:m], src, dst)
        strict_s = time.time() - t0
        buf = np.empty(m, dtype=np.float32)
        ref.sddmm_x86_fast(coo.row[:m], coo.col[:m], src, dst, False, buf)
        t0 = time.time()
        ref.sddmm_x86_fast(coo.row[:m], coo.col[:m], src, dst, False, buf)
        simd_s = time.time() - t0
        # courtesy number, not the reference's schedule: the whole edge list, edge-parallel on every core
        full = np.empty(nnz, dtype=np.float32)
        ref.sddmm_x86_fast(coo.row, coo.col, src, dst, True, full)
        t0 = time.time()
        ref.sddmm_x86_fast(coo.row, coo.col, src, dst, True, full)
        all_cores_s = time.time() - t0
        del full
        result["cpu_baseline_sddmm"] = {
            "value": 2.0 * m * F / strict_s / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "cpu_model": cpu_model(),
            "value_all_cores_edge_parallel_not_the_reference_schedule": 2.0 * nnz * F / all_cores_s / 1e9,
            "all_cores": cores,
            "variant": "strict serial nest: edge loop outside, k loop inside, sequential float32 sum "
                       "(op/vanilla_sddmm.py:43-47 under the default schedule :66-74, which has no parallel axis)",
            "value_with_reassociated_simd_k_loop": 2.0 * m * F / simd_s / 1e9,
            "sample": "first %d edges of the row-sorted COO list, feat-len %d, one run after one warm-up" % (m, F)}
    try:
        import tvm  # noqa: F401  (the reference's code generator; not expected on this machine)
        result["tvm_available"] = True
    except Exception:
        result["tvm_available"] = False
    emit(result)


if __name__ == "__main__":
    main()
