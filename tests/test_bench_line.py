"""The benchmark's last stdout line must stay short enough for a harness that keeps only the tail of stdout:
built here from a canned detail record of realistic size (every optional part present), no GPU involved."""
import json

import bench


def _canned():
    long_text = "x" * 400
    roofline = {
        "bound": "hbm", "achieved": 16886.123456789, "peak": 8000.0, "unit": "GB/s", "frac": 2.110765432,
        "frac_bounded": 0.655123456, "traffic": 9410000000.0, "traffic_source": "profiles/spmm_c2_counters.txt",
        "algorithmic_bytes": 30316754220, "kernel": "spmm_multi_kernel<16,true,true,-1,0> (CSR, feat-len 64)",
        "dispatches_per_launch": 12, "launch_ms": 1.7951234, "compulsory_bytes": 1036000000,
        "hbm_frac_compulsory": 0.0721234, "l2_fabric_frac": 0.655123456,
        "gather_ceiling": {"ms": 1.0, "tile": 64, "band_rows": 16384, "note": long_text},
        "frac_of_gather_ceiling": 0.5571234, "gather_at_the_operators_l2_hit_rate": {"ms": 1.3, "note": long_text},
        "frac_of_gather_at_the_operators_l2_hit_rate": 0.72123456,
        "gather_and_stream_at_the_operators_l2_hit_rate": {"ms": 1.5, "note": long_text},
        "frac_of_gather_and_stream_at_the_operators_l2_hit_rate": 0.85123456, "note": long_text * 3}
    return {
        "metric": "SpMM GFLOP/s (vanilla CSR, fp32, feat-len 64)", "value": 8171.123456, "unit": "GFLOP/s",
        "n_gpus": 1, "steps": 20, "warmup": 3, "ms_per_step": 1.7951234, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "c2: vanilla CSR SpMM, 232965 vertices, 114606755 nonzeros, feat-len 64",
                   "graph_checksum": "0123456789abcdef"},
        "roofline": roofline,
        "roofline_hbm_bound_config": {
            "workload": "c5: multi-head CSR SpMM, 2449029 vertices, 61948164 edges, H=8, D=64", "ms": 23.48123,
            "algorithmic_bytes": 134130000000, "achieved": 5712.3456, "frac": 0.7140432, "traffic": 143900000000.0,
            "frac_traffic": 0.766123, "parity": True},
        "launch": long_text, "plan_seconds": {"spmm": 0.1, "sddmm": 0.1},
        "sweep": [{"op": "spmm", "F": f, "ms": 1.0, "note": long_text} for f in (32, 64, 128, 256, 512)] * 3,
        "multi_head": {"graph": "c4", "rows": [{"op": "mh_sddmm", "D": 16, "note": long_text}] * 10, "note": long_text},
        "cpu_baseline": {
            "value": 145.123456, "unit": "GFLOP/s", "cores": 16, "kind": "port", "seconds": 0.101234,
            "cpu_model": "AMD EPYC 9575F 64-Core Processor", "best_num_feat_partitions": 4,
            "value_at_num_feat_partitions_1": 44.1, "per_num_feat_partitions": {"1": {"seconds": 0.33, "runs": 10}},
            "sample": "whole workload, restated x86 nest, num_feat_partitions in [1, 2, 4], mean of 10 run(s)"},
        "parity": {"spmm_bit_exact_vs_cpu_restatement": True, "spmm_max_abs_diff": 0.0,
                   "every_sweep_row_passes": True, "spmm_float32_vs_exact_sum_by_row_degree": [{"rows": 1}] * 4},
        "tvm_available": False}


def test_headline_is_short_and_round_trips():
    line = bench.headline_line(_canned(), "bench_out/bench_detail.json")
    assert "\n" not in line and len(line) < 1500
    got = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "dtype", "config",
                "roofline", "cpu_baseline", "parity", "vs_baseline", "higher_is_better", "scaling", "data"):
        assert key in got
    assert got["config"]["workload"].startswith("c2")
    for key in ("bound", "achieved", "peak", "unit", "frac", "frac_bounded", "traffic", "traffic_source",
                "algorithmic_bytes", "kernel"):
        assert key in got["roofline"]
    assert got["roofline"]["frac_bounded"] <= 1.0
    assert abs(got["roofline"]["frac"] - got["roofline"]["achieved"] / got["roofline"]["peak"]) < 1e-3
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in got["cpu_baseline"]
    assert got["parity"] is True
    assert abs(got["roofline_hbm_bound_config"]["frac"] - 0.714) < 1e-3


def test_headline_reports_a_failed_parity_flag():
    rec = _canned()
    rec["parity"]["every_sweep_row_passes"] = False
    assert json.loads(bench.headline_line(rec))["parity"] is False


def test_headline_refuses_to_grow():
    rec = _canned()
    rec["cpu_baseline"]["sample"] = "y" * 2000
    try:
        bench.headline_line(rec)
    except RuntimeError as e:
        assert "limit" in str(e)
    else:
        raise AssertionError("an oversized line was printed")


def test_the_committed_counter_summaries_are_still_what_the_benchmark_reads():
    """roofline.traffic, frac_bounded and the probes' bands come from profiles/*_counters.txt: every swept feature
    length and multi-head row must parse, with bytes and hit rates in a plausible range."""
    for op in ("spmm", "sddmm"):
        for F in (32, 64, 128, 256, 512):
            traffic, src = bench.committed_traffic(op, "c2", F)
            hit, src2 = bench.committed_hit_rate(op, "c2", F)
            assert src == src2 == "profiles/%s_c2_counters.txt" % op
            assert 1e9 < traffic < 2e11 and 0.3 < hit < 1.0, (op, F, traffic, hit)
    for kind, D in (("mh_sddmm", 16), ("mh_sddmm", 64), ("mh_spmm", 64)):
        traffic, src = bench.committed_traffic_mh(kind, D)
        assert src == "profiles/multihead_c4_counters.txt" and 1e10 < traffic < 5e11, (kind, D, traffic)
    assert bench.committed_traffic("spmm", "c2", 48) == (None, None)
