"""The last stdout line of bench.py stays short enough to survive a consumer that keeps only the tail of stdout, and the
reachability bound it reports is what a breadth-first search over the graph gives (no GPU needed)."""
import argparse
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import bench  # noqa: E402


def fake_result(name, met):
    """A result of the shape run_workload() returns, with long lists where the real one has them."""
    stage = dict(bound="hbm", seconds=0.123456789, algorithmic_bytes=12345678901234, achieved=5247.222706563232, peak=8000.0, unit="GB/s",
                 frac=0.6559028383204041, valu_yardstick_frac=0.951234567)
    return dict(
        workload=bench.WORKLOADS[name][5], gen_sec=3.2, build_sec=0.31912345678, stage_rooflines={k: dict(stage) for k in ("assign", "reorder", "knn", "subgraph+boundary", "refine")},
        build_stages=dict(pre=0.0051234567, knn=0.14412345678, index=0.0712345678, refine=0.0991234567, detail={k: 0.0123456789 for k in "abcdefg"}),
        nnd_iterations=20, nnd_offers=1351000000, nnd_offers_declined_by_threshold=238000000, nnd_offers_note=bench.NND_OFFERS_NOTE,
        graph_recall_at_32=0.98723456789, graph_recall_at_32_global=0.9912345678, partition_sizes=list(range(17)), empty_slots_fraction=0.4512345,
        sweep=[dict(beam=b, recall_at_10=0.22612345678, qps=3340000.123456, ms=2.99412345, iterations_per_query=261.12345, rows_per_query=3090.12345,
                    algorithmic_bytes=16160000000) for b in (32, 64, 128, 192, 224, 256, 320, 384, 448, 512)],
        beam=256, recall_at_10=0.22612345678, recall_target_met=met, reachable_recall_bound=0.2512345678, reachable_fraction_of_points=0.2412345,
        qps=3340000.123456, ms_per_step=2.99412345678, kernel_ms=2.9871234567,
        roofline=dict(bound="hbm", achieved=5400.123456789, peak=8000.0, unit="GB/s", frac=0.67501234567, traffic=12960000000.0,
                      traffic_source="profiles/search_kernels_hbm_traffic.md", kernel="search_kernel_dense<64,256,1>", algorithmic_bytes_per_launch=16160000000),
        cpu_baseline=dict(value=14200.123456, unit="queries/s", cores=16, kind="port",
                          sample="beam search of the first 10000 queries (same index, beam 256) with the CPU restatement, 16 threads",
                          recall_at_10=0.22614, nnd_points_per_sec=20900.12345, nnd_sample="x" * 90, bruteforce_qps=510.12345, bruteforce_sample="y" * 90))


def test_headline_line_is_compact_and_round_trips():
    args = argparse.Namespace(steps=20, warmup=5)
    for met in (False, True):
        details = {n: fake_result(n, met or n in ("cfg1-navigable", "cfg3")) for n in ("cfg1", "cfg1-navigable", "cfg0", "cfg2", "cfg3")}
        text = json.dumps(bench.headline(args, "cfg1", details, "AMD Instinct MI355X"), default=float)
        assert len(text) <= 4096, len(text)
        line = json.loads(text)
        for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data",
                    "config", "roofline", "cpu_baseline", "recall_target_met", "reachable_recall_bound", "build_sec", "graph_recall_at_32"):
            assert key in line, key
        assert set(("bound", "achieved", "peak", "unit", "frac", "traffic")) <= set(line["roofline"])
        assert set(("value", "unit", "cores", "kind", "sample")) <= set(line["cpu_baseline"])
        assert line["config"]["workload"].startswith("cfg1:")
        # the metric string says what `value` is
        assert ("unreachable" in line["metric"]) == (not met)
        assert (line["qps_at_recall_target"] is None) == (not met)
        assert sorted(line["recall_target_met_on"]) == (sorted(details) if met else ["cfg1-navigable", "cfg3"])


def test_reachable_recall_bound_on_a_hand_built_graph():
    """Two chains that never meet; each centroid's start point sits at the head of one.  A query's true neighbours on the
    other chain are out of reach, those on its own chain (behind the start point) are in; the start point itself counts
    only if an edge leads back to it."""
    E = 0xFFFFFFFF
    graph = np.array([[1, E], [2, E], [3, E], [E, E],          # chain A: 0 -> 1 -> 2 -> 3
                      [5, E], [6, 4], [7, E], [E, E]], np.uint32)   # chain B: 4 -> 5 -> 6 -> 7, and 5 -> 4 leads back to the start
    centroids = np.array([[0.0, 0.0], [10.0, 0.0]], np.float32)
    start_points = np.array([0, 4], np.uint32)
    queries = np.array([[1.0, 0.0], [9.0, 0.0], [9.0, 1.0]], np.float32)
    gt = np.array([[0, 1], [4, 3], [7, 6]], np.uint32)   # query 0: start point 0 is never scored (no edge back), 1 is reachable
    from glide_amd import datasets as Ds
    bound, frac, per_query = Ds.reachable_recall_bound(graph, centroids, start_points, queries, gt)
    assert per_query.tolist() == [0.5, 0.5, 1.0]
    # query 0: {1} of {0, 1} -> 0.5; query 1: 4 reachable (edge back), 3 on the other chain -> 0.5; query 2: both -> 1.0
    assert abs(bound - (0.5 + 0.5 + 1.0) / 3) < 1e-12
    assert abs(frac - (3 / 8 + 4 / 8) / 2) < 1e-12


def test_committed_profile_tables_are_readable():
    """bench.py takes measured traffic, stage counters and the scattered-row ceiling from the committed profile summaries;
    a change of their table format must not silently turn those fields into nulls."""
    for workload, beam in (("cfg1", 256), ("cfg1-navigable", 32), ("cfg3", 448)):
        t = bench.measured_traffic(workload, beam)
        assert t and t["bytes"] > 1e9, (workload, beam)
    for workload in ("cfg1", "cfg1-navigable", "cfg0", "cfg2", "cfg3"):
        for stage in ("subgraph+boundary", "refine"):
            m = bench.measured_stage(stage, workload)
            assert m and m[0] > 1e9 and m[2] > 100 and m[3] > 1.5, (stage, workload)
    assert bench.measured_knn("cfg1") and bench.measured_knn_bytes("cfg1") > 1e11
    for row_bytes, low, high in ((384, 0.8, 0.9), (512, 0.8, 0.9), (3840, 0.7, 0.82)):
        c = bench.scattered_row_ceiling(row_bytes)
        assert c and low < c["GBps"] / bench.HBM_PEAK_GBS < high, row_bytes
    assert bench.scattered_row_ceiling(8192)["row_bytes"] == 4096      # beyond the table: its longest row
