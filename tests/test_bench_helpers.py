"""The host-side helpers of bench.py that turn profiler output into the figures it prints: counter CSVs ->
profiles/traffic.json (scaled by the calibration copy, one section per batch mode, stamped with the kernel
sources' hash), the rearrangements of the replay's id chunks, compulsory bytes, and the refusal of more than
one GPU.  No GPU needed."""
import csv
import importlib.util
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
bench = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(bench)


def _write_csv(path, counter, bag_values, copy_values):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value"])
        w.writeheader()
        for v in bag_values:
            w.writerow({"Kernel_Name": "void fwdmi::bag_reduce_kernel<_Float16, int, 8, 0, false>(BagLaunch)",
                        "Counter_Name": counter, "Counter_Value": v})
        for v in copy_values:
            w.writerow({"Kernel_Name": "__amd_rocclr_copyBuffer", "Counter_Name": counter, "Counter_Value": v})
        w.writerow({"Kernel_Name": "other_kernel", "Counter_Name": counter, "Counter_Value": 1e9})
        w.writerow({"Kernel_Name": "__amd_rocclr_copyBuffer", "Counter_Name": "OTHER", "Counter_Value": 5})


def test_record_traffic_scales_by_the_calibration_copy_and_keeps_one_section_per_mode(tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "TRAFFIC_JSON", str(tmp_path / "traffic.json"))
    f, w = str(tmp_path / "f.csv"), str(tmp_path / "w.csv")
    _write_csv(f, "FETCH_SIZE", [500000.0, 500002.0], [524300.0, 524304.0, 10.0])      # 64-byte units: scale 2
    _write_csv(w, "WRITE_SIZE", [400000.0, 400000.0], [1048576.0, 1048576.0, 4.0])     # scale 1; small copies are ignored
    bench.record_traffic(f, w, batches=8)
    t = json.load(open(bench.TRAFFIC_JSON))
    sec = t["rotating_batches"]
    assert sec["fetch_size_scale"] == 2.0 and sec["write_size_scale"] == 1.0 and sec["dispatches"] == [2, 2]
    assert sec["fetch_bytes"] == int(round(500001.0 * 2 * 1024)) and sec["write_bytes"] == 400000 * 1024
    assert sec["bytes_per_launch"] == sec["fetch_bytes"] + sec["write_bytes"]
    assert t["kernel_source_sha256"] == bench.kernel_source_hash() and "same_batch" not in t
    # the launch's L2 hit rate from a third counter pass goes into the same section
    h = str(tmp_path / "h.csv")
    with open(h, "w") as fh:
        fh.write("Kernel_Name,Counter_Name,Counter_Value\n")
        for name, vals in (("TCC_HIT_sum", [300.0, 500.0]), ("TCC_MISS_sum", [100.0, 100.0])):
            for v in vals:
                fh.write("fwdmi::bag_reduce_kernel<x>,%s,%s\n" % (name, v))
    bench.record_traffic(f, w, batches=8, l2_csv=h)
    assert json.load(open(bench.TRAFFIC_JSON))["rotating_batches"]["l2_hit_rate"] == 400.0 / 500.0
    bench.record_traffic(f, w, batches=1)                                                # the other mode joins it
    t = json.load(open(bench.TRAFFIC_JSON))
    assert set(t) >= {"rotating_batches", "same_batch"} and t["same_batch"]["batches"] == 1
    assert bench.load_traffic("same_batch")["bytes_per_launch"] == sec["bytes_per_launch"]
    # figures of another state of the kernel are not mixed with new ones, and are not used
    t["kernel_source_sha256"] = "0" * 64
    json.dump(t, open(bench.TRAFFIC_JSON, "w"))
    assert bench.load_traffic("rotating_batches") is None
    bench.record_traffic(f, w, batches=8)
    t = json.load(open(bench.TRAFFIC_JSON))
    assert "same_batch" not in t and t["kernel_source_sha256"] == bench.kernel_source_hash()


def test_committed_traffic_figures_belong_to_the_committed_kernel_sources():
    t = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert t["kernel_source_sha256"] == bench.kernel_source_hash(), \
        "profiles/traffic.json was measured on other kernel sources: collect the counters again (bench.py --record-traffic)"
    for sec in ("rotating_batches", "same_batch"):
        assert t[sec]["bytes_per_launch"] == t[sec]["fetch_bytes"] + t[sec]["write_bytes"]
        assert t[sec]["write_bytes"] == 26 * 65536 * 128 * 2 or abs(t[sec]["write_bytes"] - 26 * 65536 * 256) < 4096


def test_replay_chunk_orders_keep_every_chunks_ids():
    r = np.random.default_rng(1)
    ids = (r.zipf(1.2, 9000) % 700).astype(np.int32)
    for order in ("phased", "phased_unsorted", "bursts", "grouped"):
        out = bench.reorder_chunks(ids, 1830, order)
        for s0 in range(0, ids.size, 1830):
            assert np.array_equal(np.sort(out[s0:s0 + 1830]), np.sort(ids[s0:s0 + 1830])), order
    c = ids[:1830]
    _, inv, cnt = np.unique(c, return_inverse=True, return_counts=True)
    once = c[cnt[inv] == 1]
    # "phased": slot k of the workgroup reads elements k, k+16, ... of [once-only ids, repeated ids sorted]
    o = np.concatenate([once, np.sort(c[cnt[inv] > 1])])
    assert np.array_equal(bench.reorder_chunks(c, 1830, "phased"), np.concatenate([o[k::16] for k in range(16)]))


def test_compulsory_bytes_counts_distinct_rows_ids_offsets_and_output():
    from forward_amd import workloads
    wl = workloads.config4(n_tables=3, n_bags=200, max_rows=5000)
    b, unique_rows = bench.compulsory_bytes(wl)
    assert unique_rows == sum(np.unique(i).size for i in wl.indices)
    assert b == unique_rows * 128 * 2 + wl.n_indices() * 4 + 3 * 200 * 4 + 3 * 200 * 128 * 2
    fresh = workloads.config4_fresh_batch(wl, 2)
    assert fresh.rows == wl.rows and fresh.table_seeds == wl.table_seeds and fresh.n_bags == wl.n_bags
    assert not np.array_equal(fresh.indices[0][:50], wl.indices[0][:50])
    assert workloads.config4_fresh_batch(wl, 0) is wl


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 2 and "one GPU" in p.stderr
