#!/usr/bin/env python3
"""Benchmark of the embedding-side hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K (200)] [--warmup W (20)] [--prewarm P (300)] [--batches B (8)]
                  [--workload config4] [--no-cpu] [--no-extra]

A step is one pass of the DLRM-style sparse stage (BASELINE config 4): 26 sum-mode tables, fp16
rows of dim 128, 65536 bags per table with truncated-Zipf lengths, Zipf ids, fp16 output
concatenated to [65536, 3328], issued as ONE fused launch.  Inputs are resident in HBM before the
timed region; the steps cycle through B batches of fresh ids and bag lengths over the same tables
(a serving loop never sees the same ids twice), the same-batch figure is reported beside it.
Prints one JSON line: bags/s over the whole job, the roofline block of the kernel from HIP-event
timing of the same launches (frac = algorithmic bytes / kernel time / HBM peak, which exceeds 1
when caches serve most rows; frac_hbm_side = bytes counted beyond L2 / kernel time / HBM peak), and a
CPU baseline: libtorch CPU (the path the reference's unit tests compare against) at all host
threads this process may use, with the C oracle port beside it.

  python bench.py --record-traffic FETCH_CSV WRITE_CSV [--batches B]
      (no GPU) turns two rocprofv3 --pmc counter_collection CSVs of
      `bench.py --steps 16 --warmup 0 --prewarm 0 --batches B --no-cpu --no-extra --copy-calibration`
      (FETCH_SIZE in one run, WRITE_SIZE in the other) into profiles/traffic.json (section
      "rotating_batches" for B > 1, "same_batch" for B = 1), stamped with the hash of the kernel
      sources they were measured on.
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0
MI355X_PEAK_CLOCK_HZ = 2.4e9    # published peak engine clock
ROOT = os.path.dirname(os.path.abspath(__file__))
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
# the sources the 26-table kernel is compiled from: counter figures belong to one state of them
KERNEL_SOURCES = ("forward_amd/csrc/kernels/embedding_bag.hip", "forward_amd/csrc/kernels/bag_plan.h",
                  "forward_amd/csrc/kernels/bag_plan.cpp", "forward_amd/csrc/kernels/device_util.h")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--prewarm", type=int, default=300,
                    help="untimed launches before the warm-up steps, so that a short run (--steps 20 --warmup 5) is "
                         "timed at the steady engine clock like a long one; reported as prewarm_launches")
    ap.add_argument("--batches", type=int, default=8,
                    help="batches of fresh ids / bag lengths (same tables) the steps cycle through; 1 = every step "
                         "replays the same batch")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU: write profiles/traffic.json from two rocprofv3 --pmc counter_collection CSVs")
    ap.add_argument("--record-l2", metavar="HIT_MISS_CSV",
                    help="with --record-traffic: also the L2 hit rate of the launch, from a rocprofv3 --pmc TCC_HIT_sum "
                         "TCC_MISS_sum counter_collection CSV of the same batch mode")
    ap.add_argument("--workload", default="config4", choices=["config4"])
    ap.add_argument("--tables", type=int, default=26, help="debug only: fewer tables (not the named config)")
    ap.add_argument("--bags", type=int, default=65536, help="debug only: smaller batch (not the named config)")
    ap.add_argument("--per-table", action="store_true", help="26 launches instead of the fused one")
    ap.add_argument("--no-xcd-affinity", action="store_true",
                    help="fused launch without per-XCD table affinity (every XCD works on every table)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    ap.add_argument("--no-extra", action="store_true", help="skip the config 2/3/5 side measurements")
    ap.add_argument("--cpu-bags", type=int, default=65536,
                    help="bags per table in the CPU baseline sample (default: the whole batch)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (known traffic, to scale rocprof byte counters)")
    ap.add_argument("--replay", action="store_true",
                    help="instead of the benchmark: the workload's row-id stream replayed as a plain gather (no "
                         "bags), without and with result stores, beside the product launch (a table on stdout)")
    ap.add_argument("--ids", default="zipf", choices=["zipf", "equal", "uniform"],
                    help="--replay only: keep the workload's ids, or replace them (lengths kept) by one row per "
                         "table / by uniform random rows")
    ap.add_argument("--order", default="stream", choices=["stream", "phased", "phased_unsorted", "bursts", "grouped"],
                    help="--replay only: the order of the ids inside every workgroup's chunk: as they come; the ids "
                         "that occur once in the chunk first and the repeated ones after them, all slots in the same "
                         "phase at the same time (likely misses apart from likely hits; phased_unsorted: the repeated "
                         "ones in their original order, phased: sorted by row); bursts: no phases, but the repeated "
                         "ids sorted among themselves, so that equal rows are fetched together; or all sorted by row")
    ap.add_argument("--hot", type=int, default=0, metavar="K",
                    help="--replay only: also replay with the K (at most 64) most frequent rows of every table served "
                         "from LDS instead of through the L1 (the split of every chunk done on the host: an upper bound)")
    ap.add_argument("--lru-sim", action="store_true",
                    help="no GPU: rows fetched by an LRU cache of one XCD's L2 size over each table's id stream "
                         "(the floor of the re-fetch ratio for table-at-a-time processing)")
    ap.add_argument("--hbm-gather", action="store_true",
                    help="instead of the benchmark: uniform random ids over one 4 GiB fp16 table of dim 128 (far beyond "
                         "every cache), the gather rate that is HBM and nothing else (one JSON line on stdout)")
    ap.add_argument("--sweep", action="store_true",
                    help="instead of the benchmark: single-table bag reduction over row widths, table types and "
                         "bag lengths with uniform random ids beside torch's GPU embedding_bag, then SkipLayerNorm "
                         "over row lengths and counts beside torch's add + layer_norm (two tables on stdout)")
    return ap.parse_args()


def host_threads():
    """CPU threads this process may use for the CPU baseline, and where the figure comes from.

    The scheduler affinity mask bounds it; a box that hands a job a share of a larger host says so
    through OMP_NUM_THREADS (libtorch's own default thread count follows the same variable)."""
    info = {"os_cpu_count": os.cpu_count() or 1}
    try:
        info["sched_affinity"] = len(os.sched_getaffinity(0))
    except AttributeError:
        info["sched_affinity"] = info["os_cpu_count"]
    env = os.environ.get("OMP_NUM_THREADS", "")
    info["omp_num_threads_env"] = int(env) if env.isdigit() and int(env) > 0 else None
    info["threads_used"] = min([info["sched_affinity"]] + ([info["omp_num_threads_env"]] if info["omp_num_threads_env"] else []))
    return info


def kernel_source_hash():
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def load_traffic(section):
    """HBM-side bytes per launch of the default workload from profiles/traffic.json (`section`:
    "rotating_batches" or "same_batch"), or None (with a warning) when the file or the section is
    absent or was measured on other kernel sources than the tree holds."""
    if not os.path.exists(TRAFFIC_JSON):
        log("warning: %s is absent: roofline.traffic is null" % TRAFFIC_JSON)
        return None
    with open(TRAFFIC_JSON) as f:
        t = json.load(f)
    if t.get("kernel_source_sha256") != kernel_source_hash():
        log("warning: profiles/traffic.json was measured on other kernel sources (hash %s, tree %s): "
            "roofline.traffic is null until the counters are collected again (bench.py --record-traffic)"
            % (str(t.get("kernel_source_sha256"))[:12], kernel_source_hash()[:12]))
        return None
    if section not in t:
        log("warning: profiles/traffic.json has no %s section: roofline.traffic is null" % section)
        return None
    return dict(t[section], kernel_source_sha256=t["kernel_source_sha256"])


def record_traffic(fetch_csv, write_csv, batches, l2_csv=None):
    """profiles/traffic.json from two rocprofv3 counter CSVs (FETCH_SIZE / WRITE_SIZE, KiB per
    dispatch).  Each counter is scaled by what it reads for the 1 GiB device copy of the same run
    (--copy-calibration: 1 048 576 KiB read and as many written).  The counters sit at the L2's
    far side (requests from L2 to the fabric): bytes the memory-side cache serves are counted like
    bytes from DRAM."""
    import csv

    def per_kernel(path, counter):
        bag, cal = [], []
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != counter:
                    continue
                v = float(r["Counter_Value"])
                if "bag_reduce_kernel" in r["Kernel_Name"]:
                    bag.append(v)
                elif "copyBuffer" in r["Kernel_Name"]:   # the runtime's device-to-device copy kernel
                    cal.append(v)
        if not bag:
            raise SystemExit("%s holds no %s rows of bag_reduce_kernel" % (path, counter))
        # the calibration copies are the largest dispatches of their kind: keep those near the maximum
        cal = [v for v in cal if v > 0.9 * max(cal)] if cal else []
        return float(np.mean(bag)), (float(np.mean(cal)) if cal else None), len(bag)

    fetch, fetch_cal, nf = per_kernel(fetch_csv, "FETCH_SIZE")
    write, write_cal, nw = per_kernel(write_csv, "WRITE_SIZE")
    kib = float(1 << 20)
    fs = kib / fetch_cal if fetch_cal else 2.0
    ws = kib / write_cal if write_cal else 1.0
    # the counters come in two granularities (32- and 64-byte units): snap the measured factor
    fs, ws = (min((1.0, 2.0, 4.0), key=lambda c: abs(c - x)) for x in (fs, ws))
    sec = {
        "batches": batches,
        "fetch_size_kib_raw": fetch, "write_size_kib_raw": write, "dispatches": [nf, nw],
        "fetch_size_copy_kib_raw": fetch_cal, "write_size_copy_kib_raw": write_cal,
        "fetch_size_scale": fs, "write_size_scale": ws,
        "fetch_bytes": int(round(fetch * fs * 1024)), "write_bytes": int(round(write * ws * 1024)),
    }
    sec["bytes_per_launch"] = sec["fetch_bytes"] + sec["write_bytes"]
    if l2_csv:
        hit, _, nh = per_kernel(l2_csv, "TCC_HIT_sum")
        miss, _, _ = per_kernel(l2_csv, "TCC_MISS_sum")
        sec["l2_hits"], sec["l2_misses"], sec["l2_hit_rate"] = hit, miss, hit / (hit + miss)
        sec["dispatches"].append(nh)
    out = {}
    if os.path.exists(TRAFFIC_JSON):
        with open(TRAFFIC_JSON) as f:
            out = json.load(f)
        if out.get("kernel_source_sha256") != kernel_source_hash():
            out = {}           # figures of another state of the kernel: nothing of them is kept
    out["_comment"] = ("bytes per launch of bench.py's default workload beyond L2 (requests from L2 to the fabric: "
                       "memory-side-cache hits count like DRAM reads) from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE "
                       "(KiB per dispatch), each scaled by what the counter reads for a 1 GiB device copy of the same "
                       "run; rotating_batches: the steps cycle through fresh id batches, same_batch: every step "
                       "replays one batch; written by bench.py --record-traffic")
    out["kernel_source_sha256"] = kernel_source_hash()
    out["kernel_source_files"] = list(KERNEL_SOURCES)
    out["rotating_batches" if batches > 1 else "same_batch"] = sec
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print(json.dumps(out, indent=1))


def compulsory_bytes(wl, table_itemsize=2, out_itemsize=2, index_itemsize=4):
    """Bytes a launch cannot avoid moving to or from HBM: every DISTINCT row once, the ids and
    offsets once, the output once."""
    unique_rows = int(sum(np.unique(i).size for i in wl.indices))
    t = len(wl.rows)
    b = (unique_rows * wl.dim * table_itemsize + wl.n_indices() * index_itemsize +
         t * wl.n_bags * index_itemsize + t * wl.n_bags * wl.dim * out_itemsize)
    return b, unique_rows


def device_tables(wl, torch):
    """fp16 rows ~U(-0.05, 0.05) generated in HBM (seeded per table)."""
    return [wl.device_table(t, torch) for t in range(len(wl.rows))]


def time_events(torch, fn, steps, warmup):
    """Wall-clock over `steps` back-to-back calls plus per-call HIP-event durations (ms)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = np.array([a.elapsed_time(b) for a, b in evs])
    return wall, per


def time_graph(torch, fn, inner=20, reps=15):
    """GPU time per call of a launch-bound kernel: `inner` calls captured into one HIP graph
    (no host work between them), replayed `reps` times between HIP events; median / inner (ms)."""
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(inner):
            fn()
    g.replay()
    torch.cuda.synchronize()
    per = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        per.append(a.elapsed_time(b) / inner)
    return float(np.median(per))


def cpu_baseline(wl, tabs_dev, n_cpu_bags, torch):
    """libtorch CPU (26 x F.embedding_bag + cat: the path the reference's unit tests take as ground
    truth, source/unit_test/unit_test_torch_helper.h:82-87) at all threads this process may use and
    at one thread, and the C oracle port, on the first `n_cpu_bags` bags of every table."""
    from oracle import oracle          # checker, used here only as a timed CPU baseline
    oracle.build()
    threads = host_threads()
    cores = threads["threads_used"]
    oracle.set_threads(cores)
    nb = min(n_cpu_bags, wl.n_bags)
    host_tabs, idxs, offs = [], [], []
    for t in range(len(wl.rows)):
        end = int(wl.offsets[t][nb]) if nb < wl.n_bags else wl.indices[t].size
        host_tabs.append(tabs_dev[t].cpu().numpy())
        idxs.append(np.ascontiguousarray(wl.indices[t][:end]))
        offs.append(np.ascontiguousarray(wl.offsets[t][:nb]))
    total_bags = nb * len(wl.rows)
    out = np.zeros((nb, len(wl.rows) * wl.dim), np.float16)

    def run_oracle():
        for t in range(len(wl.rows)):
            oracle.embedding_bag(host_tabs[t], idxs[t], offs[t], oracle.OP_SUM, out=out, out_col=t * wl.dim)

    def timed(fn, budget_s=8.0, min_reps=2):
        fn()
        reps, t0 = 0, time.perf_counter()
        while True:
            fn()
            reps += 1
            dt = time.perf_counter() - t0
            if reps >= min_reps and dt > budget_s or reps >= 20:
                return dt / reps

    tt = [torch.from_numpy(a) for a in host_tabs]
    ti = [torch.from_numpy(a) for a in idxs]
    to = [torch.from_numpy(a) for a in offs]

    def run_torch():
        return torch.cat([torch.nn.functional.embedding_bag(ti[t], tt[t], to[t], mode="sum")
                          for t in range(len(tt))], dim=1)

    lt = {}
    for n in sorted({cores, 1}, reverse=True):
        torch.set_num_threads(n)
        lt["threads_%d" % n] = total_bags / timed(run_torch, budget_s=6.0)
    torch.set_num_threads(cores)
    lt_out = run_torch().numpy()
    res = {"value": lt["threads_%d" % cores], "unit": "bags/s", "cores": cores, "kind": "libtorch_cpu",
           "what": "26 x torch.nn.functional.embedding_bag(mode='sum') + torch.cat on CPU tensors (fp16 tables, "
                   "int32 ids): the ground truth of the reference's unit tests",
           "sample": "all %d tables x first %d of %d bags per table, same ids/offsets as the GPU launch" %
                     (len(wl.rows), nb, wl.n_bags),
           "host_threads": threads, "libtorch_cpu_bags_per_s": lt, "torch_version": torch.__version__}
    res["port_c_oracle_bags_per_s"] = total_bags / timed(run_oracle, budget_s=6.0)
    res["port_c_oracle_threads"] = cores
    try:
        with open("/proc/cpuinfo") as f:
            res["cpu_model"] = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except Exception:
        pass
    log("cpu baseline: os.cpu_count()=%d, sched affinity=%d, OMP_NUM_THREADS=%s, threads used=%d" %
        (threads["os_cpu_count"], threads["sched_affinity"], threads["omp_num_threads_env"], cores))
    # the oracle's output doubles as a check of the whole GPU result; libtorch's own result goes with it
    return res, out, nb, lt_out


def compare_with_libtorch(got, want, what="the whole fp16 result against libtorch's fp16 result, element by element",
                          fp32=False):
    """A GPU launch's fp16 result against libtorch CPU's on the same inputs (the ground truth the reference's
    unit tests use), at the stated bar: fp16 after fp32 accumulation abs 1e-2 / rel 5e-3, fp32 rel 1e-5 (with the
    same figure as absolute floor for sums that cancel)."""
    g, w = got.astype(np.float32), want.astype(np.float32)
    diff = np.abs(g - w)
    return {"elements": int(g.size), "max_abs_diff": float(diff.max()), "differing_elements": int((diff > 0).sum()),
            ("within_rel_1e-5" if fp32 else "within_abs_1e-2_rel_5e-3"):
                bool((diff <= (1e-5 + 1e-5 * np.abs(w) if fp32 else 1e-2 + 5e-3 * np.abs(w))).all()),
            "what": what}


def copy_bandwidth(torch):
    """Device-to-device copy of 1 GiB (read + write), GB/s: what a streaming kernel gets on this box."""
    src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
    dst = torch.empty_like(src)
    _, per = time_events(torch, lambda: dst.copy_(src), 10, 3)
    return 2 * src.numel() * 4 / (float(np.median(per)) * 1e-3) / 1e9


def cpu_bert(torch, wl, threads):
    """libtorch CPU tokens/s of embedding x3 + add + layer_norm (+ residual/bias add + layer_norm)."""
    tw, tp, tt = (torch.from_numpy(a) for a in (wl.word, wl.pos, wl.tok))
    ids, seg = torch.from_numpy(wl.input_ids).long(), torch.from_numpy(wl.segment_ids).long()
    g, b = torch.from_numpy(wl.gamma), torch.from_numpy(wl.beta)
    S, H = wl.input_ids.shape[0], wl.word.shape[1]
    F = torch.nn.functional
    sk = None if wl.skip is None else [torch.from_numpy(a) for a in (wl.skip, wl.skip_bias, wl.skip_gamma, wl.skip_beta)]

    def run():
        e = F.layer_norm(F.embedding(ids, tw) + tp[:S].unsqueeze(1) + F.embedding(seg, tt), (H,), g, b, wl.eps)
        if sk is not None:
            e = F.layer_norm(e + sk[0] + sk[1], (H,), sk[2], sk[3], wl.eps)
        return e

    res = {}
    for n in threads:
        torch.set_num_threads(n)
        for _ in range(3):
            run()
        ts = []
        for _ in range(10):
            t0 = time.perf_counter()
            run()
            ts.append(time.perf_counter() - t0)
        res["threads_%d" % n] = wl.n_tokens / float(np.median(ts))
    torch.set_num_threads(threads[0])
    return res, run().numpy()


def bert_libtorch_fp32(torch, wl):
    """The same stage through libtorch CPU in fp32 on the workload's fp16 parameters (embedding x3 + add +
    layer_norm, then the residual / bias add + layer_norm where the workload has one): what the GPU result
    is compared with.  Returns (first stage, final stage or None)."""
    F = torch.nn.functional
    tw, tp, tt = (torch.from_numpy(a).float() for a in (wl.word, wl.pos, wl.tok))
    ids, seg = torch.from_numpy(wl.input_ids).long(), torch.from_numpy(wl.segment_ids).long()
    S, H = wl.input_ids.shape[0], wl.word.shape[1]
    g, b = torch.from_numpy(wl.gamma).float(), torch.from_numpy(wl.beta).float()
    e = F.layer_norm(F.embedding(ids, tw) + tp[:S].unsqueeze(1) + F.embedding(seg, tt), (H,), g, b, wl.eps)
    if wl.skip is None:
        return e.numpy(), None
    sk, bi, g2, b2 = (torch.from_numpy(a).float() for a in (wl.skip, wl.skip_bias, wl.skip_gamma, wl.skip_beta))
    return e.numpy(), F.layer_norm(e + sk + bi, (H,), g2, b2, wl.eps).numpy()


def plugin_level(torch, wl, tabs, idx, off, want):
    """The same stage issued the way the reference's graph issues it
    (layer_creators/trt_embedding_bag_creator.h:70-75): plugin objects created from creator fields,
    configured, then enqueued.  One EmbeddingBagGroup_TRT enqueue (all tables, one launch) and 26
    EmbeddingBag_TRT "002" enqueues (one per table, as the reference does), each timed as a HIP-graph
    replay and compared bit for bit with the fused C-ABI launch's output `want`.  The tables reach
    the plugins by file reference (creator field data_file), the same bytes the C-ABI launch reads."""
    import tempfile
    from forward_amd import lib, plugin
    from forward_amd.plugin import PluginFieldData as F
    res = {}
    need = sum(t.numel() * t.element_size() for t in tabs)
    shm = "/dev/shm" if os.path.isdir("/dev/shm") and os.access("/dev/shm", os.W_OK) else None
    if shm is not None:
        st = os.statvfs(shm)
        if st.f_bavail * st.f_frsize < need + (1 << 30):
            shm = None                     # too small for the tables: the default temporary directory then
    fd, path = tempfile.mkstemp(prefix="fwdmi_tables_", suffix=".bin", dir=shm)
    plugins = []
    try:
        t0 = time.time()
        row0 = [0]
        with os.fdopen(fd, "wb") as f:
            for t in tabs:
                f.write(t.cpu().numpy().tobytes())
                row0.append(row0[-1] + t.shape[0])
        path_field = F("data_file", np.frombuffer(path.encode(), np.int8), lib.FIELD_CHAR)
        reg = plugin.getPluginRegistry()
        n_bags, dim, T = wl.n_bags, wl.dim, len(tabs)
        ins = [x for pair in zip(idx, off) for x in pair]
        group = reg.getPluginCreator("EmbeddingBagGroup_TRT", "001").createPlugin("sparse", [
            F("dim", dim), F("op", 0), F("count", np.array(wl.rows, np.int32)), path_field,
            F("table_type", lib.F16), F("output_fp16", 1)])
        plugins.append(group)
        got = torch.zeros_like(want)
        group.configurePlugin([(tuple(t.shape), lib.I32) for t in ins], [((n_bags, T * dim), lib.F16)])
        group.enqueue(ins, [got])
        torch.cuda.synchronize()
        res["group_plugin_setup_s"] = time.time() - t0
        ms = time_graph(torch, lambda: group.enqueue(ins, [got]), inner=20, reps=7)
        res["group_plugin_one_enqueue"] = {
            "ms": ms, "bags_per_s": n_bags * T / (ms * 1e-3),
            "bit_identical_to_c_abi_launch": bool(torch.equal(got.view(torch.int16), want.view(torch.int16))),
            "what": "EmbeddingBagGroup_TRT/001: one enqueue = one fused launch, the call's table descriptors among its "
                    "kernel arguments; 20 enqueues per replayed HIP graph"}
        group.destroy()
        del got
        single = reg.getPluginCreator("EmbeddingBag_TRT", "002")
        outs = []
        for t in range(T):
            p = single.createPlugin("bag%d" % t, [
                F("dim", dim), F("count", wl.rows[t]), F("offset", 0), F("op", 0), path_field,
                F("table_type", lib.F16), F("data_file_row_offset", row0[t]), F("output_fp16", 1)])
            plugins.append(p)
            o = torch.zeros((n_bags, dim), dtype=torch.float16, device="cuda")
            p.configurePlugin([(tuple(idx[t].shape), lib.I32), (tuple(off[t].shape), lib.I32)], [((n_bags, dim), lib.F16)])
            outs.append(o)

        def per_table():
            for t in range(T):
                plugins[1 + t].enqueue([idx[t], off[t]], [outs[t]])
        per_table()
        torch.cuda.synchronize()
        same = all(bool(torch.equal(outs[t].view(torch.int16), want[:, t * dim:(t + 1) * dim].view(torch.int16)))
                   for t in range(T))
        ms = time_graph(torch, per_table, inner=3, reps=11)
        res["per_table_plugins_26_enqueues"] = {
            "ms": ms, "bags_per_s": n_bags * T / (ms * 1e-3), "bit_identical_to_c_abi_launch": same,
            "what": "26 x EmbeddingBag_TRT/002 enqueue, one [65536, 128] output each (no concatenation pass)"}
    finally:
        for p in plugins:
            p.destroy()
        os.remove(path)
    return res


def microbench_dll():
    """bench_aux/libfwdmi_microbench.so (the measurement aids), or None when it is not built."""
    import ctypes as C
    path = os.path.join(ROOT, "bench_aux", "libfwdmi_microbench.so")
    return C.CDLL(path) if os.path.exists(path) else None


def launch_floor_ms(torch, grid=1024, block=256):
    """GPU time per launch of a kernel that does nothing, with the grid of the short launches (1024
    workgroups of 256 lanes: four per CU), timed like them: 20 launches per replayed HIP graph."""
    import ctypes as C
    dll = microbench_dll()
    if dll is None:
        return None
    stream = lambda: C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def fn():
        rc = dll.fwdmi_mb_empty_launch(grid, block, stream())
        if rc:
            raise RuntimeError("empty launch failed: hipError %d" % rc)
    return time_graph(torch, fn)


def hbm_gather(torch, ops, copy_gbs=None, rows=1 << 24, dim=128, n_bags=262144, bag_len=32, steps=20):
    """The gather rate that is HBM and nothing else: uniform random int32 ids over one fp16 table of
    2^24 rows x 128 (4 GiB: sixteen times the memory-side cache, 128 times all L2s), 262144 bags of
    32 ids (8.4 M rows = 2.1 GB of row bytes per launch, 1.7 GB of them distinct), two id sets in
    turn.  Algorithmic bytes as in the benchmark."""
    r = np.random.Generator(np.random.PCG64(77))
    table = torch.empty((rows, dim), dtype=torch.float16, device="cuda")
    for c0 in range(0, rows, 1 << 21):          # filled in slices: no fp32 copy of the whole table
        table[c0:c0 + (1 << 21)] = (torch.rand((min(1 << 21, rows - c0), dim), device="cuda") - 0.5) * 0.1
    sets = []
    for _ in range(2):
        ids = torch.from_numpy(r.integers(0, rows, n_bags * bag_len, dtype=np.int64).astype(np.int32)).cuda()
        sets.append(ids)
    off = torch.arange(0, n_bags * bag_len, bag_len, dtype=torch.int32, device="cuda")
    out = torch.empty((n_bags, dim), dtype=torch.float16, device="cuda")
    n = [0]

    def fn():
        ops.embedding_bag(table, sets[n[0] & 1], off, "sum", out=out)
        n[0] += 1
    _, per = time_events(torch, fn, steps, 5)
    ms = float(np.mean(per))
    # the same table read front to back by a kernel that does nothing else: what contiguous reads get from HBM here
    read_gbs = None
    dll = microbench_dll()
    if dll is not None:
        import ctypes as C
        dll.fwdmi_mb_stream_read.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        nbytes_tab = table.numel() * 2
        grid = torch.cuda.get_device_properties(0).multi_processor_count * 8

        def rd():
            rc = dll.fwdmi_mb_stream_read(table.data_ptr(), nbytes_tab, grid, torch.cuda.current_stream().cuda_stream)
            if rc:
                raise RuntimeError("stream read failed: hipError %d" % rc)
        _, per_r = time_events(torch, rd, 10, 3)
        read_gbs = nbytes_tab / (float(np.mean(per_r)) * 1e-3) / 1e9
    nbytes = n_bags * bag_len * (dim * 2 + 4) + n_bags * 4 + n_bags * dim * 2
    res = {"what": "uniform random ids over a 4 GiB fp16 table (2^24 rows x 128): %d bags x %d ids per launch, sum"
                   % (n_bags, bag_len),
           "ms": ms, "algorithmic_bytes": nbytes, "algorithmic_GBs": nbytes / (ms * 1e-3) / 1e9,
           "frac_of_hbm_peak": nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "rows_per_s": n_bags * bag_len / (ms * 1e-3)}
    if copy_gbs:
        res["device_copy_GBs"] = copy_gbs
        res["over_device_copy_rate"] = res["algorithmic_GBs"] / copy_gbs
    if read_gbs:
        res["contiguous_read_GBs"] = read_gbs
        res["contiguous_read_is"] = "the same 4 GiB table read front to back with 128-bit loads by a kernel that does nothing else"
        res["over_contiguous_read_rate"] = res["algorithmic_GBs"] / read_gbs
    return res


def extra_measurements(torch, ops, workloads, steps, with_cpu=True):
    """Tokens/s of the BERT configs and bags/s of config 2.  These launches take ~10 us, less than
    a Python launch costs, so they are timed as HIP-graph replays (GPU time, launch gaps included)."""
    ex = {}
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    f32 = lambda a: dev(np.asarray(a, np.float32))
    for name, wl in (("config3_emb_layer_norm", workloads.config3()), ("config5_emb_layer_norm", workloads.config5())):
        a = [dev(wl.input_ids), dev(wl.segment_ids), dev(wl.input_mask), dev(wl.word), dev(wl.pos), dev(wl.tok),
             f32(wl.gamma), f32(wl.beta)]
        out = torch.empty((wl.input_ids.shape[0], wl.input_ids.shape[1], wl.word.shape[1]), dtype=torch.float16,
                          device="cuda")
        midx = torch.empty((wl.input_ids.shape[1],), dtype=torch.int32, device="cuda")
        fn = lambda: ops.emb_layer_norm(*a, eps=wl.eps, out=out, mask_idx=midx)
        ms = time_graph(torch, fn)
        ex[name] = {"tokens_per_s": wl.n_tokens / (ms * 1e-3), "ms": ms,
                    "algorithmic_GBs": wl.emb_algorithmic_bytes() / (ms * 1e-3) / 1e9}
        if with_cpu:
            cores = host_threads()["threads_used"]
            ex[name.split("_")[0] + "_libtorch_cpu_tokens_per_s"], native = cpu_bert(
                torch, wl, tuple(sorted({cores, 1}, reverse=True)))
            ref1, ref2 = bert_libtorch_fp32(torch, wl)
            if wl.skip is None:   # (with a second stage, libtorch's fp16 result is that stage's: compared there)
                ex[name]["gpu_vs_libtorch_cpu_native_fp16"] = compare_with_libtorch(
                    out.cpu().numpy(), native, "against libtorch's fp16 path, which rounds after every operation")
            ex[name]["gpu_vs_libtorch_cpu_fp32"] = compare_with_libtorch(
                out.cpu().numpy(), ref1, "the whole fp16 result against libtorch's fp32 evaluation of the same fp16 parameters")
        if wl.skip is not None:
            x, sk = out, dev(wl.skip)
            g, b, bi = f32(wl.skip_gamma), f32(wl.skip_beta), f32(wl.skip_bias)
            o2 = torch.empty_like(x)
            fn2 = lambda: ops.skip_layer_norm(x, g, b, skip=sk, bias=bi, eps=wl.eps, out=o2)
            ms = time_graph(torch, fn2)
            ex["config5_skip_layer_norm"] = {"tokens_per_s": wl.n_tokens / (ms * 1e-3), "ms": ms,
                                             "algorithmic_GBs": wl.skip_algorithmic_bytes() / (ms * 1e-3) / 1e9}
            if with_cpu:   # the chain EmbLayerNorm -> SkipLayerNorm against libtorch's, fp32 and its own fp16 path
                ex["config5_skip_layer_norm"]["gpu_vs_libtorch_cpu_native_fp16"] = compare_with_libtorch(
                    o2.cpu().numpy(), native, "against libtorch's fp16 path, which rounds after every operation")
                ex["config5_skip_layer_norm"]["gpu_vs_libtorch_cpu_fp32"] = compare_with_libtorch(
                    o2.cpu().numpy(), ref2, "the whole fp16 result of the two-stage chain against libtorch's fp32 evaluation")
            # yardsticks: torch's add on the same tensors (the same traffic, no reduction) and
            # PyTorch-ROCm's own GPU kernels for the same stage (add + bias, then layer_norm)
            ms_add = time_graph(torch, lambda: torch.add(x, sk, out=o2))
            ex["config5_same_traffic_torch_add"] = {"ms": ms_add,
                                                    "GBs": wl.skip_algorithmic_bytes() / (ms_add * 1e-3) / 1e9}
            g16, b16, bi16 = g.half(), b.half(), bi.half()
            H = x.shape[-1]
            try:
                ms_t = time_graph(torch, lambda: torch.nn.functional.layer_norm(x + sk + bi16, (H,), g16, b16, wl.eps))
                ex["config5_skip_layer_norm_pytorch_rocm_gpu"] = {"ms": ms_t,
                                                                  "tokens_per_s": wl.n_tokens / (ms_t * 1e-3)}
            except Exception as e:  # noqa: BLE001  (a yardstick must not fail the measurement)
                ex["config5_skip_layer_norm_pytorch_rocm_gpu"] = {"error": repr(e)}
            # the same two stages in one pass (no intermediate round trip through HBM)
            fn3 = lambda: ops.emb_layer_norm(*a, eps=wl.eps, out=o2, mask_idx=midx, skip=sk, gamma2=g, beta2=b,
                                             bias2=bi, eps2=wl.eps)
            ms = time_graph(torch, fn3)
            h2 = wl.n_tokens * wl.word.shape[1] * wl.word.itemsize
            ex["config5_fused_emb_skip_layer_norm"] = {
                "tokens_per_s": wl.n_tokens / (ms * 1e-3), "ms": ms,
                "algorithmic_GBs": (wl.emb_algorithmic_bytes() + wl.skip_algorithmic_bytes() - 2 * h2) / (ms * 1e-3) / 1e9}
    # config 1 (64 bags, the reference's own unit-test shape): one launch's fixed cost, no roofline
    wl = workloads.config1()
    tb, ix, of = dev(wl.table), dev(wl.indices), dev(wl.offsets)
    out = torch.empty((wl.n_bags, wl.table.shape[1]), dtype=tb.dtype, device="cuda")
    ms = time_graph(torch, lambda: ops.embedding_bag(tb, ix, of, "sum", out=out))
    ex["config1_sum_fp32_int64"] = {"bags_per_s": wl.n_bags / (ms * 1e-3), "ms": ms}
    cpu_bag = lambda w: torch.nn.functional.embedding_bag(torch.from_numpy(w.indices).long(), torch.from_numpy(w.table),
                                                          torch.from_numpy(w.offsets).long(), mode="sum").numpy()
    if with_cpu:
        ex["config1_sum_fp32_int64"]["gpu_vs_libtorch_cpu"] = compare_with_libtorch(
            out.cpu().numpy(), cpu_bag(wl), "the whole fp32 result against libtorch's, element by element", fp32=True)
    for tdt, tname in ((np.float32, "fp32"), (np.float16, "fp16")):
        wl = workloads.config2(table_dtype=tdt)
        tb, ix, of = dev(wl.table), dev(wl.indices), dev(wl.offsets)
        out = torch.empty((wl.n_bags, 128), dtype=tb.dtype, device="cuda")
        fn = lambda: ops.embedding_bag(tb, ix, of, "sum", out=out)
        ms = time_graph(torch, fn)
        ex["config2_sum_%s_int32" % tname] = {"bags_per_s": wl.n_bags / (ms * 1e-3), "ms": ms,
                                              "algorithmic_GBs": wl.algorithmic_bytes() / (ms * 1e-3) / 1e9}
        if with_cpu:
            ex["config2_sum_%s_int32" % tname]["gpu_vs_libtorch_cpu"] = compare_with_libtorch(
                out.cpu().numpy(), cpu_bag(wl), "the whole %s result against libtorch's, element by element" % tname,
                fp32=tdt == np.float32)
        ix64, of64 = ix.long(), of.long()
        try:
            ms_t = time_graph(torch, lambda: torch.nn.functional.embedding_bag(ix64, tb, of64, mode="sum"))
            ex["config2_sum_%s_pytorch_rocm_gpu" % tname] = {"bags_per_s": wl.n_bags / (ms_t * 1e-3), "ms": ms_t}
        except Exception as e:  # noqa: BLE001
            ex["config2_sum_%s_pytorch_rocm_gpu" % tname] = {"error": repr(e)}
    # these kernels move their algorithmic bytes once (rocprofv3 FETCH_SIZE / WRITE_SIZE agree, see
    # profiles/): the algorithmic rate over the HBM peak is their roofline position.  They are short:
    # beside it, the same figure with the time of a launch that does nothing taken off.
    floor = launch_floor_ms(torch)
    for k, v in ex.items():
        if isinstance(v, dict) and "algorithmic_GBs" in v:
            v["frac_of_hbm_peak"] = v["algorithmic_GBs"] / HBM_PEAK_GBS
        if floor is not None and isinstance(v, dict) and "ms" in v and "pytorch" not in k and "torch_add" not in k:
            v["ms_above_launch_floor"] = v["ms"] - floor
            if "algorithmic_GBs" in v and v["ms"] > floor:
                v["frac_of_hbm_peak_above_launch_floor"] = v["frac_of_hbm_peak"] * v["ms"] / (v["ms"] - floor)
    if floor is not None:
        ex["launch_floor_us"] = floor * 1e3
        ex["launch_floor_is"] = ("GPU time per launch of a kernel that does nothing (1024 workgroups x 256 lanes), 20 "
                                 "launches per replayed HIP graph like the figures above")
    return ex


def sweep(torch, ops):
    """Regime table of the single-table launcher: 65536 fixed-length bags (8192 for the widest
    cases) of uniform random int32 ids over a table of up to 1 M rows / 1 GiB; algorithmic bytes
    per launch as in the benchmark; every case beside torch.nn.functional.embedding_bag on the
    same GPU, both timed as 10 launches captured in one HIP graph."""
    import torch.nn.functional as F
    r = np.random.Generator(np.random.PCG64(5))
    print("%5s %5s %4s %6s | %9s %9s | %9s | %s" % ("dim", "type", "L", "mode", "ms", "GB/s", "torch ms", "speedup"),
          flush=True)
    for tdt in (torch.float16, torch.float32):
        for dim in (8, 16, 32, 64, 128, 256, 512, 1024):
            rows = min(1_000_000, (1 << 30) // (dim * 4))
            table = (torch.randn((rows, dim), device="cuda") * 0.1).to(tdt)
            sz = table.element_size()
            for bag_len in (1, 4, 16, 64):
                nb = 65536 if dim * bag_len <= 128 * 64 else 8192
                for mode in ("sum", "max") if bag_len == 16 else ("sum",):
                    idx = torch.from_numpy(r.integers(0, rows, nb * bag_len).astype(np.int32)).cuda()
                    off = torch.arange(0, nb * bag_len, bag_len, dtype=torch.int32, device="cuda")
                    out = torch.empty((nb, dim), dtype=tdt, device="cuda")
                    ms = time_graph(torch, lambda: ops.embedding_bag(table, idx, off, mode, out=out), inner=10, reps=7)
                    nbytes = nb * bag_len * (dim * sz + 4) + nb * 4 + nb * dim * sz
                    i64, o64 = idx.long(), off.long()
                    tms = time_graph(torch, lambda: F.embedding_bag(i64, table, o64, mode=mode), inner=10, reps=5)
                    print("%5d %5s %4d %6s | %9.4f %9.0f | %9.4f | %.2f" % (
                        dim, "f16" if sz == 2 else "f32", bag_len, mode, ms, nbytes / ms / 1e6, tms, tms / ms),
                        flush=True)


def sweep_layer_norm(torch, ops):
    """SkipLayerNorm (out = LN(x + skip), fp32 gamma / beta) over row lengths, row counts and types;
    algorithmic bytes = two operands read + one written; beside torch's add + layer_norm on the
    same GPU, both timed as 10 launches captured in one HIP graph."""
    print("%7s %6s %5s | %9s %8s | %9s | %s" % ("rows", "ld", "type", "ms", "GB/s", "torch ms", "speedup"), flush=True)
    for tdt in (torch.float16, torch.float32):
        for ld in (64, 128, 256, 768, 1000, 1024, 2048, 4096, 8192, 32768):
            for rows in (1024, 8192, 65536, 262144):
                if rows * ld * 4 > (1 << 30):
                    continue
                x = torch.randn((rows, ld), device="cuda").to(tdt)
                sk = torch.randn((rows, ld), device="cuda").to(tdt)
                g, b = torch.randn(ld, device="cuda"), torch.randn(ld, device="cuda")
                out = torch.empty_like(x)
                ms = time_graph(torch, lambda: ops.skip_layer_norm(x, g, b, skip=sk, eps=1e-5, out=out), inner=10, reps=7)
                gt, bt = g.to(tdt), b.to(tdt)
                tms = time_graph(torch, lambda: torch.nn.functional.layer_norm(x + sk, (ld,), gt, bt, 1e-5),
                                 inner=10, reps=5)
                nbytes = 3 * rows * ld * x.element_size()
                print("%7d %6d %5s | %9.4f %8.0f | %9.4f | %.2f" % (
                    rows, ld, "f16" if tdt == torch.float16 else "f32", ms, nbytes / ms / 1e6, tms, tms / ms), flush=True)


def mixed_bag_lengths(torch, ops, workloads, wl, tabs):
    """The workload's tables with every other table one-hot (one id per bag) and the rest with bags twice
    as long (Zipf lengths 2 .. 200, mean 32.6), ids Zipf(1.1) as in the workload: the fused launch with
    and without each table's own mean bag length (fwdmi_bag_ext.table_avg_len), checked equal."""
    rng = np.random.Generator(np.random.PCG64(4005))
    cdf = workloads.zipf_cdf(100, 1.1)
    idx, off, n_ids = [], [], 0
    for t in range(len(tabs)):
        if t % 2 == 0:
            lengths = np.ones(wl.n_bags, np.int64)
        else:
            lengths = 2 * (workloads.zipf_ranks(rng, 100, 1.1, wl.n_bags, cdf).astype(np.int64) + 1)
        n = int(lengths.sum())
        n_ids += n
        ids = workloads.scatter_ranks(workloads.zipf_ranks(rng, wl.rows[t], 1.1, n), wl.rows[t]).astype(np.int32)
        idx.append(torch.from_numpy(ids).cuda())
        off.append(torch.from_numpy(workloads.offsets_from_lengths(lengths, np.int32)).cuda())
    b = ops.MultiTableBatch(tabs, idx, off)
    out = torch.empty((wl.n_bags, len(tabs) * wl.dim), dtype=tabs[0].dtype, device="cuda")
    res = {"what": "every other table one-hot, the others Zipf lengths 2 .. 200 (mean 32.6); ids Zipf(1.1)",
           "total_ids": n_ids, "bags": wl.n_bags * len(tabs)}
    _, per = time_events(torch, lambda: b.forward(out=out, xcd_table_affinity=True), 40, 10)
    res["ms_per_launch"] = float(per.mean())
    res["bags_per_s"] = wl.n_bags * len(tabs) / (float(per.mean()) * 1e-3)
    with_hints = out.clone()
    hints, b.table_avg_len = b.table_avg_len, None
    _, per = time_events(torch, lambda: b.forward(out=out, xcd_table_affinity=True), 40, 10)
    b.table_avg_len = hints
    res["ms_per_launch_without_table_avg_len"] = float(per.mean())
    res["results_equal"] = bool(torch.equal(out.view(torch.int16), with_hints.view(torch.int16)))
    return res


REPLAY_CHUNK = 1830                   # ids per replay workgroup, as the product's runs of 112 bags x 16.3 ids


def replay_times(torch, ops, wl, tabs, idx, off, steps=60):
    """Times (ms, median of HIP-event durations) of bench_aux/replay_gather.hip on the
    workload's id stream: the rows alone, the rows plus as many stored bytes as the product writes
    (plain / non-temporal stores), and with the stores confined to 4 MiB.  None when the measurement
    aid is not built."""
    import ctypes as C
    dll = microbench_dll()
    if dll is None:
        return None
    chunk = REPLAY_CHUNK
    it_t, it_s, it_c = [], [], []
    for t in range(len(wl.rows)):
        n = wl.indices[t].size
        for s0 in range(0, n, chunk):
            it_t.append(t), it_s.append(s0), it_c.append(min(chunk, n - s0))
    n_items = len(it_t)
    cost = ops.MultiTableBatch(tabs, idx, off).default_table_cost()
    c = np.cumsum(cost[np.array(it_t)] * np.array(it_c))
    c /= c[-1]
    xs = [0] + [int(np.searchsorted(c, k / 8.0)) for k in range(1, 8)] + [n_items]
    longest = max(xs[k + 1] - xs[k] for k in range(8))

    class Args(C.Structure):
        _fields_ = [("tables", C.c_void_p), ("item_table", C.c_void_p), ("item_start", C.c_void_p),
                    ("item_count", C.c_void_p), ("out", C.c_void_p), ("xcd_start", C.c_int32 * 9),
                    ("store_every", C.c_int32), ("store_mode", C.c_int32), ("one", C.c_float)]
    td = np.zeros((len(tabs), 2), np.int64)
    for t in range(len(tabs)):
        td[t] = (tabs[t].data_ptr(), idx[t].data_ptr())
    d_td = torch.from_numpy(td).cuda()
    d_t, d_s, d_c = (torch.tensor(a, dtype=torch.int32).cuda() for a in (it_t, it_s, it_c))
    buf = torch.zeros((n_items * 16 * 64, 128), dtype=torch.float16, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    avg_len = wl.n_indices() / float(wl.n_bags * len(wl.rows))
    every = max(8, int(round(avg_len / 8.0)) * 8)   # whole 8-row steps: 16 rows per result for config 4
    res = {"rows_per_result_row": every}
    for key, store_every, mode in (("gather_only_ms", 0, 1), ("gather_plain_stores_ms", every, 1),
                                   ("gather_streaming_stores_ms", every, 2), ("gather_stores_within_4MiB_ms", every, 3)):
        a = Args(d_td.data_ptr(), d_t.data_ptr(), d_s.data_ptr(), d_c.data_ptr(), buf.data_ptr(),
                 (C.c_int32 * 9)(*xs), store_every, mode, 1.0)

        def fn():
            rc = dll.fwdmi_mb_replay_gather(C.byref(a), longest, stream)
            if rc:
                raise RuntimeError("replay launch failed: hipError %d" % rc)
        _, per = time_events(torch, fn, steps, 10)
        res[key] = float(np.median(per))
    return res


def reorder_chunks(ids, chunk, order):
    """The id stream of one table with every `chunk` ids (what one replay workgroup fetches)
    rearranged.  "phased": the ids that occur once in the chunk, then the repeated ones sorted by row,
    dealt to the sixteen slots of the workgroup in turn so that all slots fetch once-only rows
    (likely misses) at the same time and repeated rows (likely hits) at the same time;
    "phased_unsorted": the same two phases with the repeated ids in their original order; "bursts":
    every id stays where a once-only or a repeated id was, but the repeated ones are sorted among
    themselves (equal rows are fetched together, misses and hits stay mixed); "grouped": sorted by row."""
    out = np.empty_like(ids)
    for s0 in range(0, ids.size, chunk):
        c = ids[s0:s0 + chunk]
        if order == "grouped":
            o = np.sort(c)
        else:
            _, inv, cnt = np.unique(c, return_inverse=True, return_counts=True)
            once = cnt[inv] == 1
            if order == "phased":
                o = np.concatenate([c[once], np.sort(c[~once])])
            elif order == "phased_unsorted":
                o = np.concatenate([c[once], c[~once]])
            else:   # bursts
                o = c.copy()
                o[~once] = np.sort(c[~once])
        # slot k of the workgroup sums a contiguous sixteenth of the chunk: give it elements k, k+16, ... of `o`
        out[s0:s0 + c.size] = np.concatenate([o[k::16] for k in range(16)])
    return out


def replay_hot_times(torch, ops, wl, tabs, k_hot, steps=60):
    """bench_aux/replay_hot.hip on the workload's id stream: every chunk rearranged on the host into the
    ids of rows that are not among the table's `k_hot` most frequent ones (counted on this batch) and,
    behind them, one LDS slot number per fetch of a hot row.  Returns ms (median of HIP-event
    durations) without and with result stores, and the share of the fetches that LDS serves."""
    import ctypes as C
    dll = microbench_dll()
    if dll is None:
        return None
    chunk = REPLAY_CHUNK
    it_t, it_s, it_c, it_h, streams, hots = [], [], [], [], [], []
    n_hot_fetches = 0
    for t in range(len(wl.rows)):
        ids = wl.indices[t]
        rows, cnt = np.unique(ids, return_counts=True)
        top = rows[np.argsort(-cnt, kind="stable")[:k_hot]].astype(np.int32)
        top = np.concatenate([top, np.zeros(k_hot - top.size, np.int32)])      # a table of fewer rows than k_hot
        lut = np.full(wl.rows[t], -1, np.int32)
        lut[top[::-1]] = np.arange(k_hot - 1, -1, -1, dtype=np.int32)
        out = np.empty_like(ids)
        for s0 in range(0, ids.size, chunk):
            c = ids[s0:s0 + chunk]
            slot = lut[c]
            hot = slot >= 0
            out[s0:s0 + c.size] = np.concatenate([c[~hot], slot[hot]])
            it_t.append(t), it_s.append(s0), it_c.append(c.size), it_h.append(int(hot.sum()))
        n_hot_fetches += int(sum(it_h[-((ids.size + chunk - 1) // chunk):]))
        streams.append(torch.from_numpy(out).cuda())
        hots.append(torch.from_numpy(top).cuda())
    n_items = len(it_t)
    cost = ops.MultiTableBatch(tabs, streams, [torch.zeros(wl.n_bags, dtype=torch.int32, device="cuda")] * len(tabs)
                               ).default_table_cost()
    c = np.cumsum(cost[np.array(it_t)] * np.array(it_c))
    c /= c[-1]
    xs = [0] + [int(np.searchsorted(c, k / 8.0)) for k in range(1, 8)] + [n_items]
    longest = max(xs[k + 1] - xs[k] for k in range(8))

    class Args(C.Structure):
        _fields_ = [("tables", C.c_void_p), ("item_table", C.c_void_p), ("item_start", C.c_void_p),
                    ("item_count", C.c_void_p), ("item_hot", C.c_void_p), ("out", C.c_void_p),
                    ("xcd_start", C.c_int32 * 9), ("store_every", C.c_int32), ("store_mode", C.c_int32),
                    ("n_hot", C.c_int32), ("one", C.c_float)]
    td = np.zeros((len(tabs), 3), np.int64)
    for t in range(len(tabs)):
        td[t] = (tabs[t].data_ptr(), streams[t].data_ptr(), hots[t].data_ptr())
    d_td = torch.from_numpy(td).cuda()
    d_t, d_s, d_c, d_h = (torch.tensor(a, dtype=torch.int32).cuda() for a in (it_t, it_s, it_c, it_h))
    buf = torch.zeros((n_items * 16 * 64, 128), dtype=torch.float16, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    avg_len = wl.n_indices() / float(wl.n_bags * len(wl.rows))
    every = max(8, int(round(avg_len / 8.0)) * 8)
    res = {"hot_rows_per_table": k_hot, "share_of_fetches_served_by_lds": n_hot_fetches / float(wl.n_indices())}
    for key, store_every, mode in (("gather_only_ms", 0, 1), ("gather_streaming_stores_ms", every, 2)):
        a = Args(d_td.data_ptr(), d_t.data_ptr(), d_s.data_ptr(), d_c.data_ptr(), d_h.data_ptr(), buf.data_ptr(),
                 (C.c_int32 * 9)(*xs), store_every, mode, k_hot, 1.0)

        def fn():
            rc = dll.fwdmi_mb_replay_hot(C.byref(a), longest, stream)
            if rc:
                raise RuntimeError("replay launch failed: hipError %d" % rc)
        _, per = time_events(torch, fn, steps, 10)
        res[key] = float(np.median(per))
    return res


def replay(torch, ops, workloads, ids_mode, order="stream", k_hot=0):
    """`--replay`: the product launch beside the bag-free replay of the same id stream (a table on stdout)."""
    wl = workloads.config4()
    rng = np.random.Generator(np.random.PCG64(1))
    for t in range(len(wl.rows)):
        n = wl.indices[t].size
        if ids_mode == "equal":
            wl.indices[t] = np.zeros(n, np.int32)
        elif ids_mode == "uniform":
            wl.indices[t] = rng.integers(0, wl.rows[t], n).astype(np.int32)
    tabs = device_tables(wl, torch)
    idx = [torch.from_numpy(i).cuda() for i in wl.indices]
    off = [torch.from_numpy(o).cuda() for o in wl.offsets]
    batch = ops.MultiTableBatch(tabs, idx, off)
    out = torch.zeros((wl.n_bags, batch.width), dtype=torch.float16, device="cuda")
    for _ in range(300):
        batch.forward(out=out, xcd_table_affinity=True)
    _, per = time_events(torch, lambda: batch.forward(out=out, xcd_table_affinity=True), 60, 10)
    print("ids: %s" % ids_mode)
    print("%-72s %8.4f ms" % ("product launch (bags, ordered by length, %d result rows of 256 B)" %
                              (wl.n_bags * len(wl.rows)), float(np.median(per))), flush=True)
    del out, batch
    if order != "stream":
        # the replay knows no bags, so the order inside a workgroup's chunk is free: the product launch above
        # ran on the ids as they come, the replay below runs on the rearranged stream (the same rows in all)
        t0 = time.time()
        idx = [torch.from_numpy(reorder_chunks(i, REPLAY_CHUNK, order)).cuda() for i in wl.indices]
        print("ids inside every chunk of %d rearranged (%s) in %.1f s" % (REPLAY_CHUNK, order, time.time() - t0), flush=True)
    r = replay_times(torch, ops, wl, tabs, idx, off)
    if r is None:
        raise SystemExit("build the measurement aid first: make -C bench_aux")
    e = r["rows_per_result_row"]
    print("replay, ids inside a chunk: %s" % order)
    for label, key in (("gather only (one result row per slot)", "gather_only_ms"),
                       ("gather + a 256 B result row every %d rows, plain stores" % e, "gather_plain_stores_ms"),
                       ("gather + a 256 B result row every %d rows, non-temporal stores" % e, "gather_streaming_stores_ms"),
                       ("gather + a 256 B result row every %d rows, stores confined to 4 MiB (never leave L2)" % e,
                        "gather_stores_within_4MiB_ms")):
        print("%-72s %8.4f ms" % (label, r[key]), flush=True)
    if k_hot > 0:
        del idx, off
        h = replay_hot_times(torch, ops, wl, tabs, min(64, k_hot))
        print("replay with the %d most frequent rows of every table in LDS (%.1f %% of the fetches):" %
              (h["hot_rows_per_table"], 100.0 * h["share_of_fetches_served_by_lds"]))
        print("%-72s %8.4f ms" % ("gather only (one result row per slot)", h["gather_only_ms"]), flush=True)
        print("%-72s %8.4f ms" % ("gather + a 256 B result row every %d rows, non-temporal stores" % e,
                                  h["gather_streaming_stores_ms"]), flush=True)


def lru_sim(workloads, capacities=(8192, 12288, 16384, 32768)):
    """Rows an LRU cache of `capacity` 256-byte rows fetches over each table's id stream in bag
    order (one table at a time, as an XCD works through it): a 4 MiB L2 holds 16384 rows if it held
    nothing else."""
    from collections import OrderedDict
    wl = workloads.config4()
    distinct = sum(int(np.unique(i).size) for i in wl.indices)
    print("ids %d, distinct rows %d" % (wl.n_indices(), distinct), flush=True)
    for cap in capacities:
        t0, miss = time.time(), 0
        for ids in wl.indices:
            cache = OrderedDict()
            for r in ids.tolist():
                if r in cache:
                    cache.move_to_end(r)
                else:
                    miss += 1
                    cache[r] = None
                    if len(cache) > cap:
                        cache.popitem(last=False)
        print("capacity %6d rows (%4.1f MiB): %8d rows fetched = %.2f x the distinct rows  (%.0f s)" %
              (cap, cap * 256 / 2**20, miss, miss / distinct, time.time() - t0), flush=True)


def main():
    args = parse()
    if args.record_traffic:
        record_traffic(*args.record_traffic, batches=args.batches, l2_csv=args.record_l2)
        return
    if args.lru_sim:
        sys.path.insert(0, ROOT)
        from forward_amd import workloads as _wl   # imports torch (CPU is enough) through the package
        lru_sim(_wl)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (got --gpus %d)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    import torch
    from forward_amd import ops, workloads
    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(1)
    if args.hbm_gather:
        print(json.dumps(hbm_gather(torch, ops, copy_bandwidth(torch))), flush=True)
        return
    if args.sweep:
        sweep(torch, ops)
        sweep_layer_norm(torch, ops)
        return
    if args.replay:
        replay(torch, ops, workloads, args.ids, args.order, args.hot)
        return

    t0 = time.time()
    wl = workloads.config4(n_tables=args.tables, n_bags=args.bags)
    n_batches = max(1, args.batches)
    wls = [workloads.config4_fresh_batch(wl, b) for b in range(n_batches)]
    log("ids/offsets of %d batches generated in %.1fs: %d tables, %d bags each, %d ids in batch 0, rows %s" %
        (n_batches, time.time() - t0, len(wl.rows), wl.n_bags, wl.n_indices(), wl.rows))
    tabs = device_tables(wl, torch)
    idxs = [[torch.from_numpy(i).cuda() for i in w.indices] for w in wls]
    offs = [[torch.from_numpy(o).cuda() for o in w.offsets] for w in wls]
    batches = [ops.MultiTableBatch(tabs, idxs[b], offs[b]) for b in range(n_batches)]
    idx, off, batch = idxs[0], offs[0], batches[0]
    out = torch.zeros((wl.n_bags, batch.width), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    log("tables resident: %.2f GB, setup %.1fs" % (sum(t.numel() * 2 for t in tabs) / 1e9, time.time() - t0))

    issued = []          # batch number of every step issued so far: step i works on batch i mod B

    if args.per_table:
        def step():
            b = len(issued) % n_batches
            issued.append(b)
            for t in range(batch.n_tables):
                ops.embedding_bag(tabs[t], idxs[b][t], offs[b][t], "sum", out=out, out_col=t * wl.dim)
        launches_per_step = batch.n_tables
    else:
        def step():
            b = len(issued) % n_batches
            issued.append(b)
            batches[b].forward(out=out, xcd_table_affinity=not args.no_xcd_affinity)
        launches_per_step = 1

    # untimed: brings the engine clock to its steady state, so that a short timed run measures
    # what a long one does (the first tens of launches after start-up run below the steady clock)
    for _ in range(max(0, args.prewarm)):
        step()
    torch.cuda.synchronize()
    wall, per = time_events(torch, step, args.steps, args.warmup)
    timed = issued[-args.steps:]
    checked_batch = timed[-1]               # `out` now holds this batch's result, written by a timed step
    ms_per_step = wall / args.steps * 1e3
    total_bags = wl.n_bags * len(wl.rows)
    alg_per_batch = [w.algorithmic_bytes(table_itemsize=2, out_itemsize=2, index_itemsize=4) for w in wls]
    alg_bytes = float(np.mean([alg_per_batch[b] for b in timed]))     # per step, over the steps that were timed
    ev_ms = float(np.mean(per))
    achieved = alg_bytes / (ev_ms * 1e-3) / 1e9
    full = not args.per_table and args.tables == 26 and args.bags == 65536
    comp_bytes, unique_rows = compulsory_bytes(wl)
    # what the 256 vector L1s can return: 64 B per clock and CU at the published peak clock
    l1_peak = torch.cuda.get_device_properties(0).multi_processor_count * 64.0 * MI355X_PEAK_CLOCK_HZ / 1e9
    traffic = load_traffic("rotating_batches" if n_batches > 1 else "same_batch") if full else None
    traffic_bytes = traffic["bytes_per_launch"] if traffic else None
    # Time floor of one launch: the bytes that really cross the L2 boundary (rocprofv3 counters of
    # this launch; the compulsory bytes when no counter figure belongs to this kernel) at the HBM
    # peak, or every algorithmic row byte through the L1s at their return rate, whichever is longer.
    hbm_bytes = traffic_bytes if traffic_bytes else comp_bytes
    floor_hbm_ms = hbm_bytes / (HBM_PEAK_GBS * 1e9) * 1e3    # per step (the counter figure is of the one fused launch)
    floor_l1_ms = alg_bytes / (l1_peak * 1e9) * 1e3
    floor_ms = max(floor_hbm_ms, floor_l1_ms)

    result = {
        "metric": "EmbeddingBag bags/sec + achieved HBM GB/s (% peak), 26-table fp16 batch 64K",
        "value": total_bags / (ms_per_step * 1e-3), "unit": "bags/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "prewarm_launches": max(0, args.prewarm), "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config4: DLRM sparse stage, %d tables x %d bags, dim %d fp16, int32 ids, "
                               "Zipf(1.1) ids and bag lengths (mean %.2f), fp16 output [%d, %d]%s"
                               % (len(wl.rows), wl.n_bags, wl.dim, wl.n_indices() / total_bags, wl.n_bags,
                                  batch.width, "" if (args.tables == 26 and args.bags == 65536) else " (REDUCED, debug)"),
                   "storage": "fp16 rows and output, fp32 accumulation, int32 ids",
                   "launch": "per-table" if args.per_table else
                   ("fused multi-table" if args.no_xcd_affinity else "fused multi-table, per-XCD table affinity"),
                   "id_batches": n_batches,
                   "id_batches_are": ("step i works on batch i mod %d: fresh bag lengths and ids over the same tables, all "
                                      "resident in HBM before the timed region" % n_batches) if n_batches > 1 else
                                     "every step replays the same batch",
                   "total_ids": wl.n_indices(), "table_bytes": int(sum(t.numel() * 2 for t in tabs)),
                   "device": dict(zip(("compute_units", "xcds"), ops.device_topology()))},
        "roofline": {
            "bound": "hbm",
            "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "frac_is": "algorithmic bytes per launch (every gathered row + its id, offsets, output) / kernel time / HBM "
                       "peak; above 1 because L1 / L2 serve most row bytes under Zipf ids: not a position under the HBM "
                       "ceiling, see frac_hbm_side",
            "frac_algorithmic": achieved / HBM_PEAK_GBS,
            "frac_algorithmic_is": "the same figure under the name that says what it counts",
            "traffic": traffic_bytes,
            "traffic_is": "bytes per launch beyond L2 (rocprofv3 FETCH_SIZE + WRITE_SIZE of this launch in this batch "
                          "mode, scaled by a 1 GiB copy; memory-side-cache hits included), from profiles/traffic.json",
            "algorithmic_bytes_per_launch": alg_bytes / launches_per_step,
            "kernel_ms_avg": ev_ms / launches_per_step, "kernel_ms_median": float(np.median(per)),
            "kernel_ms_p10": float(np.percentile(per, 10)),
            "kernel_ms_p90": float(np.percentile(per, 90)), "launches_per_step": launches_per_step,
            # a bounded reading: the longer of "bytes beyond L2 at the HBM peak" and "every row byte through
            # the L1s at their return rate" over the kernel time
            "frac_time_floor": floor_ms / ev_ms,
            "frac_time_floor_is": "max(hbm-side bytes / 8 TB/s, algorithmic bytes / l1_peak) / kernel time",
            "hbm_side_bytes_used": hbm_bytes, "hbm_side_bytes_are": "counters" if traffic_bytes else "compulsory",
            "floor_ms": floor_ms, "floor_hbm_ms": floor_hbm_ms, "floor_l1_ms": floor_l1_ms,
            "compulsory_bytes_batch0": comp_bytes, "unique_rows_batch0": unique_rows,
            "compulsory_floor_ms": comp_bytes / (HBM_PEAK_GBS * 1e9) * 1e3,
            "l1_peak_GBs": l1_peak, "l1_frac": achieved / l1_peak},
        "samples_per_s": wl.n_bags / (ms_per_step * 1e-3),
    }
    if traffic_bytes:
        r = result["roofline"]
        # bytes that crossed the L2 boundary (rocprofv3 counters of the same launch) over this run's time
        r["traffic_GBs"] = traffic_bytes / (ev_ms * 1e-3) / 1e9
        r["frac_hbm_side"] = r["traffic_GBs"] / HBM_PEAK_GBS
        r["frac_hbm_side_is"] = "traffic / kernel time / HBM peak: what crosses the L2 boundary against the 8 TB/s ceiling"
        r["refetch_ratio"] = traffic["fetch_bytes"] / float(
            comp_bytes - len(wl.rows) * wl.n_bags * wl.dim * 2)   # fetched / (distinct rows + ids + offsets), batch 0
        if "l2_hit_rate" in traffic:
            r["l2_hit_rate"] = traffic["l2_hit_rate"]
            r["l2_hit_rate_is"] = "TCC_HIT_sum / (TCC_HIT_sum + TCC_MISS_sum) of this launch (rocprofv3, a pass of its own)"
        r["traffic_kernel_source_sha256"] = traffic["kernel_source_sha256"]
    else:
        result["roofline"]["frac_hbm_side"] = None
    # the result of the last timed step, kept for the comparison with the oracle below
    gpu_out_checked = out.cpu().numpy() if not args.no_cpu else None

    if n_batches > 1 and not args.no_extra and not args.per_table:
        # the figure of a loop that replays one batch: part of its rows is served by the memory-side
        # cache from the step before, which fresh ids do not get
        same_step = lambda: batches[0].forward(out=out, xcd_table_affinity=not args.no_xcd_affinity)
        for _ in range(max(0, args.prewarm)):      # the copy above left the GPU idle: back to the steady clock first
            same_step()
        torch.cuda.synchronize()
        wall1, per1 = time_events(torch, same_step, args.steps, args.warmup)
        same = {"ms_per_step": wall1 / args.steps * 1e3, "kernel_ms_avg": float(np.mean(per1)),
                "bags_per_s": total_bags / (wall1 / args.steps),
                "what": "every step replays batch 0 (the same ids and bag lengths)"}
        t1 = load_traffic("same_batch") if full else None
        if t1:
            same["traffic"] = t1["bytes_per_launch"]
            same["frac_hbm_side"] = t1["bytes_per_launch"] / (same["kernel_ms_avg"] * 1e-3) / 1e9 / HBM_PEAK_GBS
        result["same_batch_replay"] = same

    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)      # one elementwise kernel: reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    if not args.no_cpu:
        t1 = time.time()
        cpu, cpu_out, nb, lt_out = cpu_baseline(wls[checked_batch], tabs, args.cpu_bags, torch)
        cpu["gpu_matches_oracle_on_sample"] = bool(np.array_equal(gpu_out_checked[:nb].view(np.uint16),
                                                                  cpu_out.view(np.uint16)))
        cpu["checked"] = "the output of the last timed step (batch %d of %d) against the oracle, bit for bit" % (
            checked_batch, n_batches)
        cpu["gpu_vs_libtorch_cpu"] = compare_with_libtorch(gpu_out_checked[:nb], lt_out)
        del gpu_out_checked, cpu_out, lt_out
        result["cpu_baseline"] = cpu
        log("cpu baseline leg %.1fs" % (time.time() - t1))
    if not args.no_extra:
        # the side measurements below work on batch 0 and compare with its result
        batch.forward(out=out, xcd_table_affinity=not args.no_xcd_affinity)
        torch.cuda.synchronize()
    if not args.no_extra and not args.per_table:
        # the same stage through PyTorch-ROCm's own GPU kernels: 26 embedding_bag launches + cat
        # (a yardstick only: a failure here is recorded, it does not fail the measurement)
        try:
            idx64, off64 = [i.long() for i in idx], [o.long() for o in off]

            def torch_step():
                return torch.cat([torch.nn.functional.embedding_bag(idx64[t], tabs[t], off64[t], mode="sum")
                                  for t in range(len(tabs))], dim=1)
            _, per_t = time_events(torch, torch_step, 5, 2)
            result["pytorch_rocm_gpu"] = {
                "ms_per_step": float(np.mean(per_t)), "bags_per_s": total_bags / (float(np.mean(per_t)) * 1e-3),
                "what": "26 x torch.nn.functional.embedding_bag (int64 ids) + torch.cat on the same GPU"}
            del idx64, off64
        except Exception as e:  # noqa: BLE001
            result["pytorch_rocm_gpu"] = {"error": repr(e)}
    if not args.no_extra and full:
        try:
            result["plugin_level"] = plugin_level(torch, wl, tabs, idx, off, out)
        except Exception as e:  # noqa: BLE001  (a side measurement must not lose the headline)
            result["plugin_level"] = {"error": repr(e)}
    if not args.no_extra and full:
        # the same id stream as a plain gather that knows no bags and stores as many bytes: what the
        # memory system charges for this workload with this lane mapping, measured in this run
        try:
            rt = replay_times(torch, ops, wl, tabs, idx, off, steps=40)
            if rt:
                rt["kernel_over_replay_with_streaming_stores"] = (ev_ms / rt["gather_streaming_stores_ms"])
                result["replay_without_bags"] = rt
        except Exception as e:  # noqa: BLE001
            result["replay_without_bags"] = {"error": repr(e)}
    if not args.no_extra and full:
        # the same 26 tables with bag lengths that differ from table to table (one-hot features beside
        # multi-hot ones): not the headline workload, reported for the launch's run sizing by table
        try:
            result["mixed_bag_lengths"] = mixed_bag_lengths(torch, ops, workloads, wl, tabs)
        except Exception as e:  # noqa: BLE001
            result["mixed_bag_lengths"] = {"error": repr(e)}
    if not args.no_extra:
        del tabs, batch, batches, idxs, offs, idx, off
        result["extra"] = extra_measurements(torch, ops, workloads, max(10, args.steps), with_cpu=not args.no_cpu)
        result["extra"]["device_copy_GBs"] = copy_bandwidth(torch)
        try:
            result["extra"]["hbm_gather_uniform_4GiB"] = hbm_gather(torch, ops, result["extra"]["device_copy_GBs"])
        except Exception as e:  # noqa: BLE001
            result["extra"]["hbm_gather_uniform_4GiB"] = {"error": repr(e)}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
