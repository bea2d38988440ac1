"""EmbeddingBagGroup_TRT: the T EmbeddingBag layers + concatenation of a DLRM-style sparse stage as
one plugin.  Its output must equal, bit for bit, the column blocks that T EmbeddingBag_TRT "002"
plugins produce one by one, and the oracle's."""
import numpy as np
import pytest
import torch

from forward_amd import lib, plugin, workloads
from forward_amd.plugin import PluginFieldData as F
from gpu_util import assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu
REG = plugin.getPluginRegistry()
GROUP = REG.getPluginCreator("EmbeddingBagGroup_TRT", "001")
SINGLE = REG.getPluginCreator("EmbeddingBag_TRT", "002")


def group_fields(tables, op=0, extra=()):
    return [F("dim", tables[0].shape[1]), F("op", op), F("count", np.array([t.shape[0] for t in tables], np.int32)),
            F("data", np.concatenate([t.reshape(-1) for t in tables]))] + list(extra)


def interleave(ids, offs):
    return [x for pair in zip(ids, offs) for x in pair]


def random_batch(rng, rows, n_bags, idt, max_len=12, lo_spill=0):
    ids, offs = [], []
    for r in rows:
        lengths = rng.integers(0, max_len, n_bags)
        offs.append(np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt))
        ids.append(rng.integers(-lo_spill, r + lo_spill, int(lengths.sum())).astype(idt))
    return ids, offs


@pytest.mark.parametrize("op", [0, 1, 2, 3])
@pytest.mark.parametrize("tdt,idt,out16", [(np.float16, np.int32, 1), (np.float32, np.int64, 0), (np.float16, np.int64, 0)])
def test_group_equals_single_table_plugins_and_oracle(oracle, op, tdt, idt, out16):
    rng = np.random.Generator(np.random.PCG64(400 + op))
    rows, dim, n_bags = [50, 4000, 7, 900, 20000], 64, 700
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(tdt) for r in rows]
    ids, offs = random_batch(rng, rows, n_bags, idt)
    it = lib.I64 if idt == np.int64 else lib.I32
    extra = [F("index_type", it), F("output_fp16", out16)]
    g = GROUP.createPlugin("sparse", group_fields(tables, op, extra))
    got = host(g(*[dev(x) for x in interleave(ids, offs)]))
    odt = np.float16 if out16 else np.float32
    assert got.shape == (n_bags, len(rows) * dim) and got.dtype == odt
    for t, tab in enumerate(tables):
        one = SINGLE.createPlugin("bag", [F("dim", dim), F("count", rows[t]), F("offset", 0), F("op", op),
                                          F("data", tab)] + extra)
        block = host(one(dev(ids[t]), dev(offs[t])))
        assert_bits_equal(got[:, t * dim:(t + 1) * dim], block, "table %d against EmbeddingBag_TRT 002" % t)
        want, _, _ = oracle.embedding_bag(tab, ids[t], offs[t], op, out_dtype=odt)
        assert_bits_equal(block, want, "table %d against the oracle" % t)
    assert not g.takeOobFlag()


def test_group_new_buffers_every_call_offsets_out_of_range_ids_and_clones(oracle):
    """The descriptors are rewritten on every enqueue: new id / offset buffers (and id counts) per
    call; per-table data_offset with ids outside the shard (skipped and flagged); [1, B] offsets
    with a trailing end offset; clone and serialize -> deserialize run on the same tables."""
    rng = np.random.Generator(np.random.PCG64(9))
    rows, dim, n_bags = [300, 5, 1200], 32, 257
    shift = [0, 1000, 40]
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(np.float32) for r in rows]
    g = GROUP.createPlugin("sparse", group_fields(tables, 0, [F("offset", np.array(shift, np.int32)),
                                                             F("include_last_offset", 1), F("xcd_affinity", 0)]))
    loaded = GROUP.deserializePlugin("sparse", g.serialize())
    for call, p in enumerate([g, g, g.clone(), loaded]):
        spill = 3 if call % 2 else 0
        ids, offs = random_batch(rng, rows, n_bags, np.int32, max_len=5 + 9 * call, lo_spill=spill)
        ids = [i + s for i, s in zip(ids, shift)]
        offs = [np.append(o, i.size).astype(np.int32).reshape(1, -1) for o, i in zip(offs, ids)]
        got = host(p(*[dev(x) for x in interleave(ids, offs)]))
        any_oob = False
        for t, tab in enumerate(tables):
            want, _, n_oob = oracle.embedding_bag(tab, ids[t], offs[t].reshape(-1), 0, include_last_offset=True,
                                                  data_offset=shift[t])
            any_oob |= n_oob > 0
            assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "call %d table %d" % (call, t))
        assert p.takeOobFlag() == any_oob


def test_group_of_many_tables_and_scaled_config4(oracle):
    # more tables than one descriptor launch carries (56), odd row width (scalar loads)
    rng = np.random.Generator(np.random.PCG64(10))
    rows = [int(r) for r in rng.integers(1, 40, 70)]
    tables = [rng.standard_normal((r, 6)).astype(np.float32) for r in rows]
    ids, offs = random_batch(rng, rows, 33, np.int32, max_len=4)
    got = host(GROUP.createPlugin("many", group_fields(tables, 0))(*[dev(x) for x in interleave(ids, offs)]))
    for t, tab in enumerate(tables):
        want, _, _ = oracle.embedding_bag(tab, ids[t], offs[t], 0)
        assert_bits_equal(got[:, t * 6:(t + 1) * 6], want, "table %d of 70" % t)

    # the 26-table shape at reduced size, fp16 rows and output, with the default cost estimate
    wl = workloads.config4(variant=3, n_tables=26, n_bags=2048, max_rows=20000)
    tabs = [wl.host_table(t) for t in range(26)]
    g = GROUP.createPlugin("sparse", group_fields(tabs, 0, [F("output_fp16", 1)]))
    got = host(g(*[dev(x) for x in interleave(wl.indices, wl.offsets)]))
    want = np.zeros((2048, 26 * 128), np.float16)
    for t in range(26):
        oracle.embedding_bag(tabs[t], wl.indices[t], wl.offsets[t], oracle.OP_SUM, out=want, out_col=128 * t)
    assert_bits_equal(got, want, "26 tables through the group plugin")


def test_group_enqueue_checks_and_graph_replay(oracle):
    rng = np.random.Generator(np.random.PCG64(11))
    rows, dim, n_bags, n_ids = [100, 2000], 16, 64, 500
    tables = [rng.standard_normal((r, dim)).astype(np.float32) for r in rows]
    g = GROUP.createPlugin("sparse", group_fields(tables, 0))

    def batch(seed):
        r = np.random.Generator(np.random.PCG64(seed))
        ids = [r.integers(0, n, n_ids).astype(np.int32) for n in rows]
        offs = [np.sort(r.integers(0, n_ids + 1, n_bags)).astype(np.int32) for _ in rows]
        for o in offs:
            o[0] = 0
        return ids, offs

    ids, offs = batch(0)
    d_in = [dev(x) for x in interleave(ids, offs)]
    d_out = torch.zeros((n_bags, 2 * dim), dtype=torch.float32, device="cuda")
    descs = [(tuple(t.shape), lib.I32) for t in d_in]
    g.configurePlugin(descs, [((n_bags, 2 * dim), lib.F32)])
    ptrs = [t.data_ptr() for t in d_in]
    # no workspace, tables that disagree on the bag count: refused before any launch
    assert g.enqueue_raw(descs, [((n_bags, 2 * dim), lib.F32)], ptrs, [d_out.data_ptr()]) == lib.ERR_BAD_ARG
    assert "workspace" in lib.last_error()
    ws = torch.empty(256, dtype=torch.uint8, device="cuda")
    bad = list(descs)
    bad[3] = ((n_bags + 1,), lib.I32)
    rc = g.enqueue_raw(bad, [((n_bags, 2 * dim), lib.F32)], ptrs, [d_out.data_ptr()], workspace_ptr=ws.data_ptr())
    assert rc == lib.ERR_BAD_ARG and "number of bags" in lib.last_error()

    def want(ids, offs):
        w = np.zeros((n_bags, 2 * dim), np.float32)
        for t in range(2):
            oracle.embedding_bag(tables[t], ids[t], offs[t], 0, out=w, out_col=t * dim)
        return w

    g.enqueue(d_in, [d_out], workspace=ws)
    torch.cuda.synchronize()
    assert_bits_equal(host(d_out), want(ids, offs), "eager")
    # captured once (descriptor launch + reduction), replayed with new values in the same buffers
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g.enqueue(d_in, [d_out], workspace=ws)
    for seed in (1, 2, 3):
        ids, offs = batch(seed)
        for t, x in zip(d_in, interleave(ids, offs)):
            t.copy_(torch.from_numpy(x))
        d_out.fill_(5.0)
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(host(d_out), want(ids, offs), "replay %d" % seed)


@pytest.mark.parametrize("tdt", [np.float16, np.float32])
def test_group_with_per_sample_weights(oracle, tdt):
    rng = np.random.Generator(np.random.PCG64(12))
    rows, dim, n_bags = [40, 3000, 700], 64, 500
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(tdt) for r in rows]
    ids, offs = random_batch(rng, rows, n_bags, np.int32, max_len=30)
    psw = [rng.random(i.size).astype(tdt) for i in ids]
    g = GROUP.createPlugin("sparse", group_fields(tables, 0, [F("per_sample_weights", 1)]))
    ins = [x for trio in zip(ids, offs, psw) for x in trio]
    got = host(g(*[dev(x) for x in ins]))
    for t, tab in enumerate(tables):
        want, _, _ = oracle.embedding_bag(tab, ids[t], offs[t], 0, per_sample_weights=psw[t], out_dtype=np.float32)
        assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "weighted table %d" % t)
    # the launcher form: weights on some tables only (the others count every id once)
    from forward_amd import ops
    batch = ops.MultiTableBatch([dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs],
                                per_sample_weights=[dev(psw[0]), None, dev(psw[2])])
    out = host(batch.forward(out_dtype=torch.float32, xcd_table_affinity=True))
    for t, tab in enumerate(tables):
        want, _, _ = oracle.embedding_bag(tab, ids[t], offs[t], 0, per_sample_weights=None if t == 1 else psw[t],
                                          out_dtype=np.float32)
        assert_bits_equal(out[:, t * dim:(t + 1) * dim], want, "launcher, table %d" % t)
    with pytest.raises(lib.FwdmiError, match="SUM"):
        batch.forward(mode="max")


@pytest.mark.parametrize("count", [0, -3])
@pytest.mark.parametrize("op", ["sum", "max"])
def test_descriptor_of_a_table_without_rows(oracle, count, op):
    """A descriptor with count <= 0 (and a null data pointer) handed straight to the C ABI: no row
    address may be formed; the table's block is zeros, its ids count as out of range (flag set),
    and the other tables of the launch are unaffected."""
    import ctypes as C
    from forward_amd import ops
    rng = np.random.Generator(np.random.PCG64(77 + count))
    rows, dim, n_bags = [300, 0, 4000], 128, 900
    tables = [(rng.standard_normal((max(r, 1), dim)) * 0.3).astype(np.float16) for r in rows]
    ids, offs = random_batch(rng, [300, 50, 4000], n_bags, np.int32)
    d_tab = [dev(t) for t in tables]
    d_ids, d_off = [dev(i) for i in ids], [dev(o) for o in offs]
    desc = np.zeros((3, 8), np.int64)
    for t in range(3):
        desc[t] = (d_tab[t].data_ptr(), d_ids[t].data_ptr(), d_off[t].data_ptr(), rows[t], ids[t].size, 0, t * dim, 0)
    desc[1, 0], desc[1, 3] = 0, count
    d_desc = torch.from_numpy(desc).cuda()
    for affinity in (0, lib.BAG_XCD_TABLE_AFFINITY):
        out = torch.full((n_bags, 3 * dim), 7.0, dtype=torch.float16, device="cuda")
        flag = torch.zeros(1, dtype=torch.int32, device="cuda")
        x = ops._ext(d_tab[0], d_ids[0], torch.float16, out_row_stride=3 * dim, oob_flag=flag, flags=affinity)
        lib.check(lib.dll.fwdmi_embedding_bag_multi(C.c_void_p(d_desc.data_ptr()), 3, n_bags, C.c_void_p(out.data_ptr()),
                                                    dim, ops.MODES[op], float(sum(i.size for i in ids)) / (3 * n_bags),
                                                    C.byref(x), C.c_void_p(torch.cuda.current_stream().cuda_stream)))
        got = host(out)
        assert int(flag.item()) == 1
        assert not got[:, dim:2 * dim].any()
        for t in (0, 2):
            want, _, _ = oracle.embedding_bag(tables[t], ids[t], offs[t], ops.MODES[op])
            assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "table %d beside the empty one" % t)
    # bags of the empty table that hold no ids raise no flag
    d_ids[1] = dev(np.zeros(1, np.int32))
    desc[1, 1], desc[1, 2], desc[1, 4] = d_ids[1].data_ptr(), dev(np.zeros(n_bags, np.int32)).data_ptr(), 0
    zero_off = dev(np.zeros(n_bags, np.int32))
    desc[1, 2] = zero_off.data_ptr()
    d_desc = torch.from_numpy(desc).cuda()
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    out = torch.full((n_bags, 3 * dim), 7.0, dtype=torch.float16, device="cuda")
    x = ops._ext(d_tab[0], d_ids[0], torch.float16, out_row_stride=3 * dim, oob_flag=flag)
    lib.check(lib.dll.fwdmi_embedding_bag_multi(C.c_void_p(d_desc.data_ptr()), 3, n_bags, C.c_void_p(out.data_ptr()), dim,
                                                ops.MODES[op], 4.0, C.byref(x),
                                                C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    assert int(flag.item()) == 0 and not host(out)[:, dim:2 * dim].any()


@pytest.mark.parametrize("tdt,idt", [(np.float32, np.int32), (np.float16, np.int64)])
def test_quarter_runs_at_segment_ends_on_ragged_tables(oracle, tdt, idt):
    """A launch large enough for the XCD mapping to cut the last runs of every segment in four
    (several hundred runs per XCD), on shapes that make those quarters ragged: a bag count that
    leaves a table's last run with one bag (three of its quarters are empty), segment cuts in the
    middle of tables (uneven costs) and at table ends (equal costs), a bag too long for the id
    window inside a tail run, empty bags, ids outside the table.  Whole output against the oracle."""
    from forward_amd import ops
    rng = np.random.Generator(np.random.PCG64(1234))
    n_tables, n_bags = 8, 80001
    dim = 64 if tdt == np.float32 else 128          # 16 lanes per row either way: 16 bags in flight per workgroup
    rows = [int(r) for r in rng.integers(5, 30000, n_tables)]
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(tdt) for r in rows]
    ids, offs = [], []
    for t, r in enumerate(rows):
        lengths = rng.integers(0, 60, n_bags)      # mean 29.5: runs of 64 bags, quarters of 16
        lengths[-1] = 40
        lengths[n_bags - 20] = 5000                 # inside the table's last runs: that quarter reads its ids unstaged
        offs.append(np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt))
        i = rng.integers(0, r, int(lengths.sum()))
        i[rng.integers(0, i.size, 50)] = r + 3      # outside the table: skipped
        ids.append(i.astype(idt))
    d_tab, d_ids, d_off = [dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs]
    want = np.zeros((n_bags, n_tables * dim), tdt)
    for t in range(n_tables):
        oracle.embedding_bag(tables[t], ids[t], offs[t], oracle.OP_SUM, out=want, out_col=dim * t)
    batch = ops.MultiTableBatch(d_tab, d_ids, d_off)
    plain = host(batch.forward())
    assert_bits_equal(plain, want, "without the XCD mapping")
    for name, cost in (("equal costs", np.ones(n_tables)), ("uneven costs", 1.0 + 0.6 * rng.random(n_tables))):
        flag = torch.zeros(1, dtype=torch.int32, device="cuda")
        got = batch.forward(out=torch.full((n_bags, n_tables * dim), 3.0, dtype=d_tab[0].dtype, device="cuda"),
                            xcd_table_affinity=True, table_cost=cost, oob_flag=flag)
        assert_bits_equal(host(got), want, name)
        assert int(flag.item()) == 1


@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_tables_of_very_different_bag_lengths(oracle, idt):
    """One-hot tables beside tables of long bags in one launch: runs are sized from the mean bag
    length of the whole launch unless every table's own mean comes with the call
    (``fwdmi_bag_ext.table_avg_len``: the tensor wrappers pass it), which gives the tables runs of
    their own size and the XCDs shares by bag length.  Both ways, with weights too, through the
    persistent descriptors and the per-call ones; whole output against the oracle."""
    from forward_amd import ops
    rng = np.random.Generator(np.random.PCG64(77))
    dim, n_bags = 64, 30000
    rows = [9000, 400, 20000, 70, 3000, 1500]
    mean_len = [1, 90, 1, 40, 1, 150]
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(np.float16) for r in rows]
    ids, offs, psw = [], [], []
    for r, m in zip(rows, mean_len):
        lengths = np.ones(n_bags, np.int64) if m == 1 else rng.poisson(m, n_bags)
        if m == 150:
            lengths[1000:1010] = 7000          # longer than the window by themselves
            lengths[5::97] = 0
        offs.append(np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt))
        ids.append(rng.integers(0, r, int(lengths.sum())).astype(idt))
        psw.append(rng.random(ids[-1].size).astype(np.float16))
    d_tab, d_ids, d_off = [dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs]
    for weights in (None, psw):
        want = np.zeros((n_bags, len(rows) * dim), np.float16)
        for t in range(len(rows)):
            oracle.embedding_bag(tables[t], ids[t], offs[t], oracle.OP_SUM, out=want, out_col=dim * t,
                                 per_sample_weights=None if weights is None else weights[t])
        batch = ops.MultiTableBatch(d_tab, d_ids, d_off,
                                    per_sample_weights=None if weights is None else [dev(w) for w in weights])
        for affinity in (False, True):
            got = batch.forward(out=torch.full((n_bags, len(rows) * dim), 3.0, dtype=torch.float16, device="cuda"),
                                xcd_table_affinity=affinity)
            assert_bits_equal(host(got), want, "weights %s, affinity %s" % (weights is not None, affinity))
            hints, batch.table_avg_len = batch.table_avg_len, None      # one run size for all tables
            got = batch.forward(xcd_table_affinity=affinity)
            batch.table_avg_len = hints
            assert_bits_equal(host(got), want, "no length hints, weights %s, affinity %s" % (weights is not None, affinity))
        got = ops.embedding_bag_group(d_tab, d_ids, d_off, per_sample_weights=None if weights is None else
                                      [dev(w) for w in weights])
        assert_bits_equal(host(got), want, "per-call descriptors, weights %s" % (weights is not None))
    batch.table_avg_len = np.full(len(rows), -1.0, np.float32)
    with pytest.raises(lib.FwdmiError, match="table_avg_len"):
        batch.forward(xcd_table_affinity=True)


def test_host_descriptor_entry_point_limits(oracle):
    """fwdmi_embedding_bag_multi_host: up to FWDMI_BAG_INLINE_TABLES tables need no device array for their
    descriptors, more do; descriptors are checked on the host before anything is launched."""
    import ctypes as C
    from forward_amd import ops
    rng = np.random.Generator(np.random.PCG64(31))
    dim, n_bags = 32, 50
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(n, d_desc, mutate=None):
        tables = [(rng.standard_normal((20 + t, dim)) * 0.3).astype(np.float32) for t in range(n)]
        ids, offs = random_batch(rng, [t.shape[0] for t in tables], n_bags, np.int32, max_len=5)
        keep = [dev(x) for x in tables + ids + offs]
        desc = np.zeros((n, 8), np.int64)
        for t in range(n):
            desc[t] = (keep[t].data_ptr(), keep[n + t].data_ptr(), keep[2 * n + t].data_ptr(), tables[t].shape[0],
                       ids[t].size, 0, t * dim, 0)
        if mutate:
            mutate(desc)
        out = torch.full((n_bags, n * dim), 9.0, dtype=torch.float32, device="cuda")
        x = ops._ext(keep[0], keep[n], torch.float32, out_row_stride=n * dim)
        rc = lib.dll.fwdmi_embedding_bag_multi_host(desc.ctypes.data, n, C.c_void_p(d_desc.data_ptr() if d_desc is not None else 0),
                                                    n_bags, C.c_void_p(out.data_ptr()), dim, 0, 2.0, C.byref(x), stream)
        return rc, host(out), tables, ids, offs

    for n, with_array in ((lib.BAG_INLINE_TABLES, False), (lib.BAG_INLINE_TABLES + 1, True)):
        d_desc = torch.empty(n * 64, dtype=torch.uint8, device="cuda") if with_array else None
        rc, got, tables, ids, offs = call(n, d_desc)
        assert rc == 0, lib.last_error()
        for t in (0, n // 2, n - 1):
            want, _, _ = oracle.embedding_bag(tables[t], ids[t], offs[t], 0)
            assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "%d tables, table %d" % (n, t))
    rc, got, *_ = call(lib.BAG_INLINE_TABLES + 1, None)
    assert rc == lib.ERR_BAD_ARG and "device array" in lib.last_error() and (got == 9.0).all()

    def col_beyond_row(desc):
        desc[1, 6] = 3 * dim
    rc, got, *_ = call(3, None, col_beyond_row)
    assert rc == lib.ERR_BAD_ARG and "beyond the row" in lib.last_error() and (got == 9.0).all()

    def no_offsets(desc):
        desc[2, 2] = 0
    rc, got, *_ = call(3, None, no_offsets)
    assert rc == lib.ERR_BAD_ARG and "offsets" in lib.last_error() and (got == 9.0).all()


def test_device_topology_is_reported():
    """The bag launches size themselves from what the runtime says of the device; the same figures are
    available to the caller (and end up in bench.py's JSON)."""
    from forward_amd import ops
    cus, xcds = ops.device_topology()
    assert cus > 0 and 1 <= xcds <= cus
    props = torch.cuda.get_device_properties(0)
    assert cus == props.multi_processor_count
