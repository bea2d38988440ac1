"""fwdmi_embedding_bag_multi_noalloc: the multi-table launch for callers that cannot allocate
device memory (its descriptor buffer is part of the library's code object).  Called through the
C ABI and compared bit for bit with fwdmi_embedding_bag_multi on the same inputs, on two calls in
a row, the second with a smaller input (fewer tables, fewer bags), so that what the first call
left in the shared buffer must not leak into the second.  Calls of more than
FWDMI_BAG_INLINE_TABLES tables go through that buffer; smaller ones carry their descriptors among
the launch's arguments: both sizes are covered."""
import ctypes as C

import numpy as np
import pytest
import torch

from forward_amd import lib, ops
from gpu_util import assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu


def make_batch(rng, rows, n_bags, dim, tdt, idt, max_len):
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(tdt) for r in rows]
    ids, offs = [], []
    for r in rows:
        lengths = rng.integers(0, max_len, n_bags)
        offs.append(np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt))
        ids.append(rng.integers(0, r, int(lengths.sum())).astype(idt))
    return tables, ids, offs


def descriptors(d_tab, d_ids, d_off, dim):
    desc = np.zeros((len(d_tab), 8), np.int64)
    for t in range(len(d_tab)):
        desc[t] = (d_tab[t].data_ptr(), d_ids[t].data_ptr(), d_off[t].data_ptr(), d_tab[t].shape[0],
                   d_ids[t].numel(), 0, t * dim, 0)
    return desc


def launch_both(tables, ids, offs, dim, op, flags):
    """(existing entry point's output, new entry point's output), each into its own buffer."""
    d_tab, d_ids, d_off = [dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs]
    n_tables, n_bags = len(tables), offs[0].size
    desc = descriptors(d_tab, d_ids, d_off, dim)
    d_desc = torch.from_numpy(desc).cuda()
    avg = float(sum(i.size for i in ids)) / max(1, n_tables * n_bags)
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for entry, tab_arg in ((lib.dll.fwdmi_embedding_bag_multi, C.c_void_p(d_desc.data_ptr())),
                           (lib.dll.fwdmi_embedding_bag_multi_noalloc, C.c_void_p(desc.ctypes.data))):
        out = torch.full((n_bags, n_tables * dim), -3.0, dtype=d_tab[0].dtype, device="cuda")
        x = ops._ext(d_tab[0], d_ids[0], d_tab[0].dtype, out_row_stride=n_tables * dim, flags=flags)
        lib.check(entry(tab_arg, n_tables, n_bags, C.c_void_p(out.data_ptr()), dim, op, avg, C.byref(x), s))
        outs.append(out)
    torch.cuda.synchronize()
    return host(outs[0]), host(outs[1])


@pytest.mark.parametrize("tdt,idt", [(np.float16, np.int32), (np.float32, np.int64)])
@pytest.mark.parametrize("through_buffer", [True, False])
def test_no_alloc_entry_point_equals_the_allocating_form_twice_in_a_row(oracle, tdt, idt, through_buffer):
    rng = np.random.Generator(np.random.PCG64(2024))
    dim = 128 if tdt == np.float16 else 64
    rows1 = [4000, 17, 90000, 512, 30000, 7, 1200, 65000, 300]
    rows2 = [900, 20000, 5]
    if through_buffer:          # more tables than travel with a launch: the built-in descriptor buffer is used
        rows1 = rows1 + [int(v) for v in rng.integers(3, 5000, lib.BAG_INLINE_TABLES + 8 - len(rows1))]
        rows2 = rows2 + [int(v) for v in rng.integers(3, 5000, lib.BAG_INLINE_TABLES + 2 - len(rows2))]
        assert len(rows2) > lib.BAG_INLINE_TABLES and len(rows2) < len(rows1)
    first = make_batch(rng, rows1, 3000, dim, tdt, idt, 24)
    second = make_batch(rng, rows2, 257, dim, tdt, idt, 9)        # smaller: fewer tables, 257 bags
    for call, (tables, ids, offs) in enumerate((first, second)):
        for op in (ops.MODES["sum"], ops.MODES["max"]):
            want, got = launch_both(tables, ids, offs, dim, op, lib.BAG_XCD_TABLE_AFFINITY if call == 0 else 0)
            assert_bits_equal(got, want, "call %d op %d: no-allocation form against fwdmi_embedding_bag_multi" % (call, op))
            for t, tab in enumerate(tables):                                  # and both against the oracle
                ref, _, _ = oracle.embedding_bag(tab, ids[t], offs[t], op)
                assert_bits_equal(got[:, t * dim:(t + 1) * dim], ref, "call %d table %d against the oracle" % (call, t))


@pytest.mark.parametrize("affinity", [False, True])
def test_many_tables_of_very_different_bag_lengths_with_descriptors_in_device_memory(oracle, affinity):
    """48 tables, one-hot ones alternating with long-bag ones: more tables than travel with a launch, few
    enough for runs sized per table, so the kernel takes per-table run sizes while it reads its descriptors
    from device memory.  Through fwdmi_embedding_bag_multi_host with a caller's device array and through the
    no-allocation entry point, with and without the per-XCD mapping; whole output against the oracle."""
    rng = np.random.Generator(np.random.PCG64(48))
    n_tables, dim, n_bags = 48, 64, 6000
    rows = [int(v) for v in rng.integers(50, 30000, n_tables)]
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(np.float16) for r in rows]
    ids, offs = [], []
    for t, r in enumerate(rows):
        lengths = np.ones(n_bags, np.int64) if t % 2 == 0 else rng.poisson(45, n_bags)
        if t == 7:
            lengths[100:104] = 5000            # bags longer than the id window
            lengths[3::50] = 0
        offs.append(np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.int32))
        ids.append(rng.integers(0, r, int(lengths.sum())).astype(np.int32))
    want = np.zeros((n_bags, n_tables * dim), np.float16)
    for t in range(n_tables):
        oracle.embedding_bag(tables[t], ids[t], offs[t], oracle.OP_SUM, out=want, out_col=dim * t)
    d_tab, d_ids, d_off = [dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs]
    desc = descriptors(d_tab, d_ids, d_off, dim)
    avg = float(sum(i.size for i in ids)) / (n_tables * n_bags)
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    flags = lib.BAG_XCD_TABLE_AFFINITY if affinity else 0
    d_desc = torch.empty(n_tables * 64, dtype=torch.uint8, device="cuda")
    for name in ("host descriptors + device array", "no allocation"):
        out = torch.full((n_bags, n_tables * dim), -3.0, dtype=torch.float16, device="cuda")
        x = ops._ext(d_tab[0], d_ids[0], torch.float16, out_row_stride=n_tables * dim, flags=flags)
        if name == "no allocation":
            rc = lib.dll.fwdmi_embedding_bag_multi_noalloc(C.c_void_p(desc.ctypes.data), n_tables, n_bags,
                                                           C.c_void_p(out.data_ptr()), dim, 0, avg, C.byref(x), s)
        else:
            rc = lib.dll.fwdmi_embedding_bag_multi_host(C.c_void_p(desc.ctypes.data), n_tables,
                                                        C.c_void_p(d_desc.data_ptr()), n_bags,
                                                        C.c_void_p(out.data_ptr()), dim, 0, avg, C.byref(x), s)
        lib.check(rc)
        torch.cuda.synchronize()
        assert_bits_equal(host(out), want, "%s, affinity %s" % (name, affinity))


def test_no_alloc_entry_point_limits_and_argument_errors():
    dim, n_bags = 32, 10
    table, ids, off = dev(np.ones((8, dim), np.float32)), dev(np.zeros(10, np.int32)), dev(np.arange(10, dtype=np.int32))
    out = torch.zeros((n_bags, dim), dtype=torch.float32, device="cuda")
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    one = descriptors([table], [ids], [off], dim)
    call = lambda desc, n, stride=0: lib.dll.fwdmi_embedding_bag_multi_noalloc(
        C.c_void_p(desc.ctypes.data) if desc is not None else None, n, n_bags, C.c_void_p(out.data_ptr()), dim, 0, 1.0,
        C.byref(ops._ext(table, ids, torch.float32, out_row_stride=stride)), s)
    many = np.repeat(one, 1025, axis=0)
    assert call(many, 1025) == lib.ERR_BAD_ARG and "1024" in lib.last_error()
    assert call(None, 1) == lib.ERR_BAD_ARG
    assert call(one, 0) == lib.ERR_BAD_ARG
    bad = one.copy()
    bad[0, 6] = 8                                                            # column block leaves the output row
    assert call(bad, 1) == lib.ERR_BAD_ARG and "columns" in lib.last_error()
    bad = one.copy()
    bad[0, 0] = 0                                                            # rows but no data
    assert call(bad, 1) == lib.ERR_BAD_ARG
    assert call(one, 1) == lib.OK
    torch.cuda.synchronize()
    assert host(out).tolist() == [[1.0] * dim] * n_bags                      # ids are all 0, bags of one id
    # the limit itself works: 1024 descriptors of the same small table, column blocks side by side
    wide = torch.zeros((n_bags, 1024 * dim), dtype=torch.float32, device="cuda")
    full = np.repeat(one, 1024, axis=0)
    full[:, 6] = np.arange(1024) * dim
    rc = lib.dll.fwdmi_embedding_bag_multi_noalloc(C.c_void_p(full.ctypes.data), 1024, n_bags, C.c_void_p(wide.data_ptr()),
                                                   dim, 0, 1.0, C.byref(ops._ext(table, ids, torch.float32,
                                                                                  out_row_stride=1024 * dim)), s)
    assert rc == lib.OK, lib.last_error()
    torch.cuda.synchronize()
    assert bool((wide == 1.0).all())


def test_no_alloc_entry_point_on_config4_at_full_size():
    """The whole 26-table configuration (65536 bags per table, 8 GB of tables) through the
    no-allocation entry point equals the fused launch of fwdmi_embedding_bag_multi bit for bit."""
    from forward_amd import workloads
    wl = workloads.config4()
    tabs = [wl.device_table(t, torch) for t in range(26)]
    idx = [torch.from_numpy(i).cuda() for i in wl.indices]
    off = [torch.from_numpy(o).cuda() for o in wl.offsets]
    batch = ops.MultiTableBatch(tabs, idx, off)
    want = batch.forward(xcd_table_affinity=True)
    desc = batch.desc.cpu().numpy()
    got = torch.zeros_like(want)
    x = ops._ext(tabs[0], idx[0], torch.float16, out_row_stride=want.shape[1], flags=lib.BAG_XCD_TABLE_AFFINITY,
                 table_cost=batch.default_table_cost())
    lib.check(lib.dll.fwdmi_embedding_bag_multi_noalloc(C.c_void_p(desc.ctypes.data), 26, wl.n_bags,
                                                        C.c_void_p(got.data_ptr()), 128, 0,
                                                        wl.n_indices() / (26.0 * wl.n_bags), C.byref(x),
                                                        C.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("n_tables", [3, lib.BAG_INLINE_TABLES + 4])
def test_no_alloc_entry_point_under_graph_capture(oracle, n_tables):
    """The callers the entry point is for: recorded into a HIP graph (no allocation may happen
    there) and replayed with new ids in the same buffers, with eager calls of the same entry point
    between the replays (they share the built-in descriptor buffer, in stream order)."""
    rng = np.random.Generator(np.random.PCG64(31))
    rows, dim, n_bags, n_ids = ([700, 12000, 33] + [211 + 37 * t for t in range(n_tables)])[:n_tables], 64, 500, 6000
    tables = [(rng.standard_normal((r, dim)) * 0.3).astype(np.float16) for r in rows]
    d_tab = [dev(t) for t in tables]

    def batch(seed):
        r = np.random.Generator(np.random.PCG64(seed))
        ids, offs = [], []
        for rws in rows:
            cuts = np.sort(r.integers(0, n_ids + 1, n_bags - 1))
            offs.append(np.concatenate([[0], cuts]).astype(np.int32))          # fixed id count per table
            ids.append(r.integers(0, rws, n_ids).astype(np.int32))
        return ids, offs

    ids0, offs0 = batch(0)
    d_ids, d_off = [dev(i) for i in ids0], [dev(o) for o in offs0]
    desc = descriptors(d_tab, d_ids, d_off, dim)
    out = torch.zeros((n_bags, n_tables * dim), dtype=torch.float16, device="cuda")
    x = ops._ext(d_tab[0], d_ids[0], torch.float16, out_row_stride=n_tables * dim)

    def launch(dst):
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        lib.check(lib.dll.fwdmi_embedding_bag_multi_noalloc(C.c_void_p(desc.ctypes.data), n_tables, n_bags,
                                                            C.c_void_p(dst.data_ptr()), dim, 0, n_ids / float(n_bags),
                                                            C.byref(x), s))

    def want(ids, offs):
        return np.concatenate([oracle.embedding_bag(tables[t], ids[t], offs[t], 0)[0] for t in range(n_tables)], axis=1)

    launch(out)                                     # eager first: the buffer's address is looked up here
    torch.cuda.synchronize()
    assert_bits_equal(host(out), want(ids0, offs0), "eager")
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        launch(out)
    torch.cuda.synchronize()
    other = torch.zeros_like(out)
    for seed in (1, 2, 3):
        ids, offs = batch(seed)
        for t in range(n_tables):
            d_ids[t].copy_(dev(ids[t]))
            d_off[t].copy_(dev(offs[t]))
        out.fill_(-1.0)
        g.replay()
        torch.cuda.synchronize()
        assert_bits_equal(host(out), want(ids, offs), "replay %d" % seed)
        launch(other)                               # an eager call between the replays
        torch.cuda.synchronize()
        assert_bits_equal(host(other), want(ids, offs), "eager between replays %d" % seed)


def test_no_alloc_calls_from_several_host_threads_on_one_stream(oracle):
    """Four host threads issue calls of different table sets (each more tables than travel with a launch,
    so all go through the shared descriptor buffer) on ONE stream.  A call's descriptor writes and its
    launch are enqueued under one lock, so no thread's launch can read another's descriptors; every
    output is checked against the oracle."""
    import threading
    rng = np.random.Generator(np.random.PCG64(404))
    n_tables, dim, n_bags = lib.BAG_INLINE_TABLES + 3, 32, 300
    stream = torch.cuda.Stream()
    s = C.c_void_p(stream.cuda_stream)
    sets = []
    for k in range(4):
        tables, ids, offs = make_batch(rng, [int(v) for v in rng.integers(5, 400, n_tables)], n_bags, dim, np.float32,
                                       np.int32, 6)
        d_tab, d_ids, d_off = [dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs]
        want = np.concatenate([oracle.embedding_bag(tables[t], ids[t], offs[t], 0)[0] for t in range(n_tables)], axis=1)
        sets.append((d_tab, d_ids, d_off, descriptors(d_tab, d_ids, d_off, dim), want,
                     float(sum(i.size for i in ids)) / (n_tables * n_bags)))
    torch.cuda.synchronize()
    rounds = 25
    outs = [[torch.full((n_bags, n_tables * dim), -3.0, dtype=torch.float32, device="cuda") for _ in range(rounds)]
            for _ in range(4)]
    errors = []

    def work(k):
        try:
            d_tab, d_ids, _, desc, _, avg = sets[k]
            x = ops._ext(d_tab[0], d_ids[0], torch.float32, out_row_stride=n_tables * dim)
            for r in range(rounds):
                rc = lib.dll.fwdmi_embedding_bag_multi_noalloc(C.c_void_p(desc.ctypes.data), n_tables, n_bags,
                                                               C.c_void_p(outs[k][r].data_ptr()), dim, 0, avg, C.byref(x), s)
                if rc:
                    raise RuntimeError("call failed: %d" % rc)
        except Exception as e:       # pragma: no cover
            errors.append(e)

    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    stream.synchronize()
    assert not errors, errors
    for k in range(4):
        for r in range(rounds):
            assert_bits_equal(host(outs[k][r]), sets[k][4], "thread %d call %d" % (k, r))
