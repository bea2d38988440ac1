"""GPU parity of the bag-reduction kernels against the CPU oracle, through the C ABI
(kernel launchers and plugin objects).  Integer work (ids, argmax, empty bags) is bit-exact;
because rows are summed in bag order with the oracle's operations, fp32 and fp16 values are
bit-exact too, which is stricter than the stated tolerance (also asserted)."""
import numpy as np
import pytest
import torch

from forward_amd import lib, ops, plugin, workloads
from forward_amd.plugin import PluginFieldData as F
from gpu_util import assert_bits_equal, assert_close, dev, host

pytestmark = pytest.mark.gpu

OPS = {"sum": 0, "mean": 1, "max": 2, "square_sum": 3}


def run_bag(wl_table, idx, off, mode, psw=None, **kw):
    return ops.embedding_bag(dev(wl_table), dev(idx), dev(off), mode, per_sample_weights=dev(psw), **kw)


def test_config1_exact(oracle):
    wl = workloads.config1()
    got = host(run_bag(wl.table, wl.indices, wl.offsets, "sum"))
    want, _, _ = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, oracle.OP_SUM)
    assert_bits_equal(got, want, "config 1")
    ref = torch.nn.functional.embedding_bag(torch.from_numpy(wl.indices), torch.from_numpy(wl.table),
                                            torch.from_numpy(wl.offsets), mode="sum").numpy()
    assert_close(got, ref, np.float32)


@pytest.mark.parametrize("tdt", [np.float32, np.float16])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("mode", ["sum", "mean", "max", "wsum"])
def test_config2_scaled(oracle, tdt, idt, mode):
    weighted = mode == "wsum"
    m = "sum" if weighted else mode
    wl = workloads.config2(variant=1, table_dtype=tdt, index_dtype=idt, mode=m, weighted=weighted, rows=60000)
    assert (wl.lengths == 0).sum() > 10 and wl.lengths.max() > 30
    res = run_bag(wl.table, wl.indices, wl.offsets, m, wl.per_sample_weights, want_max_indices=(m == "max"))
    want, warg, oob = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, OPS[m],
                                           per_sample_weights=wl.per_sample_weights, want_max_indices=(m == "max"))
    assert oob == 0
    got = host(res[0] if m == "max" else res)
    assert got.dtype == tdt
    assert_close(got, want, tdt, scale=0.05)
    assert_bits_equal(got, want, "values")
    empty = wl.lengths == 0
    assert not got[empty].any()
    if m == "max":
        arg = host(res[1])
        assert arg.dtype == idt
        np.testing.assert_array_equal(arg, warg)
        # the plugin's form: values only (a kernel variant of its own, without the index registers)
        assert_bits_equal(host(run_bag(wl.table, wl.indices, wl.offsets, m)), want, "max, values only")


@pytest.mark.parametrize("tdt", [np.float32, np.float16])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("mode", ["sum", "mean", "max", "wsum"])
def test_config2_scaled_against_libtorch_cpu_itself(tdt, idt, mode):
    """The same launches against torch.nn.functional.embedding_bag on CPU tensors, run here and now (the
    ground truth the reference's unit tests use), without the oracle in between: values within the
    stated bar and in fact equal bit for bit, except the mean over an fp16 table (see below)."""
    weighted = mode == "wsum"
    m = "sum" if weighted else mode
    wl = workloads.config2(variant=2, table_dtype=tdt, index_dtype=idt, mode=m, weighted=weighted, rows=60000)
    psw = None if wl.per_sample_weights is None else torch.from_numpy(wl.per_sample_weights)
    try:
        ref = torch.nn.functional.embedding_bag(torch.from_numpy(wl.indices), torch.from_numpy(wl.table),
                                                torch.from_numpy(wl.offsets), mode=m, per_sample_weights=psw)
    except RuntimeError as e:   # a type / mode pair this libtorch build has no CPU kernel for
        pytest.skip("libtorch CPU: %s" % str(e).splitlines()[0])
    got = host(run_bag(wl.table, wl.indices, wl.offsets, m, wl.per_sample_weights))
    assert_close(got, ref.numpy(), tdt, scale=0.05)
    if mode == "mean" and tdt == np.float16:
        # libtorch's CPU kernel rounds the bag's sum to fp16 and divides that; the launch divides the fp32
        # sum and rounds once.  One fp16 unit apart at most, in about a quarter of the elements.
        a, b = got.view(np.int16).astype(np.int32), ref.numpy().view(np.int16).astype(np.int32)
        key = lambda v: np.where(v < 0, -(v & 0x7fff), v)     # fp16 bit patterns in value order
        assert np.abs(key(a) - key(b)).max() <= 1
    else:
        assert_bits_equal(got, ref.numpy(), "%s against libtorch CPU" % mode)


def test_max_ties_nan_and_empty_bags_match_libtorch_vectors(torch_vectors):
    """The committed libtorch CPU vectors (first maximum wins, NaN never replaces a value, a NaN
    first element stays, argmax is the row id, empty bags give 0 / 0) through the HIP path."""
    v = torch_vectors
    w, idx, off = v["tie_table"], v["tie_idx"], v["tie_off"]
    out, arg = run_bag(w, idx, off, "max", want_max_indices=True)
    assert_bits_equal(host(out), v["tie_max_out"], "max values")
    np.testing.assert_array_equal(host(arg), v["tie_max_arg"])
    assert_bits_equal(host(run_bag(w, idx, off, "max")), v["tie_max_out"], "max values, no indices")
    wq, ridx, roff = v["rnd_tableq"], v["rnd_idx"], v["rnd_off"]
    for i, o, key in ((ridx, roff, ""), (ridx.astype(np.int32), roff.astype(np.int32), "_i32")):
        out, arg = run_bag(wq, i, o, "max", want_max_indices=True)
        assert_bits_equal(host(out), v["rnd_max" + key], "max on the quantised table")
        np.testing.assert_array_equal(host(arg), v["rnd_max_arg" + key])
        assert_bits_equal(host(run_bag(wq, i, o, "max")), v["rnd_max" + key], "no indices")
    assert_bits_equal(host(run_bag(wq.astype(np.float16), ridx, roff, "max")), v["rnd_max_f16"], "fp16 max")


@pytest.mark.parametrize("tdt", [np.float32, np.float16])
def test_max_special_values_against_oracle(oracle, tdt):
    """Rows full of ties, signed zeros, infinities and NaN in every position of a bag."""
    rng = np.random.Generator(np.random.PCG64(404))
    specials = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 0.5, 2.0], np.float32)
    table = specials[rng.integers(0, specials.size, size=(300, 16))].astype(tdt)
    lengths = rng.integers(0, 12, size=500)
    off = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.int32)
    idx = rng.integers(0, 300, size=int(lengths.sum())).astype(np.int32)
    want, warg, _ = oracle.embedding_bag(table, idx, off, oracle.OP_MAX, want_max_indices=True)
    out, arg = run_bag(table, idx, off, "max", want_max_indices=True)
    assert_bits_equal(host(out), want, "values")
    np.testing.assert_array_equal(host(arg), warg)
    assert_bits_equal(host(run_bag(table, idx, off, "max")), want, "values, no indices")


def test_config2_full_size_sum_fp16(oracle):
    wl = workloads.config2(variant=0, table_dtype=np.float16, index_dtype=np.int32)
    assert wl.table.shape == (1_000_000, 128) and wl.n_bags == 4096
    got = host(run_bag(wl.table, wl.indices, wl.offsets, "sum"))
    want, _, _ = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, oracle.OP_SUM)
    assert_close(got, want, np.float16)
    assert_bits_equal(got, want, "config 2 fp16")


@pytest.fixture(scope="module")
def config2_full():
    """Config 2 at its real size, generated once: 1 000 000 x 128 fp32 table, 4096 bags, Zipf ids,
    per-sample weights.  The fp16 table is the rounded fp32 draw and the int64 ids are the int32
    ones widened, exactly as workloads.config2 makes them, so every variant shares this draw."""
    wl = workloads.config2(variant=0, table_dtype=np.float32, index_dtype=np.int32, weighted=True)
    assert wl.table.shape == (1_000_000, 128) and wl.n_bags == 4096 and (wl.lengths == 0).sum() > 10
    cache = {}

    def tables(tdt):
        if tdt not in cache:
            host_t = wl.table.astype(tdt)
            cache[tdt] = (host_t, dev(host_t))
        return cache[tdt]
    return wl, tables


@pytest.mark.parametrize("tdt", [np.float32, np.float16])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
@pytest.mark.parametrize("mode", ["sum", "mean", "max", "wsum"])
def test_config2_full_size_every_variant(oracle, config2_full, tdt, idt, mode):
    """Every table type x id type x mode of config 2 on the 1 M-row table, bit for bit against the
    oracle (values, argmax ids, empty bags)."""
    wl, tables = config2_full
    host_t, dev_t = tables(tdt)
    weighted = mode == "wsum"
    m = "sum" if weighted else mode
    idx, off = wl.indices.astype(idt), wl.offsets.astype(idt)
    psw = wl.per_sample_weights.astype(tdt) if weighted else None
    res = ops.embedding_bag(dev_t, dev(idx), dev(off), m, per_sample_weights=dev(psw), want_max_indices=(m == "max"))
    want, warg, oob = oracle.embedding_bag(host_t, idx, off, OPS[m], per_sample_weights=psw,
                                           want_max_indices=(m == "max"))
    assert oob == 0
    got = host(res[0] if m == "max" else res)
    assert got.dtype == tdt and got.shape == (4096, 128)
    assert_close(got, want, tdt, scale=0.05)
    assert_bits_equal(got, want, "config 2 %s %s %s" % (np.dtype(tdt).name, np.dtype(idt).name, mode))
    assert not got[wl.lengths == 0].any()
    if m == "max":
        arg = host(res[1])
        assert arg.dtype == idt
        np.testing.assert_array_equal(arg, warg)
        assert_bits_equal(host(ops.embedding_bag(dev_t, dev(idx), dev(off), m)), want, "max, values only")


@pytest.mark.parametrize("dim,tdt", [(1, np.float32), (2, np.float32), (4, np.float32), (10, np.float16),
                                     (64, np.float32), (100, np.float16), (200, np.float32), (1024, np.float16),
                                     (1100, np.float32), (2048, np.float32)])
def test_row_widths(oracle, dim, tdt):
    rng = np.random.Generator(np.random.PCG64(dim))
    table = rng.standard_normal((300, dim)).astype(tdt)
    lengths = rng.integers(0, 12, size=97)
    idx = rng.integers(0, 300, size=int(lengths.sum())).astype(np.int32)
    off = workloads.offsets_from_lengths(lengths, np.int32)
    for mode in ("sum", "max"):
        got = host(run_bag(table, idx, off, mode))
        want, _, _ = oracle.embedding_bag(table, idx, off, OPS[mode])
        assert_bits_equal(got, want, "dim %d %s" % (dim, mode))


def test_long_bags_exceed_lds_window(oracle):
    rng = np.random.Generator(np.random.PCG64(77))
    table = rng.standard_normal((4000, 128)).astype(np.float16)
    lengths = np.array([0, 5000, 1, 2047, 2049, 0, 9000, 3], np.int64)
    idx = rng.integers(0, 4000, size=int(lengths.sum())).astype(np.int64)
    off = workloads.offsets_from_lengths(lengths, np.int64)
    psw = rng.random(idx.size).astype(np.float16)
    for mode, w in (("sum", None), ("mean", None), ("max", None), ("sum", psw)):
        got = host(run_bag(table, idx, off, mode, w))
        want, _, _ = oracle.embedding_bag(table, idx, off, OPS[mode], per_sample_weights=w)
        assert_bits_equal(got, want, "long bags %s" % mode)


def test_out_of_range_ids_are_skipped_and_flagged(oracle):
    table = (np.arange(40, dtype=np.float32).reshape(10, 4) + 1)
    idx = np.array([100, 103, 99, 110, 109, -1, 2**31 - 1, 105], np.int32)      # shard holds ids 100..109
    off = np.array([0, 3, 3], np.int32)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    got = host(run_bag(table, idx, off, "sum", data_offset=100, oob_flag=flag))
    want, _, oob = oracle.embedding_bag(table, idx, off, oracle.OP_SUM, data_offset=100)
    assert oob == 4
    assert_bits_equal(got, want, "filtered")
    assert int(flag.item()) == 1
    flag.zero_()
    run_bag(table, np.array([100, 109], np.int32), np.array([0], np.int32), "sum", data_offset=100, oob_flag=flag)
    assert int(flag.item()) == 0
    # 64-bit ids far outside the table
    idx64 = np.array([5, 2**40, -2**40, 9], np.int64)
    got = host(run_bag(table, idx64, np.array([0], np.int64), "sum"))
    np.testing.assert_array_equal(got[0], table[5] + table[9])


def test_include_last_offset_and_empty_batches(oracle):
    wl = workloads.config2(variant=4, rows=3000, n_bags=50)
    off_last = np.append(wl.offsets, wl.indices.size).astype(np.int32)
    a = host(run_bag(wl.table, wl.indices, wl.offsets, "sum"))
    b = host(run_bag(wl.table, wl.indices, off_last, "sum", include_last_offset=True))
    assert_bits_equal(a, b, "include_last_offset")
    # all bags empty / no ids at all
    z = host(run_bag(wl.table, np.zeros(0, np.int32), np.zeros(7, np.int32), "max"))
    assert z.shape == (7, 128) and not z.any()
    # zero bags: nothing launched, nothing written
    e = ops.embedding_bag(dev(wl.table), dev(np.zeros(0, np.int32)), dev(np.zeros(0, np.int32)), "sum")
    assert e.shape == (0, 128)


def test_fixed_length_square_sum_and_gather(oracle):
    rng = np.random.Generator(np.random.PCG64(21))
    table = rng.standard_normal((50, 6)).astype(np.float32)
    idx = rng.integers(0, 50, size=(10, 5)).astype(np.int32)                   # test_tf_nodes.h:199-211 shape
    for mode in ("sum", "square_sum", "mean", "max"):
        got = host(ops.embedding_bag_fixed(dev(table), dev(idx), mode))
        want, _, _ = oracle.embedding_bag(table, idx, None, OPS[mode])
        assert_bits_equal(got, want, "fixed %s" % mode)
    g = host(ops.gather(dev(table), dev(idx)))
    want, _ = oracle.gather(table, idx)
    assert_bits_equal(g, want, "gather")
    big = rng.standard_normal((1000, 128)).astype(np.float16)
    ids = rng.integers(-3, 1003, size=(1, 1000)).astype(np.int64)
    g = host(ops.gather(dev(big), dev(ids), out_dtype=torch.float32))
    want, oob = oracle.gather(big, ids, out_dtype=np.float32)
    assert oob > 0
    assert_bits_equal(g, want, "gather fp16->fp32")


def test_multi_table_concatenated(oracle):
    wl = workloads.config4(variant=2, n_tables=5, n_bags=3000, max_rows=30000)
    tabs = [wl.host_table(t) for t in range(5)]
    want = np.zeros((3000, 5 * 128), np.float16)
    for t in range(5):
        oracle.embedding_bag(tabs[t], wl.indices[t], wl.offsets[t], oracle.OP_SUM, out=want, out_col=128 * t)
    batch = ops.MultiTableBatch([dev(t) for t in tabs], [dev(i) for i in wl.indices], [dev(o) for o in wl.offsets])
    got = host(batch.forward())
    assert_bits_equal(got, want, "fused multi-table")
    # the same through 5 single-table launches writing column blocks
    out = torch.zeros((3000, 640), dtype=torch.float16, device="cuda")
    for t in range(5):
        ops.embedding_bag(batch.tables[t], batch.indices[t], batch.offsets[t], "sum", out=out, out_col=128 * t)
    assert_bits_equal(host(out), want, "per-table launches")
    assert_bits_equal(host(batch.forward(xcd_table_affinity=True)), want, "fused, per-XCD table affinity")
    # the XCD segmentation may cut the work list anywhere: every bag is still reduced exactly once
    for cost in ([1, 1, 1, 1, 1], [1e-3, 1, 1e3, 1, 1e-3], [1e6, 1, 1, 1, 1], [1, 1, 1, 1, 1e6], [3, 1, 4, 1, 5]):
        out = torch.full((3000, 640), 7.0, dtype=torch.float16, device="cuda")
        batch.forward(out=out, xcd_table_affinity=True, table_cost=np.array(cost, np.float32))
        assert_bits_equal(host(out), want, "XCD segments for cost %r" % (cost,))
    with pytest.raises(lib.FwdmiError, match="table_cost"):
        batch.forward(xcd_table_affinity=True, table_cost=np.array([1, 1, 0, 1, 1], np.float32))
    got32 = host(batch.forward(out_dtype=torch.float32))
    np.testing.assert_allclose(got32, want.astype(np.float32), atol=1e-2, rtol=5e-3)


# ---- through the plugin objects ------------------------------------------------------------------
REG = plugin.getPluginRegistry()


def bag_fields(table, op=0, offset=0):
    count, dim = table.shape
    return [F("dim", dim), F("count", count), F("offset", offset), F("op", op), F("data", table)]


def test_plugin_reference_known_answers(kats):
    k = kats["embedding_bag_module"]
    w = np.array(k["table"], np.float32)
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    p = c.createPlugin("embedding_bag", bag_fields(w))
    # the reference engine feeds int64 ids as int32 (torch_engine.cpp:134-149)
    out = host(p(dev(np.array(k["indices"], np.int32)), dev(np.array(k["offsets"], np.int32))))
    want = np.zeros((5, 4))
    want[4] = (w[0].astype(np.float64) + 2 * w[1].astype(np.float64) + w[3] + w[4])
    np.testing.assert_allclose(out, want, atol=1e-3)           # the reference test's threshold
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-7)
    assert not out[:4].any()

    d = kats["dlrm"]
    expect = [[[0.48071694, 0.18480009], [0.41585842, -0.29087239]],
              [[-0.18103497, 0.26449448], [-0.25194445, -0.24395032]],
              [[-0.44896644, -0.45899662], [-0.44896644, -0.45899662]]]
    for t in range(3):
        tab = np.array(d["tables"][t], np.float32)
        q = c.createPlugin("emb_%d" % t, bag_fields(tab))
        off = np.array(d["offsets"][t], np.int32).reshape(1, 2)          # DLRM passes a [1, B] slice
        out = host(q(dev(np.array(d["indices"][t], np.int32)), dev(off)))
        np.testing.assert_allclose(out, expect[t], atol=1e-4)           # test_torch_dlrm.h:56
        np.testing.assert_allclose(out, expect[t], rtol=1e-6, atol=1e-7)


def test_plugin_serialize_load_run_matches(oracle):
    """Build -> save -> load -> run, as the reference's test harness does (unit_test_torch_helper.h:79-138)."""
    wl = workloads.config1()
    idx, off = wl.indices.astype(np.int32), wl.offsets.astype(np.int32)
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    p = c.createPlugin("embedding_bag", bag_fields(wl.table))
    direct = host(p(dev(idx), dev(off)))
    loaded = c.deserializePlugin("embedding_bag", p.serialize())
    again = host(loaded(dev(idx), dev(off)))
    clone = loaded.clone()
    third = host(clone(dev(idx), dev(off)))
    want, _, _ = oracle.embedding_bag(wl.table, idx, off, oracle.OP_SUM)
    for got in (direct, again, third):
        assert_bits_equal(got, want, "plugin")
    loaded.destroy()                     # the clone keeps the shared device table alive
    assert_bits_equal(host(clone(dev(idx), dev(off))), want, "clone after destroy")
    # wrong id type is refused with -1, as in the reference
    rc = p.enqueue_raw([((idx.size,), lib.I64), ((64,), lib.I64)], [((64, 64), lib.F32)], [0, 0], [0])
    assert rc == lib.ERR_UNSUPPORTED
    # shapes the plugin's own shape rules never produce are refused before any launch
    rc = p.enqueue_raw([((4, 4, 4), lib.I32)], [((4, 64), lib.F32)], [0], [0])
    assert rc == lib.ERR_BAD_ARG and "1-D or 2-D" in lib.last_error()
    rc = p.enqueue_raw([((idx.size,), lib.I32), ((2, 32), lib.I32)], [((64, 64), lib.F32)], [0, 0], [0])
    assert rc == lib.ERR_BAD_ARG and "offsets" in lib.last_error()


def test_plugin_modes_fixed_gather_and_extended(oracle):
    rng = np.random.Generator(np.random.PCG64(31))
    table = rng.standard_normal((50, 8)).astype(np.float32)
    idx2d = rng.integers(0, 50, size=(10, 5)).astype(np.int32)
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    for op in (0, 3):                                               # SUM and SQUARE_SUM: what the TF front end emits
        got = host(c.createPlugin("fm", bag_fields(table, op=op))(dev(idx2d)))
        want, _, _ = oracle.embedding_bag(table, idx2d, None, op)
        assert_bits_equal(got, want, "fixed op %d" % op)
    g = host(c.createPlugin("gather", bag_fields(table, op=999))(dev(idx2d)))
    assert g.shape == (10, 5, 8)
    assert_bits_equal(g, table[idx2d], "plugin gather")
    # torch mode ints 1 / 2 mean MEAN / MAX
    wl = workloads.config2(variant=5, rows=2000, n_bags=200)
    for op in (1, 2):
        got = host(c.createPlugin("bag", bag_fields(wl.table, op=op))(dev(wl.indices), dev(wl.offsets)))
        want, _, _ = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, op)
        assert_bits_equal(got, want, "plugin op %d" % op)
    # extended contract: fp16 table, int64 ids, fp16 output, per-sample weights, trailing offset
    c2 = REG.getPluginCreator("EmbeddingBag_TRT", "002")
    t16 = wl.table.astype(np.float16)
    psw = rng.random(wl.indices.size).astype(np.float16)
    p = c2.createPlugin("bag", bag_fields(t16) + [F("index_type", lib.I64), F("output_fp16", 1),
                                                  F("include_last_offset", 1), F("per_sample_weights", 1)])
    i64 = wl.indices.astype(np.int64)
    o64 = np.append(wl.offsets, wl.indices.size).astype(np.int64)
    got = host(p(dev(i64), dev(o64), dev(psw)))
    want, _, _ = oracle.embedding_bag(t16, i64, o64, 0, per_sample_weights=psw, include_last_offset=True)
    assert got.dtype == np.float16 and got.shape == (200, 128)
    assert_bits_equal(got, want, "extended plugin")
    assert not p.takeOobFlag()


def test_large_tables_and_offsets_take_the_wide_address_path(oracle):
    """int32 ids normally use 24-bit row arithmetic; these shapes must fall back to 64-bit:
    more than 2^24 rows, a table larger than 4 GiB, a negative data_offset, ids near 2^31."""
    rng = np.random.Generator(np.random.PCG64(91))
    rows = (1 << 24) + 4096                                        # > 2^24 rows of 16 bytes
    table = torch.empty((rows, 8), dtype=torch.float16, device="cuda")
    table.copy_(((torch.arange(rows, device="cuda") % 2039).float() / 64).unsqueeze(1)
                + torch.arange(8, device="cuda").float() / 512)
    lengths = rng.integers(0, 7, 200)
    idx = rng.integers(rows - 5000, rows, int(lengths.sum())).astype(np.int32)   # the top of the table
    idx[::3] = rng.integers(0, 1000, idx[::3].size)
    off = workloads.offsets_from_lengths(lengths, np.int32)
    got = host(ops.embedding_bag(table, dev(idx), dev(off), "sum"))
    uniq, inv = np.unique(idx, return_inverse=True)
    sub = host(table[torch.from_numpy(uniq.astype(np.int64)).cuda()])
    want, _, _ = oracle.embedding_bag(sub, inv.astype(np.int32), off, oracle.OP_SUM)
    assert_bits_equal(got, want, "2^24+ rows")
    # the same with int64 ids: the id window then holds 64-bit ids instead of 32-bit row numbers
    got = host(ops.embedding_bag(table, dev(idx.astype(np.int64)), dev(off.astype(np.int64)), "sum"))
    assert_bits_equal(got, want, "2^24+ rows, int64 ids")
    # and inside a multi-table launch, which sizes its runs for row numbers: the large table's
    # runs do not fit the window as 64-bit ids and read their ids from global memory instead
    n_bags = 3000
    lens2 = rng.integers(10, 30, n_bags)
    off2 = workloads.offsets_from_lengths(lens2, np.int64)
    idx_big = rng.integers(rows - 5000, rows, int(lens2.sum())).astype(np.int64)
    small_t = (rng.standard_normal((500, 8)) * 0.25).astype(np.float16)
    idx_small = rng.integers(0, 500, int(lens2.sum())).astype(np.int64)
    batch = ops.MultiTableBatch([dev(small_t), table], [dev(idx_small), dev(idx_big)], [dev(off2), dev(off2)])
    got = host(batch.forward())
    want_small, _, _ = oracle.embedding_bag(small_t, idx_small, off2, oracle.OP_SUM)
    uniq, inv = np.unique(idx_big, return_inverse=True)
    sub = host(table[torch.from_numpy(uniq).cuda()])
    want_big, _, _ = oracle.embedding_bag(sub, inv.astype(np.int64), off2, oracle.OP_SUM)
    assert_bits_equal(got[:, :8], want_small, "multi-table, small table")
    assert_bits_equal(got[:, 8:], want_big, "multi-table, 2^24+ rows with int64 ids")
    del table, batch

    big_rows = 2_200_000                                           # 2.2 M rows x 2 KiB = 4.5 GB > 4 GiB
    big = torch.empty((big_rows, 512), dtype=torch.float32, device="cuda")
    big.copy_((torch.arange(big_rows, device="cuda") % 4093).float().unsqueeze(1) / 8
              + torch.arange(512, device="cuda").float() / 1024)
    idx = rng.integers(big_rows - 3000, big_rows, int(lengths.sum())).astype(np.int32)
    got = host(ops.embedding_bag(big, dev(idx), dev(off), "sum"))
    uniq, inv = np.unique(idx, return_inverse=True)
    sub = host(big[torch.from_numpy(uniq.astype(np.int64)).cuda()])
    want, _, _ = oracle.embedding_bag(sub, inv.astype(np.int32), off, oracle.OP_SUM)
    assert_bits_equal(got, want, "table beyond 4 GiB")
    del big

    small = rng.standard_normal((64, 16)).astype(np.float32)
    for data_offset in (-20, 2**31 - 40):                          # id range leaves [0, 2^31)
        ids = (rng.integers(0, 64, 300) + data_offset).astype(np.int64)
        ids[::7] = data_offset - 1                                 # just below the shard: skipped
        ids32 = np.clip(ids, -2**31, 2**31 - 1).astype(np.int32)
        o = workloads.offsets_from_lengths(np.full(30, 10), np.int32)
        got = host(ops.embedding_bag(dev(small), dev(ids32), dev(o), "sum", data_offset=data_offset))
        want, _, oob = oracle.embedding_bag(small, ids32, o, oracle.OP_SUM, data_offset=data_offset)
        assert oob > 0
        assert_bits_equal(got, want, "data_offset %d" % data_offset)


def test_malformed_offsets_stay_in_bounds():
    """Offsets that decrease, exceed the id count or are negative are clamped; nothing is read or
    written out of bounds and well-formed bags of the same batch are still right."""
    rng = np.random.Generator(np.random.PCG64(92))
    table = rng.standard_normal((100, 32)).astype(np.float32)
    idx = rng.integers(0, 100, 50).astype(np.int32)
    off = np.array([0, 10, 5, 20, 1000, -7, 30, 40], np.int32)     # bag 1 "ends" before it starts, etc.
    guard = torch.full((8 + 2, 32), 123.0, device="cuda")
    out = guard[1:9]
    ops.embedding_bag(dev(table), dev(idx), dev(off), "sum", out=out)
    torch.cuda.synchronize()
    got = guard.cpu().numpy()
    assert (got[0] == 123.0).all() and (got[9] == 123.0).all()     # rows around the output untouched
    np.testing.assert_allclose(got[1], table[idx[0:10]].sum(0), rtol=1e-5, atol=1e-5)   # bag 0 = ids 0..10
    np.testing.assert_array_equal(got[2], 0.0)                                         # 10..5 -> empty
    np.testing.assert_allclose(got[3], table[idx[5:20]].sum(0), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[4], table[idx[20:50]].sum(0), rtol=1e-5, atol=1e-5)  # 20..1000 -> 20..50
    np.testing.assert_array_equal(got[5], 0.0)                                         # 50..0 -> empty
    np.testing.assert_allclose(got[6], table[idx[0:30]].sum(0), rtol=1e-5, atol=1e-5)   # -7 -> 0
    np.testing.assert_allclose(got[8], table[idx[40:50]].sum(0), rtol=1e-5, atol=1e-5)  # last bag runs to the end
    assert np.isfinite(got).all()


def test_concurrent_enqueue_from_threads_on_their_own_streams(oracle):
    """enqueue is re-entrant across plugin instances and stream-ordered: four host threads, each
    with its own stream and its own clone of one plugin, interleave launches."""
    import threading
    wl = workloads.config2(variant=12, rows=8000, n_bags=1500)
    want, _, _ = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, oracle.OP_SUM)
    c = REG.getPluginCreator("EmbeddingBag_TRT", "001")
    base = c.createPlugin("embedding_bag", bag_fields(wl.table))
    idx, off = dev(wl.indices), dev(wl.offsets)
    io_in = [((wl.indices.size,), lib.I32), ((wl.n_bags,), lib.I32)]
    io_out = [((wl.n_bags, 128), lib.F32)]
    base.configurePlugin(io_in, io_out)
    results, errors = {}, []

    def work(k):
        try:
            p = base.clone()
            p.configurePlugin(io_in, io_out)
            s = torch.cuda.Stream()
            outs = [torch.empty((wl.n_bags, 128), device="cuda") for _ in range(10)]
            for o in outs:
                p.enqueue([idx, off], [o], stream=s)
            s.synchronize()
            results[k] = [host(o) for o in outs]
            p.destroy()
        except Exception as e:       # pragma: no cover
            errors.append(e)

    torch.cuda.synchronize()
    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for k in range(4):
        for got in results[k]:
            assert_bits_equal(got, want, "thread %d" % k)


@pytest.mark.parametrize("tdt,idt", [(np.float32, np.int32), (np.float16, np.int64), (np.float16, np.int32)])
def test_sum_and_square_sum_in_one_pass(oracle, tdt, idt):
    """The two reductions of a factorisation-machine term (the reference builds them as two plugins,
    op 0 and op 3, over the same ids): one pass writes both, each bit-identical to its own launch."""
    rng = np.random.Generator(np.random.PCG64(55))
    for dim in (8, 64, 100, 128, 520):
        table = (rng.standard_normal((3000, dim)) * 0.5).astype(tdt)
        ids2d = rng.integers(-2, 3002, (400, 13)).astype(idt)            # a few ids outside the table
        s, q = ops.embedding_bag_fixed(dev(table), dev(ids2d), "sum", with_square_sum=True)
        ws, _, _ = oracle.embedding_bag(table, ids2d, None, oracle.OP_SUM)
        wq, _, _ = oracle.embedding_bag(table, ids2d, None, oracle.OP_SQUARE_SUM)
        assert_bits_equal(host(s), ws, "sums, dim %d" % dim)
        assert_bits_equal(host(q), wq, "sums of squares, dim %d" % dim)
        lengths = rng.integers(0, 30, 500)
        off = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt)
        ids = rng.integers(0, 3000, int(lengths.sum())).astype(idt)
        s, q = ops.embedding_bag(dev(table), dev(ids), dev(off), "sum", with_square_sum=True, out_dtype=torch.float32)
        ws, _, _ = oracle.embedding_bag(table, ids, off, oracle.OP_SUM, out_dtype=np.float32)
        wq, _, _ = oracle.embedding_bag(table, ids, off, oracle.OP_SQUARE_SUM, out_dtype=np.float32)
        assert_bits_equal(host(s), ws, "offsets form, sums, dim %d" % dim)
        assert_bits_equal(host(q), wq, "offsets form, sums of squares, dim %d" % dim)
    with pytest.raises(lib.FwdmiError, match="square_sum_out"):
        ops.embedding_bag_fixed(dev(table), dev(ids2d), "max", with_square_sum=True)

    # through the plugin: "002" with with_square_sum has two outputs
    c2 = REG.getPluginCreator("EmbeddingBag_TRT", "002")
    table = (rng.standard_normal((50, 8)) * 0.5).astype(np.float32)
    ids2d = rng.integers(0, 50, (10, 5)).astype(np.int32)                # the shape of the reference's TF test
    p = c2.createPlugin("fm", bag_fields(table) + [F("with_square_sum", 1)])
    assert p.getNbOutputs() == 2 and p.getOutputDimensions(1, [(10, 5)]) == [10, 8]
    s, q = p(dev(ids2d))
    assert_bits_equal(host(s), oracle.embedding_bag(table, ids2d, None, 0)[0], "plugin sums")
    assert_bits_equal(host(q), oracle.embedding_bag(table, ids2d, None, 3)[0], "plugin sums of squares")
    s2, q2 = c2.deserializePlugin("fm", p.serialize())(dev(ids2d))
    assert torch.equal(s, s2) and torch.equal(q, q2)
    with pytest.raises(lib.FwdmiError, match="with_square_sum"):
        c2.createPlugin("fm", bag_fields(table, op=3) + [F("with_square_sum", 1)])


@pytest.mark.parametrize("tdt", [np.float32, np.float16])
@pytest.mark.parametrize("odt", [np.float32, np.float16])
def test_results_large_enough_for_streaming_stores(oracle, tdt, odt):
    """Results of 8 MiB and more are written with non-temporal stores of 8, 16 or 32 bytes per
    lane (table type x result type); plain bags, a column block of a wider matrix, max mode and the
    two-output form all take that path here and must equal the oracle bit for bit."""
    rng = np.random.Generator(np.random.PCG64(88))
    rows, dim, n_bags = 3000, 128, 70000
    table = (rng.standard_normal((rows, dim)) * 0.5).astype(tdt)
    lengths = rng.integers(0, 4, n_bags)
    idx = rng.integers(0, rows, int(lengths.sum())).astype(np.int32)
    off = workloads.offsets_from_lengths(lengths, np.int32)
    tod = torch.float16 if odt == np.float16 else torch.float32
    assert n_bags * dim * np.dtype(odt).itemsize >= 8 << 20
    for mode in ("sum", "max"):
        want, _, _ = oracle.embedding_bag(table, idx, off, OPS[mode], out_dtype=odt)
        got = host(ops.embedding_bag(dev(table), dev(idx), dev(off), mode, out_dtype=tod))
        assert_bits_equal(got, want, "%s" % mode)
    wide = torch.full((n_bags, 3 * dim), 5.0, dtype=tod, device="cuda")
    ops.embedding_bag(dev(table), dev(idx), dev(off), "sum", out_dtype=tod, out=wide, out_col=dim)
    w = host(wide)
    want, _, _ = oracle.embedding_bag(table, idx, off, OPS["sum"], out_dtype=odt)
    assert_bits_equal(w[:, dim:2 * dim], want, "column block")
    assert (w[:, :dim] == 5.0).all() and (w[:, 2 * dim:] == 5.0).all()
    s1, s2 = ops.embedding_bag(dev(table), dev(idx), dev(off), "sum", out_dtype=tod, with_square_sum=True)
    want2, _, _ = oracle.embedding_bag(table, idx, off, OPS["square_sum"], out_dtype=odt)
    assert_bits_equal(host(s1), want, "sum of the two-output form")
    assert_bits_equal(host(s2), want2, "square sum of the two-output form")


@pytest.mark.parametrize("dim", [8, 16, 32, 64, 72, 200, 256, 512, 1024, 2048])
def test_fp32_results_of_fp16_tables_at_every_slot_width(oracle, dim):
    """Eight fp32 results per lane leave in two 16-byte stores; where every column slice is full
    (row widths of 2 .. 64 lanes, and 2048 columns in four slices) the lanes of a slot trade
    halves first so that each store writes contiguous bytes, elsewhere (8, 72, 200 columns) they
    store what they hold.  Large results (the streaming form), sum, mean and max, a column block
    of a wider matrix: bit-exact against the oracle."""
    rng = np.random.Generator(np.random.PCG64(dim))
    rows = 2000
    n_bags = max(4099, (8 << 20) // (dim * 4) + 3)
    table = (rng.standard_normal((rows, dim)) * 0.5).astype(np.float16)
    lengths = rng.integers(0, 4, n_bags)
    lengths[::1000] = 40
    idx = rng.integers(0, rows, int(lengths.sum())).astype(np.int32)
    off = workloads.offsets_from_lengths(lengths, np.int32)
    assert n_bags * dim * 4 >= 8 << 20
    for mode in ("sum", "mean", "max"):
        want, _, _ = oracle.embedding_bag(table, idx, off, OPS[mode], out_dtype=np.float32)
        got = host(ops.embedding_bag(dev(table), dev(idx), dev(off), mode, out_dtype=torch.float32))
        assert_bits_equal(got, want, "%s, %d columns" % (mode, dim))
    wide = torch.full((n_bags, dim + 8), 5.0, dtype=torch.float32, device="cuda")
    ops.embedding_bag(dev(table), dev(idx), dev(off), "sum", out_dtype=torch.float32, out=wide, out_col=4)
    w = host(wide)
    want, _, _ = oracle.embedding_bag(table, idx, off, OPS["sum"], out_dtype=np.float32)
    assert_bits_equal(w[:, 4:4 + dim], want, "column block")
    assert (w[:, :4] == 5.0).all() and (w[:, 4 + dim:] == 5.0).all()


@pytest.mark.parametrize("tdt,idt", [(np.float16, np.int32), (np.float32, np.int64)])
def test_ids_and_weights_at_every_alignment(oracle, tdt, idt):
    """A run's ids and weights are staged with 16-byte loads between the first and the last 16-byte
    boundary and one by one outside them: id and weight arrays that start 0 .. 3 (ids) and 0 .. 7
    (fp16 weights) elements past a 16-byte boundary, runs long enough for the wide loads, bit-exact
    for sum and for weighted sum.  The elements before and behind the arrays hold ids outside the
    table and NaN weights: reading one would raise the flag or poison a bag."""
    rng = np.random.Generator(np.random.PCG64(515))
    rows, dim, n_bags = 5000, 64, 90000      # runs of some 80 bags, 1500 ids
    table = (rng.standard_normal((rows, dim)) * 0.3).astype(tdt)
    lengths = rng.integers(0, 40, n_bags)
    n = int(lengths.sum())
    off = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(idt)
    ids = rng.integers(0, rows, n).astype(idt)
    psw = rng.random(n).astype(tdt)
    want, _, _ = oracle.embedding_bag(table, ids, off, oracle.OP_SUM)
    want_w, _, _ = oracle.embedding_bag(table, ids, off, oracle.OP_SUM, per_sample_weights=psw)
    d_tab, d_off = dev(table), dev(off)
    for shift in range(16 // ids.itemsize):
        for wshift in sorted({0, 1, 16 // psw.itemsize - 1, shift}):
            pad_i = np.full(n + 16, rows + 7, idt)
            pad_i[shift:shift + n] = ids
            pad_w = np.full(n + 16, np.nan, tdt)
            pad_w[wshift:wshift + n] = psw
            d_ids, d_w = dev(pad_i)[shift:shift + n], dev(pad_w)[wshift:wshift + n]
            assert d_ids.data_ptr() % 16 == (shift * ids.itemsize) % 16
            flag = torch.zeros(1, dtype=torch.int32, device="cuda")
            got = ops.embedding_bag(d_tab, d_ids, d_off, "sum", oob_flag=flag)
            assert_bits_equal(host(got), want, "ids %d elements past a 16-byte boundary" % shift)
            got = ops.embedding_bag(d_tab, d_ids, d_off, "sum", per_sample_weights=d_w, oob_flag=flag)
            assert_bits_equal(host(got), want_w, "ids +%d, weights +%d elements" % (shift, wshift))
            assert int(flag.item()) == 0
