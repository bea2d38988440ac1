"""Pins the CPU oracle's bag reductions: reference-held known answers, libtorch CPU vectors,
an independent numpy evaluation, and the fp16 conversion it relies on.  CPU only."""
import numpy as np
import pytest
import torch

from forward_amd import workloads


def test_half_conversion_exhaustive(oracle):
    # every binary16 bit pattern widens exactly as numpy does
    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    np.testing.assert_array_equal(oracle.half_to_float(h).view(np.uint32), h.astype(np.float32).view(np.uint32))


def test_float_to_half_matches_numpy_rne(oracle):
    rng = np.random.Generator(np.random.PCG64(7))
    f = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  2.9802326e-8, 6.1e-5, 6.097e-5, 1.0009765625, 1.00048828125, 1.00146484375], np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16)
    got = oracle.float_to_half(f)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    # halfway cases between neighbouring halves round to even
    h = np.arange(0x0001, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = (h[:-1] + h[1:]) / np.float32(2)
    np.testing.assert_array_equal(oracle.float_to_half(mid).view(np.uint16), mid.astype(np.float16).view(np.uint16))


def test_reference_kat_embedding_bag_module(oracle, kats):
    k = kats["embedding_bag_module"]
    w = np.array(k["table"], np.float32)
    idx, off = np.array(k["indices"], np.int64), np.array(k["offsets"], np.int64)
    out, _, oob = oracle.embedding_bag(w, idx, off, oracle.OP_SUM)
    w64 = w.astype(np.float64)
    want = np.zeros((5, 4))
    want[4] = w64[0] + 2 * w64[1] + w64[3] + w64[4]     # four empty bags, then all five ids
    assert oob == 0
    np.testing.assert_array_equal(out[:4], 0.0)
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(out[4], [-0.3134234, 0.5408130, -0.3899653, -0.6921769], rtol=2e-6)
    # same ids as int32 give the same bits
    out32, _, _ = oracle.embedding_bag(w, idx.astype(np.int32), off.astype(np.int32), oracle.OP_SUM)
    np.testing.assert_array_equal(out, out32)


def test_reference_kat_dlrm(oracle, kats):
    k = kats["dlrm"]
    want = [[[0.48071694, 0.18480009], [0.41585842, -0.29087239]],
            [[-0.18103497, 0.26449448], [-0.25194445, -0.24395032]],
            [[-0.44896644, -0.45899662], [-0.44896644, -0.45899662]]]
    for t in range(3):
        w = np.array(k["tables"][t], np.float32)
        idx, off = np.array(k["indices"][t], np.int64), np.array(k["offsets"][t], np.int64)
        out, _, _ = oracle.embedding_bag(w, idx, off, oracle.OP_SUM)
        np.testing.assert_allclose(out, want[t], rtol=1e-6, atol=1e-7)
        # bag 0 = first id, bag 1 = the rest (the last bag runs to the end of the ids)
        np.testing.assert_allclose(out[1], w.astype(np.float64)[idx[1:]].sum(0), rtol=1e-6, atol=1e-7)


def test_torch_vectors_ties_nan_empty(oracle, torch_vectors):
    v = torch_vectors
    w, idx, off = v["tie_table"], v["tie_idx"], v["tie_off"]
    out, arg, _ = oracle.embedding_bag(w, idx, off, oracle.OP_MAX, want_max_indices=True)
    np.testing.assert_array_equal(out.view(np.uint32), v["tie_max_out"].view(np.uint32))   # bit-exact incl. NaN
    np.testing.assert_array_equal(arg, v["tie_max_arg"])
    mean, _, _ = oracle.embedding_bag(w, idx, off, oracle.OP_MEAN)
    np.testing.assert_allclose(mean, v["tie_mean_out"], rtol=1e-6, equal_nan=True)
    s, _, _ = oracle.embedding_bag(w, idx, off, oracle.OP_SUM)
    np.testing.assert_allclose(s, v["tie_sum_out"], rtol=1e-6, equal_nan=True)
    assert not out[1].any() and not out[5].any() and not arg[1].any()      # empty bags


def test_torch_vectors_random(oracle, torch_vectors):
    v = torch_vectors
    w, wq, idx, off, psw = v["rnd_table"], v["rnd_tableq"], v["rnd_idx"], v["rnd_off"], v["rnd_psw"]
    for op, key in ((oracle.OP_SUM, "rnd_sum"), (oracle.OP_MEAN, "rnd_mean")):
        out, _, _ = oracle.embedding_bag(w, idx, off, op)
        np.testing.assert_allclose(out, v[key], rtol=1e-5, atol=1e-6)
    out, arg, _ = oracle.embedding_bag(wq, idx, off, oracle.OP_MAX, want_max_indices=True)
    np.testing.assert_array_equal(out, v["rnd_max"])
    np.testing.assert_array_equal(arg, v["rnd_max_arg"])
    out, arg, _ = oracle.embedding_bag(wq, idx.astype(np.int32), off.astype(np.int32), oracle.OP_MAX,
                                       want_max_indices=True)
    np.testing.assert_array_equal(out, v["rnd_max_i32"])
    np.testing.assert_array_equal(arg, v["rnd_max_arg_i32"])
    assert arg.dtype == np.int32
    out, _, _ = oracle.embedding_bag(w, idx, off, oracle.OP_SUM, per_sample_weights=psw)
    np.testing.assert_allclose(out, v["rnd_wsum"], rtol=1e-5, atol=1e-6)
    # fp16 tables: fp32 accumulation, one rounding at the end
    wh = w.astype(np.float16)
    out, _, _ = oracle.embedding_bag(wh, idx, off, oracle.OP_SUM)
    assert out.dtype == np.float16
    np.testing.assert_allclose(out.astype(np.float32), v["rnd_sum_f16"].astype(np.float32), atol=1e-2, rtol=5e-3)
    assert np.mean(out.view(np.uint16) == v["rnd_sum_f16"].view(np.uint16)) > 0.98
    out, _, _ = oracle.embedding_bag(wq.astype(np.float16), idx, off, oracle.OP_MAX)
    np.testing.assert_array_equal(out, v["rnd_max_f16"])
    # fp16 mean: libtorch's CPU kernel divides the sum after rounding it to fp16, the oracle divides the
    # fp32 sum and rounds once; the two stay inside the fp16 bar
    out, _, _ = oracle.embedding_bag(wh, idx, off, oracle.OP_MEAN)
    np.testing.assert_allclose(out.astype(np.float32), v["rnd_mean_f16"].astype(np.float32), atol=1e-2, rtol=5e-3)


@pytest.mark.parametrize("mode", ["sum", "mean", "max"])
@pytest.mark.parametrize("idt", [np.int32, np.int64])
def test_against_live_libtorch_and_numpy(oracle, mode, idt):
    """Config-2-shaped case (scaled down): Poisson lengths with empty bags, Zipf ids."""
    wl = workloads.config2(variant=3, index_dtype=idt, rows=5000, n_bags=300, dim=128, mode=mode)
    op = {"sum": oracle.OP_SUM, "mean": oracle.OP_MEAN, "max": oracle.OP_MAX}[mode]
    out, _, oob = oracle.embedding_bag(wl.table, wl.indices, wl.offsets, op)
    assert oob == 0 and (wl.lengths == 0).any()
    ref = torch.nn.functional.embedding_bag(torch.from_numpy(wl.indices), torch.from_numpy(wl.table),
                                            torch.from_numpy(wl.offsets), mode=mode).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-6)
    # independent numpy evaluation in float64
    ends = np.append(wl.offsets[1:], wl.indices.size).astype(np.int64)
    for b in (0, 1, 17, 150, 299):
        rows = wl.table[wl.indices[wl.offsets[b]:ends[b]]].astype(np.float64)
        if rows.shape[0] == 0:
            want = np.zeros(128)
        else:
            want = {"sum": rows.sum(0), "mean": rows.mean(0), "max": rows.max(0)}[mode]
        np.testing.assert_allclose(out[b], want, rtol=1e-5, atol=1e-6)


def test_square_sum_fixed_length_and_gather(oracle):
    rng = np.random.Generator(np.random.PCG64(11))
    w = rng.standard_normal((50, 6)).astype(np.float32)
    idx = rng.integers(0, 50, size=(10, 5)).astype(np.int32)     # the reference's TF test shape
    s, _, _ = oracle.embedding_bag(w, idx, None, oracle.OP_SUM)
    q, _, _ = oracle.embedding_bag(w, idx, None, oracle.OP_SQUARE_SUM)
    np.testing.assert_allclose(s, w.astype(np.float64)[idx].sum(1), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(q, (w.astype(np.float64)[idx] ** 2).sum(1), rtol=1e-6, atol=1e-6)
    g, oob = oracle.gather(w, idx)
    np.testing.assert_array_equal(g, w[idx])
    assert oob == 0


def test_index_filter_and_data_offset(oracle):
    """Ids outside [data_offset, data_offset+count) are skipped (embedding_bag_plugin.cu:94)."""
    w = np.arange(12, dtype=np.float32).reshape(4, 3) + 1
    idx = np.array([10, 13, 9, 14, 11, -5], np.int32)            # shard holds ids 10..13
    off = np.array([0, 3], np.int32)
    out, _, oob = oracle.embedding_bag(w, idx, off, oracle.OP_SUM, data_offset=10)
    np.testing.assert_array_equal(out, [w[0] + w[3], w[1]])
    assert oob == 3
    g, oob = oracle.gather(w, idx.reshape(1, 6), data_offset=10)
    np.testing.assert_array_equal(g[0, 2], 0)
    np.testing.assert_array_equal(g[0, 1], w[3])
    assert oob == 3
    # include_last_offset: same bags described with a trailing end offset
    out2, _, _ = oracle.embedding_bag(w, idx, np.array([0, 3, 6], np.int32), oracle.OP_SUM, data_offset=10,
                                      include_last_offset=True)
    np.testing.assert_array_equal(out, out2)


def test_concatenated_layout(oracle):
    wl = workloads.config4(variant=1, n_tables=3, n_bags=64, max_rows=2000)
    out = np.zeros((64, 3 * 128), np.float16)
    for t in range(3):
        tab = wl.host_table(t)
        oracle.embedding_bag(tab, wl.indices[t], wl.offsets[t], oracle.OP_SUM, out=out, out_col=t * 128)
        single, _, _ = oracle.embedding_bag(tab, wl.indices[t], wl.offsets[t], oracle.OP_SUM)
        np.testing.assert_array_equal(out[:, t * 128:(t + 1) * 128], single)
