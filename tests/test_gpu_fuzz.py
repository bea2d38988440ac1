"""Seeded random configurations of the bag reduction through the C ABI against the oracle:
row width, table / id / output types, mode, weights, offsets form (empty bags, one giant bag,
include_last_offset), data_offset with ids outside the shard, output column blocks.  Every value
is compared bit for bit; the out-of-range count must agree with the sticky device flag."""
import numpy as np
import pytest
import torch

from forward_amd import ops
from gpu_util import assert_bits_equal, dev, host

pytestmark = pytest.mark.gpu

MODES = ("sum", "mean", "max", "square_sum")
ORACLE_OP = {"sum": 0, "mean": 1, "max": 2, "square_sum": 3}


def make_case(seed):
    r = np.random.Generator(np.random.PCG64(9000 + seed))
    dim = int(r.choice([1, 3, 8, 16, 24, 32, 64, 96, 128, 200, 256, 520, 1024]))
    rows = int(r.choice([1, 2, 17, 300, 5000]))
    tdt = r.choice([np.float32, np.float16])
    idt = r.choice([np.int32, np.int64])
    mode = MODES[int(r.integers(0, 4))]
    weighted = mode == "sum" and r.random() < 0.3
    n_bags = int(r.choice([1, 2, 5, 33, 200, 1500]))
    style = int(r.integers(0, 4))
    if style == 0:      # short bags with many empty ones
        lengths = r.integers(0, 4, n_bags) * (r.random(n_bags) < 0.6)
    elif style == 1:    # typical
        lengths = r.integers(0, 40, n_bags)
    elif style == 2:    # one bag far longer than the LDS window, the rest tiny
        lengths = r.integers(0, 3, n_bags)
        lengths[int(r.integers(0, n_bags))] = int(r.integers(3000, 9000))
    else:               # all equal
        lengths = np.full(n_bags, int(r.integers(1, 20)))
    lengths = lengths.astype(np.int64)
    n = int(lengths.sum())
    include_last = bool(r.random() < 0.3)
    off = np.concatenate([[0], np.cumsum(lengths)])
    off = (off if include_last else off[:-1]).astype(idt)
    data_offset = int(r.choice([0, 0, 7, 1000]))
    spill = r.random() < 0.4                       # some ids outside [data_offset, data_offset + rows)
    lo, hi = (data_offset - 3, data_offset + rows + 3) if spill else (data_offset, data_offset + rows)
    idx = r.integers(lo, hi, n).astype(idt)
    table = (r.standard_normal((rows, dim)) * 0.5).astype(tdt)
    psw = r.random(n).astype(tdt) if weighted else None
    odt = tdt if r.random() < 0.7 else (np.float16 if tdt == np.float32 else np.float32)
    block = bool(r.random() < 0.3) and dim % 8 == 0
    return dict(table=table, idx=idx, off=off, mode=mode, psw=psw, include_last=include_last,
                data_offset=data_offset, odt=odt, block=block, n_bags=n_bags, dim=dim, spill=spill)


@pytest.mark.parametrize("seed", range(60))
def test_random_configuration(oracle, seed):
    c = make_case(seed)
    want_arg = c["mode"] == "max" and seed % 2 == 0
    kw = dict(per_sample_weights=c["psw"], include_last_offset=c["include_last"], data_offset=c["data_offset"])
    tdt = torch.float16 if c["odt"] == np.float16 else torch.float32
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    if c["block"]:
        width, col = c["dim"] * 3, c["dim"]
        want = np.full((c["n_bags"], width), 3.0, c["odt"])
        out = torch.full((c["n_bags"], width), 3.0, dtype=tdt, device="cuda")
        _, warg, n_oob = oracle.embedding_bag(c["table"], c["idx"], c["off"], ORACLE_OP[c["mode"]], out=want,
                                              out_col=col, out_dtype=c["odt"], want_max_indices=want_arg, **kw)
        res = ops.embedding_bag(dev(c["table"]), dev(c["idx"]), dev(c["off"]), c["mode"], out=out, out_col=col,
                                out_dtype=tdt, want_max_indices=want_arg, oob_flag=flag,
                                **{**kw, "per_sample_weights": dev(c["psw"])})
        got = host(out)
    else:
        want, warg, n_oob = oracle.embedding_bag(c["table"], c["idx"], c["off"], ORACLE_OP[c["mode"]],
                                                 out_dtype=c["odt"], want_max_indices=want_arg, **kw)
        res = ops.embedding_bag(dev(c["table"]), dev(c["idx"]), dev(c["off"]), c["mode"], out_dtype=tdt,
                                want_max_indices=want_arg, oob_flag=flag,
                                **{**kw, "per_sample_weights": dev(c["psw"])})
        got = host(res[0] if want_arg else res)
    assert_bits_equal(got, want, "seed %d: %s dim %d %s ids, %s table" % (
        seed, c["mode"], c["dim"], c["idx"].dtype, c["table"].dtype))
    if want_arg:
        np.testing.assert_array_equal(host(res[1]), warg)
    assert bool(flag.item()) == (n_oob > 0)


@pytest.mark.parametrize("seed", range(24))
def test_random_fixed_length_and_gather(oracle, seed):
    r = np.random.Generator(np.random.PCG64(7000 + seed))
    dim = int(r.choice([1, 4, 16, 64, 100, 128, 384]))
    rows = int(r.choice([1, 50, 4000]))
    tdt = r.choice([np.float32, np.float16])
    idt = r.choice([np.int32, np.int64])
    b, l = int(r.choice([1, 7, 300, 2000])), int(r.choice([1, 2, 5, 31, 130]))
    data_offset = int(r.choice([0, 11]))
    spill = 2 if r.random() < 0.4 else 0
    ids = r.integers(data_offset - spill, data_offset + rows + spill, (b, l)).astype(idt)
    table = (r.standard_normal((rows, dim)) * 0.5).astype(tdt)
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    if seed % 3 == 0:
        want, n_oob = oracle.gather(table, ids, data_offset=data_offset)
        got = host(ops.gather(dev(table), dev(ids), data_offset=data_offset, oob_flag=flag))
    else:
        mode = MODES[int(r.integers(0, 4))]
        want, _, n_oob = oracle.embedding_bag(table, ids, None, ORACLE_OP[mode], data_offset=data_offset)
        got = host(ops.embedding_bag_fixed(dev(table), dev(ids), mode, data_offset=data_offset, oob_flag=flag))
    assert_bits_equal(got.reshape(want.shape), want, "seed %d" % seed)
    assert bool(flag.item()) == (n_oob > 0)


@pytest.mark.parametrize("seed", range(40))
def test_random_layer_norm_shapes(oracle, seed):
    """LayerNorm / SkipLayerNorm over random row lengths (every kernel variant: rows sharing a
    wavefront, a wavefront per row, a workgroup per row, element-strided), row counts, types and
    operands, against the float64 oracle at the parity tolerances."""
    from gpu_util import assert_close
    r = np.random.Generator(np.random.PCG64(5000 + seed))
    kind = int(r.integers(0, 5))
    ld = int([r.integers(1, 33), r.integers(1, 65) * 8, r.integers(33, 2100), r.integers(260, 2050) * 8,
              r.integers(1, 600) * 2 + 1][kind])
    rows = int(r.choice([1, 3, 64, 257, 1500]))
    dt = r.choice([np.float32, np.float16])
    x = (r.standard_normal((rows, ld)) * r.uniform(0.1, 3.0) + r.uniform(-2, 2)).astype(dt)
    sk = r.standard_normal((rows, ld)).astype(dt) if r.random() < 0.6 else None
    bi = (0.1 * r.standard_normal(ld)).astype(np.float32) if r.random() < 0.5 else None
    g = (1 + 0.1 * r.standard_normal(ld)).astype(np.float32)
    b = (0.1 * r.standard_normal(ld)).astype(np.float32)
    eps = float(r.choice([1e-12, 1e-5]))
    if ld < 4:
        eps = 1e-5                                  # one or two elements: the variance can be exactly zero
    got = host(ops.skip_layer_norm(dev(x), dev(g), dev(b), skip=dev(sk), bias=dev(bi), eps=eps))
    want = oracle.skip_layer_norm(x, g, b, skip=sk, bias=bi, eps=eps)
    assert got.dtype == dt and got.shape == x.shape
    assert_close(got, want, dt, scale=4.0)


@pytest.mark.parametrize("seed", range(20))
def test_random_table_groups(oracle, seed):
    """The multi-table launch through ``ops.embedding_bag_group`` on random groups (table count, row
    width, types, mode, weights on some tables, trailing end offsets, XCD affinity on / off): every
    column block bit-identical to the oracle's result for that table alone."""
    r = np.random.Generator(np.random.PCG64(3000 + seed))
    n_tables = int(r.choice([1, 2, 5, 9, 30, 61]))
    dim = int(r.choice([4, 8, 32, 64, 128, 200]))
    tdt = r.choice([np.float32, np.float16])
    idt = r.choice([np.int32, np.int64])
    n_bags = int(r.choice([1, 17, 300, 2000]))
    mode = MODES[int(r.integers(0, 4))]
    include_last = bool(r.random() < 0.4)
    weighted = mode == "sum" and r.random() < 0.4
    tables, ids, offs, psw = [], [], [], []
    for t in range(n_tables):
        rows = int(r.choice([1, 3, 50, 700, 9000]))
        tables.append((r.standard_normal((rows, dim)) * 0.5).astype(tdt))
        lengths = r.integers(0, int(r.choice([2, 6, 40])), n_bags)
        n = int(lengths.sum())
        off = np.concatenate([[0], np.cumsum(lengths)])
        offs.append((off if include_last else off[:-1]).astype(idt))
        ids.append(r.integers(0, rows, n).astype(idt))
        psw.append(r.random(n).astype(tdt) if weighted and r.random() < 0.7 else None)
    odt = tdt if r.random() < 0.7 else (np.float16 if tdt == np.float32 else np.float32)
    tt = torch.float16 if odt == np.float16 else torch.float32
    got = host(ops.embedding_bag_group([dev(t) for t in tables], [dev(i) for i in ids], [dev(o) for o in offs], mode,
                                       include_last_offset=include_last, out_dtype=tt,
                                       xcd_table_affinity=bool(seed % 2),
                                       per_sample_weights=[dev(w) for w in psw] if weighted else None))
    assert got.shape == (n_bags, n_tables * dim)
    for t in range(n_tables):
        want, _, _ = oracle.embedding_bag(tables[t], ids[t], offs[t], ORACLE_OP[mode], per_sample_weights=psw[t],
                                          include_last_offset=include_last, out_dtype=odt)
        assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "seed %d table %d of %d (%s)" % (seed, t, n_tables, mode))


def _offset_copy(a, k):
    """``a`` on the device, starting ``k`` elements past an allocation boundary."""
    if a is None:
        return None
    big = torch.empty(a.size + 8, dtype=torch.from_numpy(a[:0]).dtype, device="cuda")
    big[k:k + a.size] = torch.from_numpy(a).cuda()
    return big[k:k + a.size]


@pytest.mark.parametrize("seed", range(16))
def test_random_large_batches(oracle, seed):
    """Batches of 2 500 ... 200 000 bags (runs of hundreds of bags: ids staged with wide loads, bags
    ordered by length, the XCD mapping with its quarter runs where the launch is large enough), bag
    lengths from four distributions including a heavy tail, id and weight arrays that start off a
    16-byte boundary, one table or a group: every column block bit-identical to the oracle's."""
    r = np.random.Generator(np.random.PCG64(424200 + seed))
    n_tables = int(r.choice([1, 1, 2, 3, 8, 12]))
    dim = int(r.choice([8, 32, 64, 128, 256]))
    tdt = r.choice([np.float32, np.float16])
    idt = r.choice([np.int32, np.int64])
    n_bags = int(r.choice([5000, 30000, 70001, 200000])) // (2 if n_tables > 3 else 1)
    mode = MODES[int(r.integers(0, 4))]
    weighted = mode == "sum" and r.random() < 0.4
    include_last = bool(r.random() < 0.3)
    tables, ids, offs, psw = [], [], [], []
    for t in range(n_tables):
        rows = int(r.choice([3, 700, 90000]))
        tables.append((r.standard_normal((rows, dim)) * 0.5).astype(tdt))
        style = int(r.integers(0, 4))
        if style == 0:
            lengths = r.integers(0, 4, n_bags)
        elif style == 1:
            lengths = r.integers(0, 50, n_bags)
        elif style == 2:
            lengths = np.minimum((r.pareto(1.2, n_bags) + 1).astype(np.int64), 3000)
        else:
            lengths = r.poisson(int(r.choice([2, 20, 80])), n_bags)
        lengths = lengths.astype(np.int64)
        n = int(lengths.sum())
        off = np.concatenate([[0], np.cumsum(lengths)])
        offs.append((off if include_last else off[:-1]).astype(idt))
        i = r.integers(0, rows, n)
        if r.random() < 0.3 and n:
            i[r.integers(0, n, 20)] = rows + 5
        ids.append(i.astype(idt))
        psw.append(r.random(n).astype(tdt) if weighted and r.random() < 0.8 else None)
    odt = tdt if r.random() < 0.7 else (np.float16 if tdt == np.float32 else np.float32)
    tt = torch.float16 if odt == np.float16 else torch.float32
    shift = int(r.integers(0, 4))
    d_ids = [_offset_copy(i, shift) for i in ids]
    d_psw = [_offset_copy(w, (shift * 3) % 8) for w in psw] if weighted else None
    if n_tables == 1:
        got = host(ops.embedding_bag(dev(tables[0]), d_ids[0], dev(offs[0]), mode, include_last_offset=include_last,
                                     out_dtype=tt, per_sample_weights=d_psw[0] if weighted else None))
    else:
        got = host(ops.embedding_bag_group([dev(t) for t in tables], d_ids, [dev(o) for o in offs], mode,
                                           include_last_offset=include_last, out_dtype=tt,
                                           xcd_table_affinity=bool(seed % 2), per_sample_weights=d_psw))
    for t in range(n_tables):
        want, _, _ = oracle.embedding_bag(tables[t], ids[t], offs[t], ORACLE_OP[mode], per_sample_weights=psw[t],
                                          include_last_offset=include_last, out_dtype=odt)
        assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, "seed %d table %d of %d (%s)" % (seed, t, n_tables, mode))
