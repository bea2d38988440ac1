"""More seeded random cases against the CPU oracle, beside those of test_gpu_fuzz.py: bag launches with
options drawn together that the cases there keep apart (row widths up to 2048 columns that are and
are not a multiple of a lane's slice, a negative data_offset, column blocks that start off a 16-byte
boundary, the two-output sum / square-sum form, bags longer than the id window among empty ones),
BERT embedding + LayerNorm launches (sequence length, batch, hidden size, table sizes, mask lengths),
and multi-table launches on both sides of the 40-table limit of descriptors that travel as kernel
arguments, with trailing columns the launch must leave alone.  Bag reductions are bit-exact;
LayerNorm is within the stated tolerance."""
import numpy as np
import pytest
import torch

from forward_amd import ops, workloads
from gpu_util import assert_bits_equal, assert_close, dev, host

pytestmark = pytest.mark.gpu

OPS = {"sum": 0, "mean": 1, "max": 2, "square_sum": 3}
DIMS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 24, 31, 32, 40, 48, 64, 72, 96, 100, 128, 136, 192, 200, 256, 320, 512, 520, 1024,
        1032, 2048]


def draw_bag_case(rng):
    dim = int(rng.choice(DIMS))
    tdt = rng.choice([np.float16, np.float32])
    idt = rng.choice([np.int32, np.int64])
    odt = rng.choice([np.float16, np.float32])
    mode = str(rng.choice(["sum", "mean", "max", "square_sum", "wsum", "sum+sq"]))
    rows = int(rng.choice([1, 2, 17, 1000, 40000]))
    budget = 600000 // max(dim, 8)            # ids: keeps the oracle's side of a case in milliseconds
    shape = str(rng.choice(["short", "ragged", "long", "one"]))
    if shape == "short":
        lengths = rng.integers(0, 5, int(rng.integers(1, max(2, budget // 3))))
    elif shape == "ragged":
        lengths = rng.geometric(0.08, int(rng.integers(1, max(2, budget // 14)))) - 1
    elif shape == "long":   # a few bags longer than a run's id window among short ones
        lengths = rng.integers(0, 4, int(rng.integers(4, 200)))
        lengths[rng.integers(0, lengths.size, 3)] = budget // 4
    else:
        lengths = np.array([int(rng.integers(0, budget))])
    data_offset = int(rng.choice([0, 0, 5, -3]))
    lo, hi = data_offset, data_offset + rows
    if rng.random() < 0.3:                     # some ids outside the table on either side
        lo, hi = lo - 2, hi + 3
    idx = rng.integers(lo, hi, int(lengths.sum())).astype(idt)
    include_last = bool(rng.random() < 0.3)
    off = workloads.offsets_from_lengths(lengths, idt)
    if include_last:
        off = np.concatenate([off, np.array([idx.size], idt)])
    table = (rng.standard_normal((rows, dim)) * 0.5).astype(tdt)
    psw = (rng.standard_normal(idx.size) * 0.5).astype(tdt) if mode == "wsum" else None
    out_col = int(rng.choice([0, 0, 8, 3])) if rng.random() < 0.4 else None
    return dict(dim=dim, tdt=tdt, idt=idt, odt=odt, mode=mode, rows=rows, lengths=lengths, idx=idx, off=off,
                include_last=include_last, data_offset=data_offset, table=table, psw=psw, out_col=out_col,
                any_outside=bool(((idx < data_offset) | (idx >= data_offset + rows)).any()))


def describe(c):
    return ("dim %d table %s ids %s out %s mode %s rows %d bags %d ids %d include_last %d data_offset %d out_col %s"
            % (c["dim"], np.dtype(c["tdt"]).name, np.dtype(c["idt"]).name, np.dtype(c["odt"]).name, c["mode"],
               c["rows"], c["lengths"].size, c["idx"].size, c["include_last"], c["data_offset"], c["out_col"]))


@pytest.mark.parametrize("seed", range(12))
def test_random_bag_launches_equal_the_oracle(oracle, seed):
    rng = np.random.Generator(np.random.PCG64(9000 + seed))
    for k in range(16):
        c = draw_bag_case(rng)
        what = "seed %d case %d: %s" % (seed, k, describe(c))
        print(what, flush=True)
        tod = torch.float16 if c["odt"] == np.float16 else torch.float32
        m = {"wsum": "sum", "sum+sq": "sum"}.get(c["mode"], c["mode"])
        n_bags = c["lengths"].size
        flag = torch.zeros(1, dtype=torch.int32, device="cuda")
        kw = dict(include_last_offset=c["include_last"], data_offset=c["data_offset"], out_dtype=tod, oob_flag=flag)
        okw = dict(include_last_offset=c["include_last"], data_offset=c["data_offset"], out_dtype=c["odt"])
        want, warg, n_out = oracle.embedding_bag(c["table"], c["idx"], c["off"], OPS[m], per_sample_weights=c["psw"],
                                                 want_max_indices=(m == "max"), **okw)
        assert (n_out > 0) == c["any_outside"], what
        if c["out_col"] is None:
            res = ops.embedding_bag(dev(c["table"]), dev(c["idx"]), dev(c["off"]), m, per_sample_weights=dev(c["psw"]),
                                    want_max_indices=(m == "max"), with_square_sum=(c["mode"] == "sum+sq"), **kw)
            got = host(res[0] if isinstance(res, tuple) else res)
            if m == "max":
                np.testing.assert_array_equal(host(res[1]), warg, err_msg=what)
            if c["mode"] == "sum+sq":
                want2, _, _ = oracle.embedding_bag(c["table"], c["idx"], c["off"], OPS["square_sum"], **okw)
                assert_bits_equal(host(res[1]), want2, what + " (square sums)")
        else:   # a column block of a wider matrix whose other columns must stay as they are
            col = c["out_col"]
            wide = torch.full((n_bags, c["dim"] + 11), 7.0, dtype=tod, device="cuda")
            ops.embedding_bag(dev(c["table"]), dev(c["idx"]), dev(c["off"]), m, per_sample_weights=dev(c["psw"]),
                              out=wide, out_col=col, **kw)
            w = host(wide)
            got = w[:, col:col + c["dim"]]
            assert (w[:, :col] == 7.0).all() and (w[:, col + c["dim"]:] == 7.0).all(), what
        assert_bits_equal(got, want, what)
        assert bool(flag.item()) == c["any_outside"], what


@pytest.mark.parametrize("seed", range(3))
def test_random_embedding_layer_norm_launches_equal_the_oracle(oracle, seed):
    rng = np.random.Generator(np.random.PCG64(9300 + seed))
    for k in range(8):
        hidden = int(rng.choice([8, 24, 64, 128, 200, 256, 312, 768, 1024, 1280, 2048]))
        dt = rng.choice([np.float16, np.float32])
        S, B = int(rng.integers(1, 70)), int(rng.integers(1, 20))
        V, P, T = int(rng.integers(2, 500)), int(rng.integers(S, S + 40)), int(rng.integers(1, 4))
        word, pos, tok = (rng.standard_normal((n, hidden)).astype(dt) * 0.5 for n in (V, P, T))
        ids = rng.integers(0, V, (S, B)).astype(np.int32)
        seg = rng.integers(0, T, (S, B)).astype(np.int32)
        lens = rng.integers(0, S + 1, B)
        mask = (np.arange(S)[:, None] < lens[None, :]).astype(np.int32)
        gamma = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
        beta = rng.standard_normal(hidden).astype(np.float32) * 0.1
        eps = float(rng.choice([1e-12, 1e-5]))
        what = "seed %d case %d: S %d B %d hidden %d %s V %d P %d T %d" % (seed, k, S, B, hidden, np.dtype(dt).name, V, P, T)
        print(what, flush=True)
        want, wmask, n_out = oracle.emb_layer_norm(ids, seg, mask, word, pos, tok, gamma, beta, eps=eps)
        assert n_out == 0, what
        got, gmask = ops.emb_layer_norm(dev(ids), dev(seg), dev(mask), dev(word), dev(pos), dev(tok), dev(gamma), dev(beta),
                                        eps=eps)
        assert_close(host(got).reshape(want.shape), want, dt, scale=10.0)
        np.testing.assert_array_equal(host(gmask), wmask, err_msg=what)


@pytest.mark.parametrize("seed", range(6))
def test_random_multi_table_launches_equal_the_oracle(oracle, seed):
    """One launch for 1 .. 70 tables of very different sizes and bag lengths (descriptors among the
    launch's arguments up to 40 tables, in device memory beyond), with and without the per-die table
    order, some tables weighted: every table's column block bit-exact, the other columns untouched."""
    rng = np.random.Generator(np.random.PCG64(9400 + seed))
    for k in range(5):
        n = int(rng.choice([1, 2, 3, 7, 26, 40, 41, 70]))
        dim = int(rng.choice([4, 8, 16, 32, 64, 72, 128, 256]))
        tdt = rng.choice([np.float16, np.float32])
        idt = rng.choice([np.int32, np.int64])
        odt = rng.choice([np.float16, np.float32])
        tod = torch.float16 if odt == np.float16 else torch.float32
        mode = str(rng.choice(["sum", "mean", "max", "square_sum", "wsum"]))
        m = "sum" if mode == "wsum" else mode
        include_last = bool(rng.random() < 0.3)
        affinity = bool(rng.random() < 0.6)
        n_bags = int(rng.integers(1, max(2, 60000 // (n * max(dim, 16)) * 8)))
        tables, idxs, offs, psws = [], [], [], []
        for t in range(n):
            rows = int(rng.choice([1, 50, 5000]))
            kind = rng.integers(0, 3)
            lengths = (np.ones(n_bags, np.int64) if kind == 0 else rng.integers(0, 6, n_bags) if kind == 1
                       else rng.geometric(0.05, n_bags) - 1)
            idx = rng.integers(-1 if rng.random() < 0.2 else 0, rows, int(lengths.sum())).astype(idt)
            off = workloads.offsets_from_lengths(lengths, idt)
            if include_last:
                off = np.concatenate([off, np.array([idx.size], idt)])
            tables.append((rng.standard_normal((rows, dim)) * 0.5).astype(tdt))
            idxs.append(idx), offs.append(off)
            psws.append((rng.standard_normal(idx.size) * 0.5).astype(tdt) if mode == "wsum" and rng.random() < 0.7 else None)
        what = "seed %d case %d: %d tables dim %d table %s ids %s out %s mode %s bags %d include_last %d affinity %d" % (
            seed, k, n, dim, np.dtype(tdt).name, np.dtype(idt).name, np.dtype(odt).name, mode, n_bags, include_last, affinity)
        print(what, flush=True)
        extra = int(rng.choice([0, 8]))
        out = torch.full((n_bags, n * dim + extra), 3.0, dtype=tod, device="cuda")
        flag = torch.zeros(1, dtype=torch.int32, device="cuda")
        ops.embedding_bag_group([dev(a) for a in tables], [dev(a) for a in idxs], [dev(a) for a in offs], m,
                                include_last_offset=include_last, out=out, out_dtype=tod, oob_flag=flag,
                                xcd_table_affinity=affinity,
                                per_sample_weights=[dev(w) for w in psws] if mode == "wsum" else None)
        got = host(out)
        any_outside = False
        for t in range(n):
            want, _, n_out = oracle.embedding_bag(tables[t], idxs[t], offs[t], OPS[m], per_sample_weights=psws[t],
                                                  include_last_offset=include_last, out_dtype=odt)
            any_outside |= n_out > 0
            assert_bits_equal(got[:, t * dim:(t + 1) * dim], want, what + ", table %d" % t)
        assert (got[:, n * dim:] == 3.0).all(), what
        assert bool(flag.item()) == any_outside, what
