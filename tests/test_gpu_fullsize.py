"""Config 4 at its full size (26 tables x 65536 bags, ~27.8 M ids, 8 GB of fp16 tables in HBM).

The oracle cannot hold 8 GB of host tables cheaply, so parity is checked (a) bit-exactly on a
sample of bags per table whose rows are fetched back from HBM, and (b) through size-independent
properties: the fused launch equals 26 single-table launches, int64 ids equal int32 ids, and a
float64 checksum of all outputs of a table equals the multiplicity-weighted sum of its rows."""
import numpy as np
import pytest
import torch

from forward_amd import ops, workloads
from gpu_util import assert_bits_equal, host

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def full():
    wl = workloads.config4()
    assert len(wl.rows) == 26 and wl.n_bags == 65536 and 27_000_000 < wl.n_indices() < 29_000_000
    tabs = [wl.device_table(t, torch) for t in range(26)]
    idx = [torch.from_numpy(i).cuda() for i in wl.indices]
    off = [torch.from_numpy(o).cuda() for o in wl.offsets]
    batch = ops.MultiTableBatch(tabs, idx, off)
    out = batch.forward()
    torch.cuda.synchronize()
    return wl, tabs, idx, off, batch, out


def test_sampled_bags_match_oracle_bit_exact(full, oracle):
    wl, tabs, idx, off, batch, out = full
    assert tuple(out.shape) == (65536, 26 * 128) and out.dtype == torch.float16
    rng = np.random.Generator(np.random.PCG64(44))
    for t in range(26):
        ends = np.append(wl.offsets[t][1:], wl.indices[t].size).astype(np.int64)
        lens = ends - wl.offsets[t]
        bags = np.unique(np.concatenate([rng.integers(0, 65536, 300), np.argsort(lens)[-20:], [0, 65535]]))
        ids = np.concatenate([wl.indices[t][wl.offsets[t][b]:ends[b]] for b in bags])
        uniq, inv = np.unique(ids, return_inverse=True)
        rows = host(tabs[t][torch.from_numpy(uniq.astype(np.int64)).cuda()])        # compact table of the rows needed
        sub_off = workloads.offsets_from_lengths(lens[bags], np.int32)
        want, _, oob = oracle.embedding_bag(rows, inv.astype(np.int32), sub_off, oracle.OP_SUM)
        assert oob == 0
        got = host(out[torch.from_numpy(bags).cuda(), t * 128:(t + 1) * 128])
        assert_bits_equal(got, want, "table %d (%d rows)" % (t, wl.rows[t]))


@pytest.mark.parametrize("mode", ["mean", "max", "wsum"])
def test_other_modes_sampled_bags_match_oracle_bit_exact(full, oracle, mode):
    """The fused launch in its other modes at full size (mean, max, per-sample weights through the
    table descriptors; int64 ids for max): sampled bags of every table against the oracle."""
    wl, tabs, idx, off, batch, _ = full
    weighted = mode == "wsum"
    m = "sum" if weighted else mode
    psw = None
    if weighted:
        g = torch.Generator(device="cuda").manual_seed(4004)
        psw = [torch.rand(i.numel(), generator=g, device="cuda").half() for i in idx]
        b = ops.MultiTableBatch(tabs, idx, off, per_sample_weights=psw)
    elif mode == "max":
        b = ops.MultiTableBatch(tabs, [i.long() for i in idx], [o.long() for o in off])
    else:
        b = batch
    out = b.forward(mode=m, xcd_table_affinity=True)
    torch.cuda.synchronize()
    rng = np.random.Generator(np.random.PCG64(45))
    for t in range(26):
        ends = np.append(wl.offsets[t][1:], wl.indices[t].size).astype(np.int64)
        lens = ends - wl.offsets[t]
        bags = np.unique(np.concatenate([rng.integers(0, 65536, 200), np.argsort(lens)[-10:], [0, 65535]]))
        pos = np.concatenate([np.arange(wl.offsets[t][x], ends[x]) for x in bags])
        ids = wl.indices[t][pos]
        uniq, inv = np.unique(ids, return_inverse=True)
        rows = host(tabs[t][torch.from_numpy(uniq.astype(np.int64)).cuda()])
        sub_off = workloads.offsets_from_lengths(lens[bags], np.int32)
        w = host(psw[t][torch.from_numpy(pos).cuda()]) if weighted else None
        want, _, oob = oracle.embedding_bag(rows, inv.astype(np.int32), sub_off, ops.MODES[m], per_sample_weights=w)
        assert oob == 0
        got = host(out[torch.from_numpy(bags).cuda(), t * 128:(t + 1) * 128])
        assert_bits_equal(got, want, "%s, table %d (%d rows)" % (mode, t, wl.rows[t]))


def test_fused_equals_per_table_and_int64(full):
    wl, tabs, idx, off, batch, out = full
    ref = torch.zeros_like(out)
    for t in range(26):
        ops.embedding_bag(tabs[t], idx[t], off[t], "sum", out=ref, out_col=t * 128)
    assert torch.equal(out, ref)
    t = int(np.argmax(wl.rows))                                   # the largest table (6.2 M rows)
    o64 = ops.embedding_bag(tabs[t], idx[t].long(), off[t].long(), "sum")
    assert torch.equal(o64, out[:, t * 128:(t + 1) * 128])
    assert torch.equal(batch.forward(xcd_table_affinity=True), out)


def test_checksum_of_checksums(full):
    wl, tabs, idx, off, batch, out = full
    for t in (0, 1, 19):
        o32 = ops.embedding_bag(tabs[t], idx[t], off[t], "sum", out_dtype=torch.float32)
        got = o32.double().sum(0)
        counts = torch.bincount(idx[t].long(), minlength=wl.rows[t]).double()
        want = (counts.unsqueeze(1) * tabs[t].double()).sum(0)     # sum_r multiplicity(r) * row_r
        scale = float((counts.unsqueeze(1) * tabs[t].double().abs()).sum(0).max())
        assert float((got - want).abs().max()) <= 1e-6 * scale
