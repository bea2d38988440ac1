"""Plugin enqueues recorded into a HIP graph: `enqueue` allocates nothing and never synchronises, so
a chain of plugins can be captured once and replayed with new input values in the same buffers.
Every replay is checked against the oracle, with eager launches and synchronisations between the
replays."""
import numpy as np
import pytest
import torch

from forward_amd import lib, plugin, workloads
from forward_amd.plugin import PluginFieldData as F
from gpu_util import assert_bits_equal, assert_close, dev, host

pytestmark = pytest.mark.gpu
REG = plugin.getPluginRegistry()


def test_bag_and_skip_layer_norm_chain_replays(oracle):
    rng = np.random.Generator(np.random.PCG64(77))
    rows, dim, n_bags = 5000, 64, 256
    table = (rng.standard_normal((rows, dim)) * 0.1).astype(np.float32)
    gamma = rng.normal(1.0, 0.02, dim).astype(np.float32)
    beta = rng.normal(0.0, 0.02, dim).astype(np.float32)
    bag = REG.getPluginCreator("EmbeddingBag_TRT", "001").createPlugin(
        "bag", [F("dim", dim), F("count", rows), F("offset", 0), F("op", 0), F("data", table)])
    sln = REG.getPluginCreator("CustomSkipLayerNormPluginDynamic", "1").createPlugin(
        "sln", [F("ld", dim), F("type_id", lib.F32), F("beta", beta), F("gamma", gamma)])

    def batch(seed):
        r = np.random.Generator(np.random.PCG64(seed))
        lengths = r.integers(0, 24, n_bags)
        n = 4000                                   # fixed id count so the captured shapes stay valid
        lengths = (lengths * (n / max(1, lengths.sum()))).astype(np.int64)
        lengths[-1] += n - lengths.sum()
        assert lengths.min() >= 0 and lengths.sum() == n
        off = np.concatenate([[0], np.cumsum(lengths)[:-1]]).astype(np.int32)
        ids = r.integers(0, rows, n).astype(np.int32)
        skip = r.standard_normal((n_bags, dim)).astype(np.float32)
        return ids, off, skip

    ids0, off0, skip0 = batch(0)
    d_ids, d_off, d_skip = dev(ids0), dev(off0), dev(skip0)
    d_bag = torch.zeros((n_bags, dim), dtype=torch.float32, device="cuda")
    d_out = torch.zeros_like(d_bag)
    bag.configurePlugin([((ids0.size,), lib.I32), ((n_bags,), lib.I32)], [((n_bags, dim), lib.F32)])
    sln.configurePlugin([((n_bags, dim), lib.F32)] * 2, [((n_bags, dim), lib.F32)])

    def chain():
        bag.enqueue([d_ids, d_off], [d_bag])
        sln.enqueue([d_bag, d_skip], [d_out])

    def want(ids, off, skip):
        b, _, _ = oracle.embedding_bag(table, ids, off, oracle.OP_SUM)
        return b, oracle.skip_layer_norm(b, gamma, beta, skip=skip)

    chain()                                        # eager, also warms up
    torch.cuda.synchronize()
    wb, wo = want(ids0, off0, skip0)
    assert_bits_equal(host(d_bag), wb, "eager bag")
    assert_close(host(d_out), wo, np.float32)

    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):                      # enqueue picks up torch's capturing stream
        chain()
    torch.cuda.synchronize()

    for seed in (1, 2, 3, 4):
        ids, off, skip = batch(seed)
        d_ids.copy_(dev(ids))
        d_off.copy_(dev(off))
        d_skip.copy_(dev(skip))
        d_bag.fill_(-1.0)
        d_out.fill_(-1.0)
        g.replay()
        torch.cuda.synchronize()
        wb, wo = want(ids, off, skip)
        assert_bits_equal(host(d_bag), wb, "replay %d bag" % seed)
        assert_close(host(d_out), wo, np.float32)
        # eager work between replays must neither disturb nor be disturbed by the graph
        scratch = torch.zeros_like(d_bag)
        bag.enqueue([d_ids, d_off], [scratch])
        torch.cuda.synchronize()
        assert_bits_equal(host(scratch), wb, "eager between replays %d" % seed)
    assert not bag.takeOobFlag()
