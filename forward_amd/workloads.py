"""Seeded synthetic inputs for the five named configurations of the embedding-side path.

Everything is numpy ``Generator(PCG64(seed))`` with ``seed = 1000 * config + variant`` and
explicit samplers (bounded Zipf by inverse CDF, Poisson, log-uniform), so two machines produce
the same bytes.  A ``scale`` < 1 shrinks row counts / batch so the same generator serves the
CPU-sized parity cases and the full-size bench.

Zipf ranks are scattered over the rows of a table by a fixed affine bijection
``row = (rank * A + C) mod rows`` (A prime, not dividing ``rows``), so hot rows are not
neighbours in memory.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

_PRIMES = (1000003, 1000033, 1000037, 1000039)


def rng_for(config, variant=0):
    return np.random.Generator(np.random.PCG64(1000 * int(config) + int(variant)))


def zipf_cdf(n, s):
    w = np.arange(1, n + 1, dtype=np.float64) ** (-float(s))
    c = np.cumsum(w)
    c /= c[-1]
    return c


def zipf_ranks(rng, n, s, size, cdf=None):
    """0-based ranks with P(rank = k) proportional to (k+1)^-s on [0, n)."""
    cdf = zipf_cdf(n, s) if cdf is None else cdf
    r = np.searchsorted(cdf, rng.random(size), side="left")
    return np.minimum(r, n - 1)


def scatter_ranks(ranks, rows):
    a = next(p for p in _PRIMES if rows % p != 0)
    return (ranks.astype(np.int64) * a + 12345) % rows


def offsets_from_lengths(lengths, dtype):
    off = np.zeros(lengths.size, np.int64)
    np.cumsum(lengths[:-1], out=off[1:])
    return off.astype(dtype)


@dataclass
class BagWorkload:
    """One EmbeddingBag call: a table plus an indices + offsets batch."""
    table: np.ndarray                  # [rows, dim] float32 / float16
    indices: np.ndarray                # [N] int32 / int64
    offsets: np.ndarray                # [B] same dtype, exclusive prefix sum of bag lengths
    lengths: np.ndarray                # [B] int64
    mode: str = "sum"
    per_sample_weights: Optional[np.ndarray] = None

    @property
    def n_bags(self):
        return int(self.offsets.size)

    def algorithmic_bytes(self, out_itemsize=None):
        """Every gathered row + its index, the offsets, the weights, and the output rows."""
        dim = self.table.shape[1]
        sw, si = self.table.itemsize, self.indices.itemsize
        so = sw if out_itemsize is None else out_itemsize
        n = int(self.indices.size)
        b = n * (dim * sw + si) + self.n_bags * si + self.n_bags * dim * so
        if self.per_sample_weights is not None:
            b += n * sw
        return b


def config1(variant=0):
    """64 bags, table 10000 x 64 fp32 ~N(0,1), lengths U{1..32}, int64 uniform ids, sum."""
    rng = rng_for(1, variant)
    table = rng.standard_normal((10000, 64)).astype(np.float32)
    lengths = rng.integers(1, 33, size=64)
    idx = rng.integers(0, 10000, size=int(lengths.sum())).astype(np.int64)
    return BagWorkload(table, idx, offsets_from_lengths(lengths, np.int64), lengths, "sum")


def config2(variant=0, table_dtype=np.float32, index_dtype=np.int32, mode="sum", weighted=False,
            rows=1_000_000, n_bags=4096, dim=128):
    """1M x 128 table ~N(0,0.05); 4096 bags, Poisson(20) lengths clipped to [0,200] with ~1 %
    forced empty; Zipf(1.05) ids."""
    rng = rng_for(2, variant)
    table = (rng.standard_normal((rows, dim), dtype=np.float32) * np.float32(0.05))
    table = table.astype(table_dtype)
    lengths = np.clip(rng.poisson(20.0, size=n_bags), 0, 200).astype(np.int64)
    lengths[rng.random(n_bags) < 0.01] = 0
    n = int(lengths.sum())
    idx = scatter_ranks(zipf_ranks(rng, rows, 1.05, n), rows).astype(index_dtype)
    psw = rng.random(n, dtype=np.float32).astype(table_dtype) if weighted else None
    return BagWorkload(table, idx, offsets_from_lengths(lengths, index_dtype), lengths, mode, psw)


@dataclass
class BertWorkload:
    """EmbLayerNorm inputs in the plugin-native [S, B] layout (+ SkipLayerNorm operands)."""
    word: np.ndarray
    pos: np.ndarray
    tok: np.ndarray
    gamma: np.ndarray
    beta: np.ndarray
    input_ids: np.ndarray              # int32 [S, B]
    segment_ids: np.ndarray            # int32 [S, B]
    input_mask: np.ndarray             # int32 [S, B]
    valid_len: np.ndarray              # int32 [B]
    eps: float = 1e-12
    skip: Optional[np.ndarray] = None  # residual [S, B, H]
    skip_bias: Optional[np.ndarray] = None
    skip_gamma: Optional[np.ndarray] = None
    skip_beta: Optional[np.ndarray] = None

    @property
    def n_tokens(self):
        return int(self.input_ids.size)

    def emb_algorithmic_bytes(self):
        h, sz = self.word.shape[1], self.word.itemsize
        s = self.input_ids.shape[0]
        return self.n_tokens * (2 * h * sz + 12) + (s + 2 + 2) * h * sz

    def skip_algorithmic_bytes(self):
        h, sz = self.word.shape[1], self.word.itemsize
        return self.n_tokens * 3 * h * sz


def _bert(config, variant, hidden, batch, seq, dtype, vocab=30522, max_pos=512, with_skip=False):
    rng = rng_for(config, variant)
    f = lambda *shape, mu=0.0, sd=0.02: (mu + sd * rng.standard_normal(shape)).astype(np.float32).astype(dtype)
    word, pos, tok = f(vocab, hidden), f(max_pos, hidden), f(2, hidden)
    gamma, beta = f(hidden, mu=1.0), f(hidden)
    lens = rng.integers(16, seq + 1, size=batch)
    ids = np.zeros((batch, seq), np.int32)
    seg = np.zeros((batch, seq), np.int32)
    msk = np.zeros((batch, seq), np.int32)
    for b in range(batch):
        n = int(lens[b])
        ids[b, :n] = rng.integers(1000, vocab, size=n)
        ids[b, 0] = 101
        split = int(rng.integers(0, n + 1))
        seg[b, split:n] = 1
        msk[b, :n] = 1
    w = BertWorkload(word, pos, tok, gamma, beta, np.ascontiguousarray(ids.T),
                     np.ascontiguousarray(seg.T), np.ascontiguousarray(msk.T), lens.astype(np.int32))
    if with_skip:
        w.skip = rng.standard_normal((seq, batch, hidden), dtype=np.float32).astype(dtype)
        w.skip_bias, w.skip_gamma, w.skip_beta = f(hidden), f(hidden, mu=1.0), f(hidden)
    return w


def config3(variant=0, dtype=np.float16, batch=32, seq=128):
    """BERT-base EmbLayerNorm: 30522/512/2 x 768, batch 32, seq 128."""
    return _bert(3, variant, 768, batch, seq, dtype)


def config5(variant=0, dtype=np.float16, batch=16, seq=512):
    """BERT-large EmbLayerNorm (H=1024, batch 16, seq 512) followed by SkipLayerNorm."""
    return _bert(5, variant, 1024, batch, seq, dtype, with_skip=True)


@dataclass
class MultiTableWorkload:
    """DLRM-style sparse stage: independent sum-mode tables over one batch of samples."""
    rows: List[int]
    dim: int
    n_bags: int
    indices: List[np.ndarray] = field(default_factory=list)   # per table int32 [N_t]
    offsets: List[np.ndarray] = field(default_factory=list)   # per table int32 [B]
    table_seeds: List[int] = field(default_factory=list)

    def n_indices(self):
        return int(sum(i.size for i in self.indices))

    def algorithmic_bytes(self, table_itemsize=2, out_itemsize=2, index_itemsize=4):
        n, t = self.n_indices(), len(self.rows)
        return (n * (self.dim * table_itemsize + index_itemsize) + t * self.n_bags * index_itemsize
                + t * self.n_bags * self.dim * out_itemsize)

    def device_table(self, t, torch):
        """Rows ~U(-0.05, 0.05) of table ``t`` as fp16, generated directly in HBM (seeded per
        table; a different stream of values than ``host_table``, for full-size runs)."""
        g = torch.Generator(device="cuda").manual_seed(self.table_seeds[t])
        x = torch.rand((self.rows[t], self.dim), generator=g, device="cuda", dtype=torch.float32)
        return ((x - 0.5) * 0.1).to(torch.float16)

    def host_table(self, t, dtype=np.float16):
        """Rows ~U(-0.05, 0.05) of table ``t`` (own seed, so tables can be made one at a time)."""
        rng = np.random.Generator(np.random.PCG64(self.table_seeds[t]))
        x = rng.random((self.rows[t], self.dim), dtype=np.float32)
        return ((x - np.float32(0.5)) * np.float32(0.1)).astype(dtype)


def _config4_ids(rng, rows, n_bags, len_cdf, max_len, len_s, idx_s):
    """One batch of the sparse stage: per table, Zipf bag lengths and Zipf ids scattered over the rows."""
    indices, offsets = [], []
    for r in rows:
        lengths = zipf_ranks(rng, max_len, len_s, n_bags, len_cdf).astype(np.int64) + 1
        n = int(lengths.sum())
        indices.append(scatter_ranks(zipf_ranks(rng, r, idx_s, n), r).astype(np.int32))
        offsets.append(offsets_from_lengths(lengths, np.int32))
    return indices, offsets


def config4(variant=0, n_tables=26, n_bags=65536, dim=128, min_rows=1e3, max_rows=1e7,
            len_s=1.1, idx_s=1.1, max_len=100):
    """26 tables, rows log-uniform in [1e3, 1e7]; bag lengths truncated Zipf(1.1) on 1..100
    (mean 16.3); ids Zipf(1.1) per table, int32.  Tables are produced lazily by ``host_table``."""
    rng = rng_for(4, variant)
    lo, hi = np.log10(min_rows), np.log10(max_rows)
    rows = [int(round(10 ** u)) for u in rng.uniform(lo, hi, size=n_tables)]
    w = MultiTableWorkload(rows, dim, n_bags)
    w.indices, w.offsets = _config4_ids(rng, rows, n_bags, zipf_cdf(max_len, len_s), max_len, len_s, idx_s)
    w.table_seeds = [1000 * 4 + 100 * (variant + 1) + t for t in range(n_tables)]
    return w


def config4_fresh_batch(w, batch, len_s=1.1, idx_s=1.1, max_len=100):
    """Another batch of samples for the tables of ``w`` (same rows, same table seeds): new bag
    lengths and ids from the same distributions, seeded by ``batch`` (>= 1; batch 0 is ``w`` itself).
    A serving loop never sees the same ids twice: the benchmark cycles through several of these."""
    if batch == 0:
        return w
    rng = rng_for(4, 500 + int(batch))
    b = MultiTableWorkload(list(w.rows), w.dim, w.n_bags, table_seeds=list(w.table_seeds))
    b.indices, b.offsets = _config4_ids(rng, w.rows, w.n_bags, zipf_cdf(max_len, len_s), max_len, len_s, idx_s)
    return b
