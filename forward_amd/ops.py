"""Tensor-level wrappers of the kernel launchers in ``libfwdmi.so``.

Each function validates that its operands are contiguous device tensors, allocates the output
with torch (device memory plumbing only) and calls one C-ABI launcher on torch's current
stream.  Nothing here computes: a missing GPU or library is an error, never a fallback.
"""
import ctypes as C

import numpy as np
import torch

from . import lib

_FDT = {torch.float32: lib.F32, torch.float16: lib.F16}
_IDT = {torch.int32: lib.I32, torch.int64: lib.I64}
MODES = {"sum": lib.OP_SUM, "mean": lib.OP_MEAN, "max": lib.OP_MAX, "square_sum": lib.OP_SQUARE_SUM}


def _dev(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError("%s must be a tensor in device memory (the HIP path has no CPU fallback)" % name)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t


def _p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _require(cond, what):
    """Argument checks that guard the launchers' memory accesses: raised, never compiled away."""
    if not cond:
        raise ValueError("forward_amd.ops: requirement not met: " + what)


def _stream(stream):
    s = torch.cuda.current_stream() if stream is None else stream
    return C.c_void_p(s.cuda_stream)


def _op(mode):
    return MODES[mode] if isinstance(mode, str) else int(mode)


def _ext(table, indices, out_dtype, include_last_offset=False, psw=None, max_indices=None, out_row_stride=0,
         oob_flag=None, flags=0, table_cost=None, square_sum_out=None, table_avg_len=None):
    x = lib.BagExt()
    x.table_dtype = _FDT[table.dtype]
    x.index_dtype = _IDT[indices.dtype]
    x.out_dtype = _FDT[out_dtype]
    x.include_last_offset = 1 if include_last_offset else 0
    x.per_sample_weights = psw.data_ptr() if psw is not None else None
    x.max_indices = max_indices.data_ptr() if max_indices is not None else None
    x.out_row_stride = int(out_row_stride)
    x.oob_flag = oob_flag.data_ptr() if oob_flag is not None else None
    x.flags = flags | (lib.BAG_TABLE_AVG_LEN if table_avg_len is not None else 0)
    x.table_cost = table_cost.ctypes.data if table_cost is not None else None
    x.square_sum_out = square_sum_out.data_ptr() if square_sum_out is not None else None
    x.table_avg_len = table_avg_len.ctypes.data if table_avg_len is not None else None
    return x


def embedding_bag(table, indices, offsets, mode="sum", per_sample_weights=None, include_last_offset=False,
                  data_offset=0, out_dtype=None, out=None, out_col=0, want_max_indices=False, oob_flag=None,
                  count=None, stream=None, with_square_sum=False):
    """Bags over a 1-D ``indices`` + ``offsets`` layout -> ``[n_bags, dim]``.

    ``out`` / ``out_col`` write a column block of an existing ``[n_bags, W]`` matrix.
    Returns ``out`` or ``(out, max_indices)``; with ``with_square_sum`` (mode "sum", no weights)
    ``(out, square_sums)``: both reductions from one pass over the rows.
    """
    table, indices, offsets = _dev(table, "table"), _dev(indices, "indices"), _dev(offsets, "offsets")
    if indices.dtype != offsets.dtype:
        raise TypeError("indices and offsets must share an integer dtype")
    offsets = offsets.reshape(-1)
    dim = table.shape[1]
    n_bags = offsets.numel() - (1 if include_last_offset else 0)
    odt = table.dtype if out_dtype is None else out_dtype
    stride = 0
    if out is None:
        out = torch.empty((n_bags, dim), dtype=odt, device=table.device)
        dst = out
    else:
        _dev(out, "out")
        _require(out.dim() == 2 and out.dtype == odt and out.shape[0] == n_bags,
                 'out is [n_bags, W] of the output dtype')
        _require(0 <= out_col and out_col + dim <= out.shape[1], '0 <= out_col and out_col + dim <= out.shape[1]')
        stride = out.shape[1]
        dst = out.reshape(-1)[out_col:]
    psw = None
    if per_sample_weights is not None:
        psw = _dev(per_sample_weights, "per_sample_weights")
        _require(psw.dtype == table.dtype and psw.numel() == indices.numel(),
                 'psw.dtype == table.dtype and psw.numel() == indices.numel()')
    mi = torch.empty((n_bags, dim), dtype=indices.dtype, device=table.device) if want_max_indices else None
    sq = None
    if with_square_sum:
        _require(stride == 0 and not want_max_indices, 'with_square_sum writes two packed [n_bags, dim] outputs')
        sq = torch.empty((n_bags, dim), dtype=odt, device=table.device)
    x = _ext(table, indices, odt, include_last_offset, psw, mi, stride, oob_flag, square_sum_out=sq)
    lib.check(lib.dll.fwdmi_embedding_bag(_p(indices), _p(offsets), _p(dst), indices.numel(), n_bags, _p(table),
                                          table.shape[0] if count is None else count, dim, data_offset, _op(mode),
                                          C.byref(x), _stream(stream)))
    if with_square_sum:
        return out, sq
    return (out, mi) if want_max_indices else out


def embedding_bag_fixed(table, indices, mode="sum", data_offset=0, out_dtype=None, oob_flag=None, stream=None,
                        with_square_sum=False):
    """Fixed-length bags: ``indices`` is ``[B, L]`` -> ``[B, dim]`` (``with_square_sum``: also the
    sums of squares, from the same pass)."""
    table, indices = _dev(table, "table"), _dev(indices, "indices")
    _require(indices.dim() == 2, 'indices.dim() == 2')
    b, l = indices.shape
    odt = table.dtype if out_dtype is None else out_dtype
    out = torch.empty((b, table.shape[1]), dtype=odt, device=table.device)
    sq = torch.empty_like(out) if with_square_sum else None
    x = _ext(table, indices, odt, oob_flag=oob_flag, square_sum_out=sq)
    lib.check(lib.dll.fwdmi_embedding_bag_fixed(_p(indices), _p(out), b, l, _p(table), table.shape[0], table.shape[1],
                                                data_offset, _op(mode), C.byref(x), _stream(stream)))
    return (out, sq) if with_square_sum else out


def gather(table, indices, data_offset=0, out_dtype=None, oob_flag=None, stream=None):
    """Plain row gather: ``[B, L]`` ids -> ``[B, L, dim]``."""
    table, indices = _dev(table, "table"), _dev(indices, "indices")
    _require(indices.dim() == 2, 'indices.dim() == 2')
    b, l = indices.shape
    odt = table.dtype if out_dtype is None else out_dtype
    out = torch.empty((b, l, table.shape[1]), dtype=odt, device=table.device)
    x = _ext(table, indices, odt, oob_flag=oob_flag)
    lib.check(lib.dll.fwdmi_gather(_p(indices), _p(out), b, l, _p(table), table.shape[0], table.shape[1],
                                   data_offset, C.byref(x), _stream(stream)))
    return out


def device_topology():
    """``(compute units, XCDs)`` of the current device as the bag launches see them."""
    cus, xcds = C.c_int32(0), C.c_int32(0)
    lib.check(lib.dll.fwdmi_bag_device_topology(C.byref(cus), C.byref(xcds)))
    return int(cus.value), int(xcds.value)


class MultiTableBatch:
    """Device-resident descriptor array for ``fwdmi_embedding_bag_multi``.

    Holds references to the tables / ids / offsets it points at so they stay alive.
    """

    def __init__(self, tables, indices, offsets, out_cols=None, data_offsets=None, per_sample_weights=None):
        _require(len(tables) == len(indices) == len(offsets) and tables,
                 'len(tables) == len(indices) == len(offsets) and tables')
        self.tables = [_dev(t, "table") for t in tables]
        self.indices = [_dev(i, "indices") for i in indices]
        self.offsets = [_dev(o, "offsets") for o in offsets]
        self.dim = self.tables[0].shape[1]
        self.n_bags = self.offsets[0].numel()
        self.n_tables = len(tables)
        out_cols = [t * self.dim for t in range(self.n_tables)] if out_cols is None else list(out_cols)
        data_offsets = [0] * self.n_tables if data_offsets is None else list(data_offsets)
        psw = [None] * self.n_tables if per_sample_weights is None else list(per_sample_weights)
        _require(len(psw) == self.n_tables, 'one per_sample_weights entry (or None) per table')
        self.weights = [None if w is None else _dev(w, "per_sample_weights") for w in psw]
        self.weighted = any(w is not None for w in self.weights)
        desc = np.zeros((self.n_tables, 8), np.int64)
        for t in range(self.n_tables):
            _require(self.tables[t].shape[1] == self.dim and self.tables[t].dtype == self.tables[0].dtype,
                     'self.tables[t].shape[1] == self.dim and self.tables[t].dtype == self.tables[0].dtype')
            _require(self.indices[t].dtype == self.indices[0].dtype == self.offsets[t].dtype,
                     'self.indices[t].dtype == self.indices[0].dtype == self.offsets[t].dtype')
            _require(self.offsets[t].numel() == self.n_bags, 'self.offsets[t].numel() == self.n_bags')
            _require(self.tables[t].dim() == 2 and self.tables[t].shape[0] > 0, 'every table is [rows > 0, dim]')
            _require((self.dim * self.tables[t].element_size()) % 16 != 0 or self.tables[t].data_ptr() % 16 == 0,
                     'tables of 16-byte-sliceable rows start on a 16-byte boundary')
            w = self.weights[t]
            _require(w is None or (w.dtype == self.tables[t].dtype and w.numel() == self.indices[t].numel()),
                     'per_sample_weights[t] has the table dtype and one entry per id')
            desc[t] = (self.tables[t].data_ptr(), self.indices[t].data_ptr(), self.offsets[t].data_ptr(),
                       self.tables[t].shape[0], self.indices[t].numel(), data_offsets[t], out_cols[t],
                       0 if w is None else w.data_ptr())
        self.width = max(out_cols) + self.dim
        self.total_indices = int(sum(i.numel() for i in self.indices))
        # mean ids per bag of every table: tables that differ much in it get runs of their own size
        self.table_avg_len = np.array([i.numel() / max(1, self.n_bags) for i in self.indices], np.float32)
        self.desc = torch.from_numpy(desc).to(self.tables[0].device)

    def default_table_cost(self):
        """The library's per-table cost estimate for the XCD segmentation (from the table sizes)."""
        nbytes = np.array([t.numel() * t.element_size() for t in self.tables], np.int64)
        cost = np.empty(self.n_tables, np.float32)
        lib.check(lib.dll.fwdmi_bag_table_cost(nbytes.ctypes.data, self.n_tables, cost.ctypes.data))
        return cost

    def forward(self, out=None, mode="sum", out_dtype=None, oob_flag=None, xcd_table_affinity=False, stream=None,
                table_cost=None):
        odt = self.tables[0].dtype if out_dtype is None else out_dtype
        if out is None:
            out = torch.empty((self.n_bags, self.width), dtype=odt, device=self.desc.device)
        _dev(out, "out")
        _require(out.dtype == odt and out.shape[0] == self.n_bags and out.shape[1] >= self.width,
                 'out.dtype == odt and out.shape[0] == self.n_bags and out.shape[1] >= self.width')
        cost = None
        if xcd_table_affinity:
            cost = self.default_table_cost() if table_cost is None else table_cost
            cost = np.ascontiguousarray(cost, np.float32)
            _require(cost.shape == (self.n_tables,), 'cost.shape == (self.n_tables,)')
        x = _ext(self.tables[0], self.indices[0], odt, out_row_stride=out.shape[1], oob_flag=oob_flag,
                 flags=(lib.BAG_XCD_TABLE_AFFINITY if xcd_table_affinity else 0) |
                       (lib.BAG_TABLE_WEIGHTS if self.weighted else 0), table_cost=cost,
                 table_avg_len=self.table_avg_len)
        avg = self.total_indices / max(1, self.n_bags * self.n_tables)
        lib.check(lib.dll.fwdmi_embedding_bag_multi(_p(self.desc), self.n_tables, self.n_bags, _p(out), self.dim,
                                                    _op(mode), avg, C.byref(x), _stream(stream)))
        return out


def embedding_bag_group(tables, indices, offsets, mode="sum", include_last_offset=False, out=None, out_dtype=None,
                        oob_flag=None, xcd_table_affinity=True, table_cost=None, per_sample_weights=None):
    """All tables of a sparse stage in one launch with this call's ids / offsets:
    ``[n_bags, T*dim]``, columns ``t*dim ..`` equal to ``embedding_bag(tables[t], indices[t], offsets[t])``.

    The table descriptors travel as kernel arguments on torch's current stream (with the launch itself,
    or for many tables through ``fwdmi_bag_tables_fill``), so nothing is staged or synchronised on the host.
    """
    n = len(tables)
    _require(n > 0 and len(indices) == n and len(offsets) == n, 'len(tables) == len(indices) == len(offsets) > 0')
    dim, tdt, idt = tables[0].shape[1], tables[0].dtype, indices[0].dtype
    n_off = offsets[0].numel()
    psw = [None] * n if per_sample_weights is None else list(per_sample_weights)
    _require(len(psw) == n, 'one per_sample_weights entry (or None) per table')
    weighted = any(w is not None for w in psw)
    desc = np.zeros((n, 8), np.int64)
    total = 0
    for t in range(n):
        tab, ids, off = _dev(tables[t], "table"), _dev(indices[t], "indices"), _dev(offsets[t], "offsets")
        if psw[t] is not None:
            w = _dev(psw[t], "per_sample_weights")
            _require(w.dtype == tab.dtype and w.numel() == ids.numel(),
                     'per_sample_weights[t] has the table dtype and one entry per id')
            desc[t, 7] = w.data_ptr()
        _require(tab.dim() == 2 and tab.shape[1] == dim and tab.dtype == tdt, 'tables share dim and dtype')
        _require(tab.shape[0] > 0, 'every table is [rows > 0, dim]')
        _require((dim * tab.element_size()) % 16 != 0 or tab.data_ptr() % 16 == 0,
                 'tables of 16-byte-sliceable rows start on a 16-byte boundary')
        _require(ids.dim() == 1 and ids.dtype == idt and off.dtype == idt, 'ids are 1-D; ids and offsets share a dtype')
        _require(off.numel() == n_off, 'every table has the same number of offsets')
        desc[t, :7] = (tab.data_ptr(), ids.data_ptr(), off.data_ptr(), tab.shape[0], ids.numel(), 0, t * dim)
        total += ids.numel()
    n_bags = n_off - (1 if include_last_offset else 0)
    _require(n_bags >= 0, 'offsets hold the trailing end offset when include_last_offset is set')
    odt = tdt if out_dtype is None else out_dtype
    if out is None:
        out = torch.empty((n_bags, n * dim), dtype=odt, device=tables[0].device)
    _dev(out, "out")
    _require(out.dtype == odt and out.dim() == 2 and out.shape[0] == n_bags and out.shape[1] >= n * dim,
             'out is [n_bags, >= T*dim] of the output dtype')
    cost = None
    if xcd_table_affinity:
        if table_cost is None:
            nbytes = np.array([t.numel() * t.element_size() for t in tables], np.int64)
            cost = np.empty(n, np.float32)
            lib.check(lib.dll.fwdmi_bag_table_cost(nbytes.ctypes.data, n, cost.ctypes.data))
        else:
            cost = np.ascontiguousarray(table_cost, np.float32)
            _require(cost.shape == (n,), 'table_cost has one entry per table')
    s = _stream(None)
    x = _ext(tables[0], indices[0], odt, include_last_offset=include_last_offset, out_row_stride=out.shape[1],
             oob_flag=oob_flag, flags=(lib.BAG_XCD_TABLE_AFFINITY if xcd_table_affinity else 0) |
             (lib.BAG_TABLE_WEIGHTS if weighted else 0), table_cost=cost)
    # up to lib.BAG_INLINE_TABLES descriptors travel with the launch as kernel arguments; more need a device array
    d_desc = None if n <= lib.BAG_INLINE_TABLES else torch.empty(n * 64, dtype=torch.uint8, device=tables[0].device)
    lib.check(lib.dll.fwdmi_embedding_bag_multi_host(desc.ctypes.data, n, _p(d_desc),
                                                     n_bags, _p(out), dim, _op(mode), total / max(1, n_bags * n),
                                                     C.byref(x), s))
    return out


def _params(gamma, beta, bias=None, ld=None):
    """gamma / beta (/ bias): fp32 device vectors of ``ld`` elements (the launchers index them by ld)."""
    g, b = _dev(gamma, "gamma"), _dev(beta, "beta")
    _require(g.dtype == torch.float32 and b.dtype == torch.float32,
             'g.dtype == torch.float32 and b.dtype == torch.float32')
    if bias is not None:
        _require(_dev(bias, "bias").dtype == torch.float32, '_dev(bias, "bias").dtype == torch.float32')
    if ld is not None:
        _require(g.numel() == ld and b.numel() == ld, 'gamma.numel() == beta.numel() == ld')
        _require(bias is None or bias.numel() == ld, 'bias.numel() == ld')
    return g, b, bias


def _out_like(out, ref, name="out"):
    """A caller-supplied result buffer: device, contiguous, same dtype and element count as ``ref``."""
    out = _dev(out, name)
    _require(out.dtype == ref.dtype and out.numel() == ref.numel(),
             '%s has the dtype and element count of the result' % name)
    return out


def skip_layer_norm(x, gamma, beta, skip=None, bias=None, eps=0.0, out=None, stream=None):
    """``LN(x (+ skip) (+ bias))`` over the last axis; gamma/beta/bias are fp32 device vectors."""
    x = _dev(x, "input")
    ld = x.shape[-1]
    g, b, bias = _params(gamma, beta, bias, ld)
    if skip is not None:
        _require(_dev(skip, "skip").shape == x.shape and skip.dtype == x.dtype,
                 '_dev(skip, "skip").shape == x.shape and skip.dtype == x.dtype')
    out = torch.empty_like(x) if out is None else _out_like(out, x)
    lib.check(lib.dll.fwdmi_skip_layer_norm(_stream(stream), ld, x.numel(), _p(x), _p(skip), _p(b), _p(g), _p(out),
                                            _p(bias), _FDT[x.dtype], eps))
    return out


def layer_norm(x, gamma, beta, bias=None, eps=0.0, out=None, stream=None):
    x = _dev(x, "input")
    ld = x.shape[-1]
    g, b, bias = _params(gamma, beta, bias, ld)
    out = torch.empty_like(x) if out is None else _out_like(out, x)
    lib.check(lib.dll.fwdmi_layer_norm(_stream(stream), ld, x.numel(), _p(x), _p(b), _p(g), _p(out), _p(bias),
                                       _FDT[x.dtype], eps))
    return out


def emb_layer_norm(input_ids, segment_ids, input_mask, word, pos, tok, gamma, beta, eps=0.0, oob_flag=None,
                   out=None, mask_idx=None, batch_major=False, skip=None, gamma2=None, beta2=None, bias2=None,
                   eps2=0.0, emb_out=None, stream=None):
    """BERT embedding + LayerNorm.  ids / mask are int32 ``[S, B]`` (``[B, S]`` with ``batch_major``);
    returns ``(out, mask_idx int32 [B])`` with ``out`` shaped like the ids plus ``H``.

    ``skip`` (+ ``gamma2``/``beta2``/``bias2``/``eps2``) fuses the SkipLayerNorm that consumes the
    embedding: ``out = LN2(LN(word+pos+tok) + skip (+ bias2))``; ``emb_out`` also keeps the first stage.
    """
    ids, seg = _dev(input_ids, "input_ids"), _dev(segment_ids, "segment_ids")
    msk = _dev(input_mask, "input_mask") if input_mask is not None else None
    _require(ids.dtype == torch.int32 and seg.dtype == torch.int32 and ids.dim() == 2 and seg.shape == ids.shape,
             'ids.dtype == torch.int32 and seg.dtype == torch.int32 and ids.dim() == 2 and seg.shape == ids.shape')
    word, pos, tok = _dev(word, "word"), _dev(pos, "pos"), _dev(tok, "tok")
    _require(word.dtype == pos.dtype == tok.dtype, 'word.dtype == pos.dtype == tok.dtype')
    _require(word.dim() == 2 and pos.dim() == 2 and tok.dim() == 2 and pos.shape[1] == tok.shape[1] == word.shape[1],
             'word, pos and tok are [rows, ld] with one ld')
    s, bsz = (ids.shape[1], ids.shape[0]) if batch_major else ids.shape
    ld = word.shape[1]
    g, b, _ = _params(gamma, beta, None, ld)
    _require(msk is None or (msk.dtype == torch.int32 and msk.shape == ids.shape),
             'input_mask is int32 and shaped like input_ids')
    if out is None:
        out = torch.empty(tuple(ids.shape) + (ld,), dtype=word.dtype, device=word.device)
    else:
        out = _dev(out, "out")
        _require(out.dtype == word.dtype and out.numel() == ids.numel() * ld, 'out holds ids.numel() * ld elements of the table dtype')
    if mask_idx is None and msk is not None:
        mask_idx = torch.empty((bsz,), dtype=torch.int32, device=word.device)
    elif mask_idx is not None:
        mask_idx = _dev(mask_idx, "mask_idx")
        _require(mask_idx.dtype == torch.int32 and mask_idx.numel() == bsz, 'mask_idx is int32 [B]')
        _require(msk is not None, 'mask_idx needs input_mask')
    x = lib.EmbExt()
    x.batch_major = 1 if batch_major else 0
    keep = []
    if skip is not None:
        g2, b2, bias2 = _params(gamma2, beta2, bias2, ld)
        _require(_dev(skip, "skip").dtype == word.dtype and skip.numel() == ids.numel() * ld,
                 '_dev(skip, "skip").dtype == word.dtype and skip.numel() == ids.numel() * ld')
        if emb_out is not None:
            _require(_dev(emb_out, "emb_out").dtype == word.dtype and emb_out.numel() == skip.numel(),
                     '_dev(emb_out, "emb_out").dtype == word.dtype and emb_out.numel() == skip.numel()')
        x.skip, x.gamma2, x.beta2 = skip.data_ptr(), g2.data_ptr(), b2.data_ptr()
        x.bias2 = bias2.data_ptr() if bias2 is not None else None
        x.emb_output = emb_out.data_ptr() if emb_out is not None else None
        x.eps2 = eps2
        keep = [g2, b2, bias2]
    lib.check(lib.dll.fwdmi_emb_layer_norm_ex(_stream(stream), s, bsz, ld, _p(ids), _p(seg), _p(msk), _p(b), _p(g),
                                              _p(word), _p(pos), _p(tok), word.shape[0], pos.shape[0], tok.shape[0],
                                              _p(out), _p(mask_idx), _FDT[word.dtype], eps, _p(oob_flag),
                                              C.byref(x)))
    del keep
    return out, mask_idx
