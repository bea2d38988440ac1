"""numpy-facing wrapper of the CPU checker in ``fwd_oracle.c``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.  Nothing in ``forward_amd/`` may import it.

Every function takes and returns host numpy arrays; fp16 data travels as ``np.float16``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfwd_oracle.so")

DT_F32, DT_F16, DT_I32, DT_I64 = 0, 1, 3, 10
OP_SUM, OP_MEAN, OP_MAX, OP_SQUARE_SUM, OP_GATHER = 0, 1, 2, 3, 999

_lib = None


def build(force=False):
    """Compile ``fwd_oracle.c`` with gcc (a second or two)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libfwd_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_embedding_bag.restype = ctypes.c_int64
        L.oracle_gather.restype = ctypes.c_int64
        L.oracle_emb_layer_norm.restype = ctypes.c_int64
        L.oracle_skip_layer_norm.restype = ctypes.c_int
        L.oracle_max_threads.restype = ctypes.c_int
        _lib = L
    return _lib


def set_threads(n):
    lib().oracle_set_threads(ctypes.c_int(int(n)))


def max_threads():
    return int(lib().oracle_max_threads())


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _fdt(a):
    if a.dtype == np.float32:
        return DT_F32
    if a.dtype == np.float16:
        return DT_F16
    raise TypeError("table / activation dtype must be float32 or float16, got %s" % a.dtype)


def _idt(a):
    if a.dtype == np.int32:
        return DT_I32
    if a.dtype == np.int64:
        return DT_I64
    raise TypeError("index dtype must be int32 or int64, got %s" % a.dtype)


def _np_f(dt):
    return np.float16 if dt == DT_F16 else np.float32


def half_to_float(h):
    h = np.ascontiguousarray(h).view(np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_half_to_float(_ptr(h), _ptr(out), ctypes.c_int64(h.size))
    return out


def float_to_half(f):
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, np.uint16)
    lib().oracle_float_to_half(_ptr(f), _ptr(out), ctypes.c_int64(f.size))
    return out.view(np.float16)


def embedding_bag(table, indices, offsets=None, op=OP_SUM, per_sample_weights=None,
                  include_last_offset=False, data_offset=0, out_dtype=None, want_max_indices=False,
                  out=None, out_col=0, count=None):
    """Bag reduction.  ``indices`` 1-D with ``offsets``, or 2-D ``[B, L]`` without.

    Returns ``(output, max_indices_or_None, n_out_of_range)``.  ``out``/``out_col`` write into a
    column block of an existing ``[B, W]`` matrix (the concatenated multi-table layout).
    """
    table = np.ascontiguousarray(table)
    indices = np.ascontiguousarray(indices)
    dim = table.shape[1]
    count = table.shape[0] if count is None else count
    tdt, idt = _fdt(table), _idt(indices)
    if offsets is None:
        assert indices.ndim == 2
        n_bags, fixed = indices.shape
        off = None
    else:
        offsets = np.ascontiguousarray(offsets).reshape(-1)
        assert offsets.dtype == indices.dtype
        fixed = 0
        n_bags = offsets.size - (1 if include_last_offset else 0)
        off = offsets
    odt = tdt if out_dtype is None else (DT_F16 if np.dtype(out_dtype) == np.float16 else DT_F32)
    if out is None:
        out = np.zeros((n_bags, dim), _np_f(odt))
        stride, view = dim, out
    else:
        assert out.flags.c_contiguous and out.dtype == _np_f(odt)
        stride = out.shape[1]
        view = out.reshape(-1)[out_col:]
    psw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=table.dtype)
    mi = np.zeros((n_bags, dim), indices.dtype) if want_max_indices else None
    oob = lib().oracle_embedding_bag(
        _ptr(indices), _ptr(off), _ptr(view), ctypes.c_int64(indices.size), ctypes.c_int64(n_bags),
        _ptr(table), ctypes.c_int64(count), ctypes.c_int(dim), ctypes.c_int64(data_offset),
        ctypes.c_int(op), ctypes.c_int(tdt), ctypes.c_int(idt), ctypes.c_int(odt), _ptr(psw),
        ctypes.c_int(1 if include_last_offset else 0), ctypes.c_int64(fixed),
        ctypes.c_int64(stride), _ptr(mi))
    return out, mi, int(oob)


def gather(table, indices, data_offset=0, out_dtype=None):
    """Plain row gather (op 999): ``[...]`` ids -> ``[..., dim]`` rows."""
    table = np.ascontiguousarray(table)
    indices = np.ascontiguousarray(indices)
    dim = table.shape[1]
    tdt = _fdt(table)
    odt = tdt if out_dtype is None else (DT_F16 if np.dtype(out_dtype) == np.float16 else DT_F32)
    out = np.zeros(indices.shape + (dim,), _np_f(odt))
    oob = lib().oracle_gather(_ptr(indices), _ptr(out), ctypes.c_int64(indices.size), _ptr(table),
                              ctypes.c_int64(table.shape[0]), ctypes.c_int(dim),
                              ctypes.c_int64(data_offset), ctypes.c_int(tdt),
                              ctypes.c_int(_idt(indices)), ctypes.c_int(odt))
    return out, int(oob)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def skip_layer_norm(x, gamma, beta, skip=None, bias=None, eps=0.0):
    """``LN(x (+ skip) (+ bias))`` over the last axis; output in ``x``'s dtype."""
    x = np.ascontiguousarray(x)
    ld = x.shape[-1]
    out = np.empty_like(x)
    if skip is not None:
        skip = np.ascontiguousarray(skip, dtype=x.dtype)
        assert skip.shape == x.shape
    g, b, bi = _f32(gamma), _f32(beta), _f32(bias)
    rc = lib().oracle_skip_layer_norm(ctypes.c_int(ld), ctypes.c_int64(x.size), _ptr(x), _ptr(skip),
                                      _ptr(b), _ptr(g), _ptr(out), _ptr(bi), ctypes.c_int(_fdt(x)),
                                      ctypes.c_double(eps))
    assert rc == 0
    return out


def layer_norm(x, gamma, beta, bias=None, eps=0.0):
    return skip_layer_norm(x, gamma, beta, None, bias, eps)


def emb_layer_norm(input_ids, segment_ids, input_mask, word, pos, tok, gamma, beta, eps=0.0):
    """ids/mask are int32 ``[S, B]``; returns ``(out [S,B,H], mask_idx int32 [B], n_oob)``."""
    ids = np.ascontiguousarray(input_ids, dtype=np.int32)
    seg = np.ascontiguousarray(segment_ids, dtype=np.int32)
    msk = np.ascontiguousarray(input_mask, dtype=np.int32)
    S, B = ids.shape
    word, pos, tok = (np.ascontiguousarray(a) for a in (word, pos, tok))
    assert word.dtype == pos.dtype == tok.dtype
    ld = word.shape[1]
    out = np.empty((S, B, ld), word.dtype)
    midx = np.empty((B,), np.int32)
    g, b = _f32(gamma), _f32(beta)
    oob = lib().oracle_emb_layer_norm(
        ctypes.c_int(S), ctypes.c_int(B), ctypes.c_int(ld), _ptr(ids), _ptr(seg), _ptr(msk), _ptr(b),
        _ptr(g), _ptr(word), _ptr(pos), _ptr(tok), ctypes.c_int(word.shape[0]),
        ctypes.c_int(pos.shape[0]), ctypes.c_int(tok.shape[0]), _ptr(out), _ptr(midx),
        ctypes.c_int(_fdt(word)), ctypes.c_double(eps))
    assert oob >= 0, "oracle_emb_layer_norm failed (%d)" % oob
    return out, midx, int(oob)
