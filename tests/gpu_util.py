"""Shared helpers of the GPU parity tests."""
import numpy as np
import torch


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view({2: np.uint16, 4: np.uint32, 8: np.uint64}[a.itemsize])


def assert_bits_equal(got, want, what=""):
    g, w = bits(got), bits(want)
    if not np.array_equal(g, w):
        bad = np.argwhere(g != w)
        i = tuple(bad[0])
        raise AssertionError("%s: %d of %d elements differ, first at %s: got %r want %r"
                             % (what, len(bad), g.size, i, got[i], want[i]))


# Tolerances of the parity bar: fp32 rel 1e-5 (+ an absolute floor for sums that cancel),
# fp16 abs 1e-2 / rel 5e-3 after fp32 accumulation.
def assert_close(got, want, dtype, scale=1.0):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    if np.dtype(dtype) == np.float16:
        np.testing.assert_allclose(got, want, rtol=5e-3, atol=1e-2)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * scale)
