"""cnet_batch_sum_noalloc, the column sum for callers that cannot allocate device memory: its partial sums live in an
array inside the library's image instead of the library workspace.  It has no counterpart upstream; it must give the
bits of cnet_batch_sum (same kernels, same slabs), also when a call follows one on a larger input that left its partial
sums in the shared array."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel  # noqa: F401

pytestmark = pytest.mark.gpu

UNSUPPORTED = -5


def both(m, ld=None, accumulate=0, start=None):
    rows, cols = m.shape
    ld = ld or cols
    wide = np.zeros((rows, ld), np.float32)
    wide[:, :cols] = m
    src = ops.Plane.from_host(wide).sub(0, cols)
    init = np.zeros((1, cols), np.float32) if start is None else start
    a, b = ops.Plane.from_host(init), ops.Plane.from_host(init)
    capi.call("cnet_batch_sum", src.ptr, src.ld, a.ptr, rows, cols, accumulate)
    capi.call("cnet_batch_sum_noalloc", src.ptr, src.ld, b.ptr, rows, cols, accumulate)
    return a.host(), b.host()


def test_no_alloc_column_sum_matches_the_allocating_one(gpu):
    rng = np.random.default_rng(5)
    big = rng.standard_normal((4099, 2048), dtype=np.float32)
    small = rng.standard_normal((130, 515), dtype=np.float32)       # odd width: scalar loads, fewer slabs
    for m in (big, small):                                           # two calls in a row, the second on a smaller input
        want, got = both(m)
        assert np.array_equal(want, got)
        assert rel(got, m.astype(np.float64).sum(0, keepdims=True)) < 1e-5
    # rows inside a wider buffer, and adding onto what the destination holds
    start = rng.standard_normal((1, 1024), dtype=np.float32)
    m = rng.standard_normal((777, 1024), dtype=np.float32)
    want, got = both(m, ld=1040, accumulate=1, start=start)
    assert np.array_equal(want, got)
    assert rel(got, start + m.astype(np.float64).sum(0, keepdims=True)) < 1e-5
    # one row, one column
    want, got = both(rng.standard_normal((1, 1), dtype=np.float32))
    assert np.array_equal(want, got)


def test_no_alloc_column_sum_refuses_what_its_array_cannot_hold(gpu):
    cols = 524288 + 4                          # one slab of partial sums is already longer than the static array
    src = ops.Plane.empty(4, cols, zero=True)
    dst = ops.Plane.empty(1, cols, zero=True)
    lib = capi.load()
    rc = lib.cnet_batch_sum_noalloc(src.ptr, src.ld, dst.ptr, 4, cols, 0)
    assert rc == UNSUPPORTED and "static scratch" in lib.cnet_last_error().decode()
    capi.call("cnet_batch_sum", src.ptr, src.ld, dst.ptr, 4, cols, 0)   # the allocating entry point takes it
    assert not dst.host().any()
