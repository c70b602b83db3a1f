"""CrossEntropy, L2Out and SoftMax (L2 normalisation) on the GPU against the CPU oracle (upstream testCE / testL2 /
testSoftmax / testSoftMaxGradient / testBatch, tests/gputests.h:266, 181, 138, 691, 1454).  argmax and labels are
compared exactly."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,n", [(1, 1), (64, 10), (7, 333), (9, 1024), (5, 2049), (16, 32768)])
def test_cross_entropy(gpu, port, B, n):
    zr, zi = seeded(port, n, (B, n)), seeded(port, n + 1, (B, n))
    labels = port.randint(n + 2, (B,), n)
    if n > 5:
        zr[0, labels[0]] = zi[0, labels[0]] = 0.0   # label on an exactly-zero logit: both clamps
        zr[1 % B, 3], zi[1 % B, 3] = zr[1 % B, 2], zi[1 % B, 2]  # an exact tie
    outr, outi, S, loss, pred = port.crossent_fwd(zr, zi, labels)
    dz_o = port.crossent_bwd(zr, zi, labels)
    z, lab = ops.CMat.from_host(zr, zi), ops.ints(labels)
    out = ops.CMat.empty(B, n)
    s, l, am = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
    ops.cross_entropy_fwd(z, lab, s, l, am, out)
    dz = ops.Grad.empty(B, n)
    ops.cross_entropy_bwd(z, s, lab, dz)
    assert np.array_equal(am.download(), pred)          # bit-exact argmax
    assert rel(s.download(), S) < 1e-6
    assert np.allclose(l.download(), loss, rtol=2e-6, atol=2e-6)
    assert rel_c(out.host(), (outr, outi)) < 1e-6
    h = dz.host()
    assert rel_c(h[2:4], dz_o[2:4]) < 1e-5 and rel_c(h[0:2], dz_o[0:2]) < 1e-5
    # forward without the normalised output planes
    s2, l2, am2 = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
    ops.cross_entropy_fwd(z, lab, s2, l2, am2, None)
    assert np.array_equal(am2.download(), pred) and np.array_equal(l2.download(), l.download())


def test_cross_entropy_batch_case_of_upstream_test(gpu, port):
    # tests/gputests.h:1470-1506 upstream: three rows padded to 6, label k; row 0 and 1 give ln 2
    zr = np.array([[1, 1, 0, 0, 0, 0], [3, 3, 0, 0, 0, 0], [5, 5, 0, 0, 0, 0]], np.float32)
    zi = np.array([[2, 2, 0, 0, 0, 0], [4, 4, 0, 0, 0, 0], [6, 6, 0, 0, 0, 0]], np.float32)
    labels = np.array([0, 1, 2], np.int32)
    _, _, S, loss, pred = port.crossent_fwd(zr, zi, labels)
    s, l, am = capi.empty(3), capi.empty(3), capi.empty(3, np.int32)
    ops.cross_entropy_fwd(ops.CMat.from_host(zr, zi), ops.ints(labels), s, l, am, None)
    assert np.array_equal(s.download(), S) and np.array_equal(am.download(), pred)
    got = l.download()
    assert np.allclose(got[:2], np.log(2), rtol=1e-6) and np.allclose(got, loss, rtol=1e-6)


@pytest.mark.parametrize("B,n", [(64, 10), (5, 3000), (300, 64)])
def test_loss_kernels_store_into_page_locked_memory(gpu, port, B, n):
    """The `loss` argument of cnet_cross_entropy_fwd, cnet_cross_entropy_fwd_bwd_sym and cnet_l2out_fwd may point into
    page-locked host memory: the same values arrive there, readable once a ticket taken behind the call has been waited for."""
    import ctypes as C
    zr, zi = seeded(port, n, (B, n)), seeded(port, n + 1, (B, n))
    z, lab = ops.CMat.from_host(zr, zi), ops.ints(port.randint(n + 2, (B,), n))
    s, l, am = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
    ops.cross_entropy_fwd(z, lab, s, l, am, None)
    l2 = capi.empty(B)
    ops.l2out_fwd(z, l2)
    host = C.c_void_p()
    capi.call("cnet_host_alloc", 4 * 3 * B, C.byref(host))
    pinned = np.ctypeslib.as_array((C.c_float * (3 * B)).from_address(host.value))
    pinned[:] = -1.0
    dz = ops.Grad.empty(B, n)
    none = C.c_void_p(None)
    capi.call("cnet_cross_entropy_fwd", *z.p(), z.ld, lab.ptr, none, none, 0, s.ptr, host.value, am.ptr, B, n)
    capi.call("cnet_cross_entropy_fwd_bwd_sym", *z.p(), z.ld, lab.ptr, none, none, 0, s.ptr, host.value + 4 * B, am.ptr, *dz.p(), dz.ld, B, n)
    capi.call("cnet_l2out_fwd", *z.p(), z.ld, host.value + 8 * B, B, n)
    t = C.c_int64(-1)
    capi.call("cnet_copy_ticket", 0, C.byref(t))
    capi.call("cnet_copy_wait", t)
    want = l.download()
    assert np.array_equal(pinned[:B], want) and np.array_equal(pinned[B:2 * B], want)
    assert np.array_equal(pinned[2 * B:], l2.download())
    del pinned
    capi.call("cnet_host_free", host)


@pytest.mark.parametrize("B,n", [(2, 6), (64, 10), (2048, 2048), (3, 5001)])
def test_l2out(gpu, port, B, n):
    zr, zi = seeded(port, 1, (B, n)), seeded(port, 2, (B, n))
    if n == 6:
        zr[:] = 0; zi[:] = 0
        zr[0, 0], zi[0, 0], zr[1, 1], zi[1, 1] = 1, 2, 3, 4    # tests/gputests.h:195-198 upstream
    z = ops.CMat.from_host(zr, zi)
    loss = capi.empty(B)
    ops.l2out_fwd(z, loss)
    assert rel(loss.download(), port.l2out_fwd(zr, zi)) < 2e-6
    if n == 6:
        assert np.array_equal(loss.download(), [5, 25])
    dz = ops.Grad.empty(B, n)
    ops.l2out_bwd(z, dz)
    for a, b in zip(dz.host(), port.l2out_bwd(zr, zi)):
        assert np.array_equal(a, b)


# (B, n, ld): the row lengths walk every kernel the dispatcher can pick: rows held in registers (128-bit path up to 8192
# columns forward / 4096 backward), the two-pass kernels beyond that with one or four wavefronts per row, their scalar
# twins for lengths that are not a multiple of 4, and rows inside a wider buffer (ld > n).
SOFTMAX_CASES = [(1, 1, 0), (3, 6, 0), (7, 97, 0), (5, 1024, 0), (3, 2048, 0), (4, 3000, 0), (2, 4100, 0), (2, 5001, 0),
                 (2, 8196, 0), (3, 32768, 0), (2, 32772, 32780), (2, 1030, 1033)]


@pytest.mark.parametrize("B,n,ld", SOFTMAX_CASES)
def test_softmax_l2_normalisation(gpu, port, B, n, ld):
    ld = ld or n
    zr, zi = seeded(port, 1, (B, n)), seeded(port, 2, (B, n))
    g4 = [seeded(port, 5 + p, (B, n)) for p in range(4)]
    yr, yi, S = port.softmax_fwd(zr, zi)

    def padded(a):   # the rows inside a buffer ld wide; the padding must come back untouched
        w = np.full((B, ld), 7.0, np.float32)
        w[:, :n] = a
        return ops.Plane.from_host(w).sub(0, n)

    z, g = ops.CMat(padded(zr), padded(zi)), ops.Grad([padded(a) for a in g4])
    y, s = ops.CMat(padded(0 * zr), padded(0 * zr)), capi.empty(B)
    dz = ops.Grad([padded(0 * zr) for _ in range(4)])
    ops.l2norm_fwd(z, y, s)
    ops.l2norm_bwd(z, s, g, dz)
    assert rel_c(y.host(), (yr, yi)) < 1e-6 and rel(s.download(), S) < 1e-6
    h = dz.host()
    # the oracle's chain rule is O(n^2) per row (6 s for two rows of 32768): the longest rows compare their first row
    # only
    rows = slice(0, B) if n <= 8196 else slice(0, 1)
    dzo = port.softmax_bwd(zr[rows], zi[rows], [a[rows] for a in g4])
    assert rel_c([a[rows] for a in h[0:2]], dzo[0:2]) < TOL and rel_c([a[rows] for a in h[2:4]], dzo[2:4]) < TOL
    Z = zr.astype(np.float64) + 1j * zi
    G, Gs = g4[0].astype(np.float64) + 1j * g4[1], g4[2].astype(np.float64) + 1j * g4[3]
    Sd = (abs(Z) ** 2).sum(1, keepdims=True)
    A = (G * Z).sum(1, keepdims=True) + (Gs * Z.conj()).sum(1, keepdims=True)
    e1 = G / np.sqrt(Sd) - Z.conj() * A / (2 * Sd ** 1.5)
    e2 = Gs / np.sqrt(Sd) - Z * A / (2 * Sd ** 1.5)
    assert rel_c(h[0:2], (e1.real, e1.imag)) < 1e-5 and rel_c(h[2:4], (e2.real, e2.imag)) < 1e-5
    # accumulate adds a second copy onto what the planes hold
    ops.l2norm_bwd(z, s, g, dz, accumulate=1)
    h2 = dz.host()
    for p in range(4):
        assert rel(h2[p], 2.0 * h[p]) < 1e-6
    if ld > n:
        for pl in [y.re, y.im] + dz.planes:
            assert np.all(pl.owner.download().reshape(B, ld)[:, n:] == 7.0)
