"""Hadamard, CGelu, Residual, SGD update, zero fill and the CInput copies on the GPU against the CPU oracle
(upstream testHadamard / testGelu / testResidual / testUpdateInputs / testZeroGradient, tests/gputests.h:464, 517,
427, 1269, 641)."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (3, 7), (64, 784), (5, 1024), (130, 36), (2048, 2048)]


@pytest.mark.parametrize("B,n", SHAPES)
@pytest.mark.parametrize("shared", [False, True])
def test_hadamard(gpu, port, B, n, shared):
    ur, ui = seeded(port, 1, (B, n)), seeded(port, 2, (B, n))
    vshape = (n,) if shared else (B, n)
    vr, vi = seeded(port, 3, vshape, 0.05), seeded(port, 4, vshape, 0.05)
    g4 = [seeded(port, 5 + p, (B, n)) for p in range(4)]
    yr, yi = port.hadamard_fwd(ur, ui, vr, vi)
    du_o, dv_o = port.hadamard_bwd(ur, ui, vr, vi, g4)
    u, v, g = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi), ops.Grad.from_host(g4)
    y, du = ops.CMat.empty(B, n), ops.Grad.empty(B, n)
    dv = ops.Grad.empty(1 if shared else B, n)
    ops.hadamard_fwd(u, v, y, shared)
    ops.hadamard_bwd(u, v, g, du, dv, shared)
    assert rel_c(y.host(), (yr, yi)) < 1e-6
    hdu, hdv = du.host(), dv.host()
    assert rel_c(hdu[0:2], du_o[0:2]) < 1e-6 and rel_c(hdu[2:4], du_o[2:4]) < 1e-6
    want = [d.reshape(hdv[0].shape) for d in dv_o]
    assert rel_c(hdv[0:2], want[0:2]) < 1e-5 and rel_c(hdv[2:4], want[2:4]) < 1e-5
    # accumulate adds a second copy
    ops.hadamard_bwd(u, v, g, du, dv, shared, accumulate=1)
    hdv2 = dv.host()
    assert rel_c((hdv2[2] / 2, hdv2[3] / 2), want[2:4]) < 1e-5
    assert rel_c((du.host()[0] / 2, du.host()[1] / 2), du_o[0:2]) < 1e-6


@pytest.mark.parametrize("B,n", SHAPES)
def test_gelu(gpu, port, B, n):
    xr, xi = seeded(port, 1, (B, n), 2.0), seeded(port, 2, (B, n), 2.0)
    if n >= 7:
        xr[0, :7] = [0, -0.0, 10, -10, 30, -30, 1e-4]  # saturated and tiny arguments
    g4 = [seeded(port, 5 + p, (B, n)) for p in range(4)]
    yr, yi = port.gelu_fwd(xr, xi)
    dxo = port.gelu_bwd(xr, xi, g4)
    x, g = ops.CMat.from_host(xr, xi), ops.Grad.from_host(g4)
    y, dx = ops.CMat.empty(B, n), ops.Grad.empty(B, n)
    ops.gelu_fwd(x, y)
    ops.gelu_bwd(x, g, dx)
    hy, hdx = y.host(), dx.host()
    assert rel_c(hy, (yr, yi)) < 1e-5
    assert np.max(np.abs(hy[0] - yr)) < 2e-6 * max(1.0, np.max(np.abs(yr)))
    assert rel_c(hdx[0:2], dxo[0:2]) < 1e-5 and rel_c(hdx[2:4], dxo[2:4]) < 1e-5
    assert np.all(np.isfinite(hdx[0])) and np.all(np.isfinite(hy[0]))


@pytest.mark.parametrize("B,n", SHAPES)
def test_residual(gpu, port, B, n):
    ur, ui, vr, vi = [seeded(port, 1 + k, (B, n)) for k in range(4)]
    g4 = [seeded(port, 5 + p, (B, n)) for p in range(4)]
    u, v, g = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi), ops.Grad.from_host(g4)
    y, du, dv = ops.CMat.empty(B, n), ops.Grad.empty(B, n), ops.Grad.empty(B, n)
    ops.residual_fwd(u, v, y)
    ops.residual_bwd(g, du, dv)
    hy = y.host()
    assert np.array_equal(hy[0], ur + vr) and np.array_equal(hy[1], ui + vi)
    for a, b, c in zip(du.host(), dv.host(), g4):
        assert np.array_equal(a, c) and np.array_equal(b, c)
    ops.residual_bwd(g, du, dv, accumulate=1)
    assert np.array_equal(du.host()[3], g4[3] + g4[3])


def test_windows_of_wider_buffers(gpu, port):
    """Operands and results living at column offsets of concatenated input blocks (unaligned offset -> scalar path)."""
    B, n = 9, 20
    wide = seeded(port, 11, (B, 3 * n + 3))
    ur, ui = seeded(port, 1, (B, n)), seeded(port, 2, (B, n))
    yr, yi = port.gelu_fwd(ur, ui)
    for off in (4, 5):
        buf = ops.CMat(ops.Plane.from_host(wide), ops.Plane.from_host(wide))
        ops.gelu_fwd(ops.CMat.from_host(ur, ui), buf.sub(off, n))
        hr = buf.re.owner.download()
        assert rel(hr[:, off:off + n], yr) < 1e-5
        keep = np.ones(wide.shape[1], bool); keep[off:off + n] = False
        assert np.array_equal(hr[:, keep], wide[:, keep])


def test_sgd_update_zero_copy_add(gpu, port):
    n = 100003
    zr, zi, dr, di = [seeded(port, k, (1, n)) for k in range(4)]
    z = ops.CMat.from_host(zr, zi)
    d_re, d_im = ops.Plane.from_host(dr), ops.Plane.from_host(di)
    ops.sgd_update(z, d_re, d_im, 0.01)
    a, b = zr.copy(), zi.copy()
    port.sgd_update(a, b, dr, di, 0.01)
    hz = z.host()
    assert np.array_equal(hz[0], a) and np.array_equal(hz[1], b)
    assert not d_re.host().any() and not d_im.host().any()
    # zero fill of an odd byte range leaves its neighbours alone
    buf = capi.to_device(np.arange(1000, dtype=np.float32) + 1)
    capi.call("cnet_memset_zero", buf.ptr + 4 * 3, 4 * 501)
    h = buf.download()
    assert not h[3:504].any() and h[2] == 3 and h[504] == 505
    # copy / add of a window
    src = ops.Plane.from_host(seeded(port, 9, (7, 33)))
    dst = ops.Plane.empty(7, 33, ld=40, zero=True)
    ops.copy2d(src, dst)
    ops.add2d(src, dst)
    assert np.array_equal(dst.host(), 2 * src.host())
    # column sum over the batch (parameter gradient from per-row gradients), deterministic
    m = seeded(port, 10, (4099, 515))
    out = ops.Plane.empty(1, 515)
    ops.batch_sum(ops.Plane.from_host(m), out)
    first = out.host().copy()
    assert rel(first, m.astype(np.float64).sum(0, keepdims=True)) < 1e-6
    ops.batch_sum(ops.Plane.from_host(m), out)
    assert np.array_equal(out.host(), first)


def test_sgd_update_of_several_tensors_in_one_launch(gpu, port):
    """cnet_sgd_update_multi against the single-tensor entry point: same bits, odd lengths and empty tensors included."""
    import ctypes as C
    sizes = [7840, 784, 1, 0, 100003, 64, 4096, 12, 999, 50000, 8]  # more than one launch's worth of tensors
    zs, ds, ref = [], [], []
    for k, n in enumerate(sizes):
        m = max(n, 1)
        zr, zi, dr, di = [seeded(port, 10 * k + j, (1, m)) for j in range(4)]
        z = ops.CMat.from_host(zr, zi)
        d = (ops.Plane.from_host(dr), ops.Plane.from_host(di))
        z2 = ops.CMat.from_host(zr, zi)
        d2 = (ops.Plane.from_host(dr), ops.Plane.from_host(di))
        if n:
            capi.call("cnet_sgd_update", z2.re.ptr, z2.im.ptr, d2[0].ptr, d2[1].ptr, n, 0.03, 1)
        zs.append(z); ds.append(d); ref.append((z2, d2))
    arr = lambda ptrs: (C.c_void_p * len(ptrs))(*ptrs)
    lens = (C.c_int64 * len(sizes))(*sizes)
    capi.call("cnet_sgd_update_multi", len(sizes), arr([z.re.ptr for z in zs]), arr([z.im.ptr for z in zs]),
              arr([d[0].ptr for d in ds]), arr([d[1].ptr for d in ds]), lens, 0.03, 1)
    for n, z, d, (z2, d2) in zip(sizes, zs, ds, ref):
        a, b = z.host(), z2.host()
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), n
        assert np.array_equal(d[0].host(), d2[0].host()) and np.array_equal(d[1].host(), d2[1].host()), n
        if n:
            assert not d[0].host()[0, :n].any()


def test_add_of_several_arrays_in_one_launch(gpu, port):
    """cnet_add_multi: dst += src for a list of dense arrays (the gathers of all input functions of a net), odd lengths,
    empty entries and more entries than one launch takes included."""
    import ctypes as C
    sizes = [15680, 1568, 1, 0, 100003, 64, 4096, 12, 999, 50000, 8]
    srcs, dsts, want = [], [], []
    for k, n in enumerate(sizes):
        m = max(n, 1)
        a, b = seeded(port, 30 + 2 * k, (1, m)), seeded(port, 31 + 2 * k, (1, m))
        srcs.append(ops.Plane.from_host(a)); dsts.append(ops.Plane.from_host(b))
        w = b.copy(); w[0, :n] += a[0, :n]
        want.append(w)
    arr = lambda ptrs: (C.c_void_p * len(ptrs))(*ptrs)
    lens = (C.c_int64 * len(sizes))(*sizes)
    capi.call("cnet_add_multi", len(sizes), arr([p.ptr for p in srcs]), arr([p.ptr for p in dsts]), lens)
    for n, d, w in zip(sizes, dsts, want):
        assert np.array_equal(d.host(), w), n
