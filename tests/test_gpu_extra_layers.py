"""CRelu, TriangFourier and the Adam-style step on the device against the CPU path (upstream impl/relu.h:32-63,
impl/ft.h:139-189, impl/cfunc.h:273-287).  Upstream's own GPU tests expect "not supported" for these two layers
(tests/gputests.h:1319-1330) and drive adamUpdate against the CPU net (tests/gputests.h:1377-1378)."""
import numpy as np
import pytest

from cnet_amd import ops
from tests.gpu_util import gpu, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols,ld", [(1, 1, 1), (3, 7, 9), (64, 784, 784), (33, 128, 132), (128, 4096, 4096)])
def test_crelu(gpu, port, rows, cols, ld):
    xr, xi = seeded(port, cols, (rows, cols)), seeded(port, cols + 1, (rows, cols))
    xr[0, 0], xi[0, 0] = 0.0, 1.0  # a zero part does not pass
    g4 = [seeded(port, 10 + p, (rows, cols)) for p in range(4)]
    x, g = ops.CMat.from_host(xr, xi), ops.Grad.from_host(g4)
    y, dx = ops.CMat.empty(rows, cols, ld), ops.Grad.empty(rows, cols, ld)
    ops.crelu_fwd(x, y)
    ops.crelu_bwd(x, g, dx)
    yr, yi = port.crelu_fwd(xr, xi)
    want = port.crelu_bwd(xr, xi, g4)
    hy, hdx = y.host(), dx.host()
    assert np.array_equal(hy[0], yr) and np.array_equal(hy[1], yi)
    for a, b in zip(hdx, want):
        assert np.array_equal(a, b)
    ops.crelu_bwd(x, g, dx, accumulate=1)  # a second consumer adds
    for a, b in zip(dx.host(), want):
        assert np.array_equal(a, b + b)


@pytest.mark.parametrize("B,n", [(2, 1), (3, 2), (5, 9), (7, 100), (64, 784), (40, 512), (16, 2048)])
def test_triang_fourier(gpu, port, B, n):
    xr, xi = seeded(port, n, (B, n)), seeded(port, n + 1, (B, n))
    g4 = [seeded(port, n + 2 + p, (B, n)) for p in range(4)]
    x, g = ops.CMat.from_host(xr, xi), ops.Grad.from_host(g4)
    y, dx = ops.CMat.empty(B, n), ops.Grad.empty(B, n)
    ops.triang_dft_fwd(x, y)
    ops.triang_dft_bwd(g, dx)
    hy, hdx = y.host(), dx.host()
    yr, yi = port.triang_fwd(xr, xi)
    want = port.triang_bwd(g4)
    assert rel_c(hy, (yr, yi)) < TOL / 5
    assert rel_c(hdx[0:2], want[0:2]) < TOL / 5 and rel_c(hdx[2:4], want[2:4]) < TOL / 5
    # against the masked fp64 operator (what the device computes)
    i, o = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    T = np.where(i <= o, np.exp(-2j * np.pi * ((i * o) % n) / n) / np.sqrt(n), 0)
    e = (xr.astype(np.float64) + 1j * xi) @ T
    assert rel_c(hy, (e.real, e.imag)) < 2e-6
    e1 = (g4[0].astype(np.float64) + 1j * g4[1]) @ T.T
    e2 = (g4[2].astype(np.float64) + 1j * g4[3]) @ np.conj(T).T
    assert rel_c(hdx[0:2], (e1.real, e1.imag)) < 2e-6 and rel_c(hdx[2:4], (e2.real, e2.imag)) < 2e-6
    ops.triang_dft_bwd(g, dx, accumulate=1)
    assert rel_c(dx.host()[0:2], (2 * e1.real, 2 * e1.imag)) < 2e-6


def test_triang_fourier_last_output_is_full_dft_bin(gpu, port):
    """Column n-1 of the triangular operator is the complete DFT column, column 0 only keeps x_0 / sqrt n; checked at
    the benchmark transform length where most blocks below the diagonal are skipped."""
    B, n = 256, 4096
    xr, xi = seeded(port, 5, (B, n)), seeded(port, 6, (B, n))
    y, f = ops.CMat.empty(B, n), ops.CMat.empty(B, n)
    x = ops.CMat.from_host(xr, xi)
    ops.triang_dft_fwd(x, y)
    ops.dft_fwd(x, f)
    hy, hf = y.host(), f.host()
    assert np.allclose(hy[0][:, n - 1], hf[0][:, n - 1], atol=2e-5) and np.allclose(hy[1][:, n - 1], hf[1][:, n - 1], atol=2e-5)
    assert np.allclose(hy[0][:, 0], xr[:, 0] / 64, atol=1e-6) and np.allclose(hy[1][:, 0], xi[:, 0] / 64, atol=1e-6)
    rows = [0, 100, 255]
    yr, yi = port.triang_fwd(np.ascontiguousarray(xr[rows]), np.ascontiguousarray(xi[rows]))
    assert rel_c((hy[0][rows], hy[1][rows]), (yr, yi)) < TOL / 5


@pytest.mark.parametrize("n", [1, 1001, 1 << 16])
def test_adam_update_is_bit_equal_to_cpu(gpu, port, n):
    zr, zi = seeded(port, 1, (1, n)), seeded(port, 2, (1, n))
    mr, mi = np.zeros((1, n), np.float32), np.zeros((1, n), np.float32)
    z = ops.CMat.from_host(zr, zi)
    m_re, m_im = ops.Plane.from_host(mr), ops.Plane.from_host(mi)
    for t in range(4):
        dr, di = seeded(port, 10 + t, (1, n)), seeded(port, 20 + t, (1, n))
        d_re, d_im = ops.Plane.from_host(dr), ops.Plane.from_host(di)
        ops.adam_update(z, m_re, m_im, d_re, d_im, 0.05, 0.9, t)
        port.adam_update(zr, zi, mr, mi, dr, di, 0.05, 0.9, t)
        hz = z.host()
        assert np.array_equal(hz[0], zr) and np.array_equal(hz[1], zi)
        assert np.array_equal(m_re.host(), mr) and np.array_equal(m_im.host(), mi)
        assert not d_re.host().any() and not d_im.host().any()
