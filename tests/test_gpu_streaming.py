"""The elementwise kernels at sizes whose operands together exceed the 256 MB memory-side cache: there the launches take
the instantiations that carry the streaming (non-temporal) hint on every access, which the small parametrised cases of
test_gpu_elementwise.py never reach.  Results are compared with the CPU oracle on a subsample of rows (the layers act row
by row) and, for the batch sums of a shared parameter, over all rows (upstream testHadamard / testGelu / testResidual /
testUpdateInputs, tests/gputests.h:464, 517, 427, 1269)."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel, rel_c, TOL  # noqa: F401

pytestmark = pytest.mark.gpu

# 4352 x 4096 = 17.8 M elements = 71 MB per plane: four planes already exceed 256 MB
ROWS, COLS = 4352, 4096
SAMPLE = np.array([0, 1, 2, 3, 255, 256, 1023, 2048, 3000, 4095, 4096, 4200, 4349, 4350, 4351])


def planes(seed, count, sig=1.0):
    rng = np.random.default_rng(seed)
    return [(sig * rng.standard_normal((ROWS, COLS), dtype=np.float32)) for _ in range(count)]


def rows_of(arrs):
    return [np.ascontiguousarray(a[SAMPLE]) for a in arrs]


def test_gelu_and_crelu_streaming(gpu, port):
    xr, xi = planes(1, 2, 2.0)
    g4 = planes(2, 4)
    x, g = ops.CMat.from_host(xr, xi), ops.Grad.from_host(g4)
    y, dx = ops.CMat.empty(ROWS, COLS), ops.Grad.empty(ROWS, COLS)
    sx, sg = rows_of([xr, xi]), rows_of(g4)
    ops.gelu_fwd(x, y)
    ops.gelu_bwd(x, g, dx)
    assert rel_c(rows_of(y.host()), port.gelu_fwd(*sx)) < 1e-5
    h, want = rows_of(dx.host()), port.gelu_bwd(sx[0], sx[1], sg)
    assert rel_c(h[0:2], want[0:2]) < 1e-5 and rel_c(h[2:4], want[2:4]) < 1e-5
    ops.gelu_bwd(x, g, dx, accumulate=1)
    h2 = rows_of(dx.host())
    assert rel_c(h2[0:2], (2 * want[0], 2 * want[1])) < 1e-5 and rel_c(h2[2:4], (2 * want[2], 2 * want[3])) < 1e-5
    ops.crelu_fwd(x, y)
    ops.crelu_bwd(x, g, dx)
    for a, b in zip(rows_of(y.host()), port.crelu_fwd(*sx)):
        assert np.array_equal(a, b)
    for a, b in zip(rows_of(dx.host()), port.crelu_bwd(sx[0], sx[1], sg)):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("shared", [False, True])
def test_hadamard_streaming(gpu, port, shared):
    ur, ui = planes(3, 2)
    g4 = planes(4, 4)
    if shared:
        rng = np.random.default_rng(5)
        vr, vi = [0.05 * rng.standard_normal((1, COLS), dtype=np.float32) for _ in range(2)]
    else:
        vr, vi = planes(5, 2, 0.05)
    u, v, g = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi), ops.Grad.from_host(g4)
    y, du = ops.CMat.empty(ROWS, COLS), ops.Grad.empty(ROWS, COLS)
    dv = ops.Grad.empty(1 if shared else ROWS, COLS)
    ops.hadamard_fwd(u, v, y, shared)
    ops.hadamard_bwd(u, v, g, du, dv, shared)
    su, sg = rows_of([ur, ui]), rows_of(g4)
    sv = [vr[0], vi[0]] if shared else rows_of([vr, vi])
    assert rel_c(rows_of(y.host()), port.hadamard_fwd(su[0], su[1], sv[0], sv[1])) < 1e-6
    du_o, dv_o = port.hadamard_bwd(su[0], su[1], sv[0], sv[1], sg)
    hdu = rows_of(du.host())
    assert rel_c(hdu[0:2], du_o[0:2]) < 1e-6 and rel_c(hdu[2:4], du_o[2:4]) < 1e-6
    if shared:
        # the parameter gradient is the sum over ALL rows: the oracle runs over the whole batch
        _, dv_all = port.hadamard_bwd(ur, ui, vr[0], vi[0], g4)
        hdv = dv.host()
        want = [d.reshape(hdv[0].shape) for d in dv_all]
        assert rel_c(hdv[0:2], want[0:2]) < 1e-5 and rel_c(hdv[2:4], want[2:4]) < 1e-5
    else:
        hdv = rows_of(dv.host())
        assert rel_c(hdv[0:2], dv_o[0:2]) < 1e-6 and rel_c(hdv[2:4], dv_o[2:4]) < 1e-6


def test_residual_and_losses_streaming(gpu, port):
    ur, ui, vr, vi = planes(6, 4)
    u, v = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi)
    y = ops.CMat.empty(ROWS, COLS)
    ops.residual_fwd(u, v, y)
    hy = rows_of(y.host())
    assert np.array_equal(hy[0], (ur + vr)[SAMPLE]) and np.array_equal(hy[1], (ui + vi)[SAMPLE])
    del y, v
    # residual backward: 12 planes
    g4 = [ur, ui, vr, vi]
    g = ops.Grad([u.re, u.im] + [ops.Plane.from_host(vr), ops.Plane.from_host(vi)])
    du, dv = ops.Grad.empty(ROWS, COLS), ops.Grad.empty(ROWS, COLS)
    ops.residual_bwd(g, du, dv)
    for a, b, c in zip(rows_of(du.host()), rows_of(dv.host()), rows_of(g4)):
        assert np.array_equal(a, c) and np.array_equal(b, c)
    ops.residual_bwd(g, du, dv, accumulate=1)
    assert np.array_equal(du.host()[3][SAMPLE], 2 * vi[SAMPLE]) and np.array_equal(dv.host()[0][SAMPLE], 2 * ur[SAMPLE])
    del dv
    # L2Out backward (6 planes) and CrossEntropy backward (6 planes + the row sums) on z = u
    ops.l2out_bwd(u, du)
    for a, b in zip(rows_of(du.host()), port.l2out_bwd(ur[SAMPLE], ui[SAMPLE])):
        assert np.array_equal(a, b)
    labels = np.random.default_rng(7).integers(0, COLS, ROWS).astype(np.int32)
    s, loss, am = capi.empty(ROWS), capi.empty(ROWS), capi.empty(ROWS, np.int32)
    lab = ops.ints(labels)
    ops.cross_entropy_fwd(u, lab, s, loss, am, None)
    ops.cross_entropy_bwd(u, s, lab, du)
    _, _, S, l_o, pred = port.crossent_fwd(ur[SAMPLE], ui[SAMPLE], labels[SAMPLE])
    assert np.array_equal(am.download()[SAMPLE], pred) and rel(s.download()[SAMPLE], S) < 1e-6
    assert np.allclose(loss.download()[SAMPLE], l_o, rtol=2e-6, atol=2e-6)
    want = port.crossent_bwd(ur[SAMPLE], ui[SAMPLE], labels[SAMPLE])
    h = rows_of(du.host())
    assert rel_c(h[0:2], want[0:2]) < 1e-5 and rel_c(h[2:4], want[2:4]) < 1e-5
    # copy and add of one plane pair (2 planes: no hint at this size) and of a taller one that takes it
    src = ops.Plane(u.re.ptr, ROWS, COLS, COLS, u.re.owner)
    ops.copy2d(src, du.planes[0])
    ops.add2d(src, du.planes[0])
    assert np.array_equal(du.planes[0].host()[SAMPLE], 2 * ur[SAMPLE])


def test_parameter_steps_streaming(gpu, port):
    n = ROWS * COLS   # 4 planes of 71 MB (SGD), 6 planes (Adam-style step)
    rng = np.random.default_rng(8)
    zr, zi, dr, di, mr, mi = [rng.standard_normal((1, n), dtype=np.float32) for _ in range(6)]
    z = ops.CMat.from_host(zr, zi)
    d_re, d_im = ops.Plane.from_host(dr), ops.Plane.from_host(di)
    ops.sgd_update(z, d_re, d_im, 0.01, zero_grad=0)
    a, b = zr.copy(), zi.copy()
    port.sgd_update(a, b, dr.copy(), di.copy(), 0.01)
    hz = z.host()
    assert np.array_equal(hz[0], a) and np.array_equal(hz[1], b)
    assert np.array_equal(d_re.host(), dr)   # zero_grad = 0 leaves the gradient
    m_re, m_im = ops.Plane.from_host(mr), ops.Plane.from_host(mi)
    z = ops.CMat.from_host(zr, zi)
    ops.adam_update(z, m_re, m_im, d_re, d_im, 0.01, 0.9, 3)
    a, b, c, d = zr.copy(), zi.copy(), mr.copy(), mi.copy()
    port.adam_update(a, b, c, d, dr.copy(), di.copy(), 0.01, 0.9, 3)
    hz = z.host()
    assert np.array_equal(hz[0], a) and np.array_equal(hz[1], b)
    assert np.array_equal(m_re.host(), c) and np.array_equal(m_im.host(), d)
    assert not d_re.host().any() and not d_im.host().any()
