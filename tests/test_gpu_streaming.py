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


# ------------------------------------------------------------------------------------------------------------------------
# The one-gradient (`*_sym`) and fused entry points of the default path at the same size.  Each result is compared twice:
# on the sampled rows with the CPU oracle, and over ALL rows with the same entry point called on blocks of 544 rows, whose
# operands fit the cache so that they take the plain instantiation (these kernels act row by row: equal bits).
CHUNK = 544


def pair_planes(seed):
    re, im = planes(seed, 2)
    return [re, im, re, -im]


def in_chunks(call):
    for r0 in range(0, ROWS, CHUNK):
        call(r0, min(CHUNK, ROWS - r0))


def same_bits(a, b, what, planes_checked=4):
    for p, (u, v) in enumerate(zip(a.host()[:planes_checked], b.host()[:planes_checked])):
        assert np.array_equal(u, v), (what, "plane", p)


def against_oracle(got, want, what, tol=1e-5):
    h = rows_of(got.host())
    assert rel_c(h[0:2], want[0:2]) < tol, (what, "dz")
    assert rel_c(h[2:4], want[2:4]) < tol, (what, "dz*")


@pytest.mark.parametrize("accumulate,mirror", [(0, True), (1, True), (0, False)])
def test_gelu_and_crelu_backward_of_a_pair_streaming(gpu, port, accumulate, mirror):
    xr, xi = planes(11, 2, 2.0)
    g4 = pair_planes(12)
    x, g = ops.CMat.from_host(xr, xi), ops.Grad.from_host(g4)
    sx, sg = rows_of([xr, xi]), rows_of(g4)
    checked = 4 if mirror else 2
    for name, sym, oracle in (("gelu", ops.gelu_bwd_sym, port.gelu_bwd), ("crelu", ops.crelu_bwd_sym, port.crelu_bwd)):
        whole, parts = ops.Grad.empty(ROWS, COLS, zero=True), ops.Grad.empty(ROWS, COLS, zero=True)
        for _ in range(1 + accumulate):   # the second pass adds the same values again
            sym(x, g, whole, accumulate=accumulate, mirror=mirror)
            in_chunks(lambda r0, r: sym(x.rows_from(r0, r), g.rows_from(r0, r), parts.rows_from(r0, r), accumulate=accumulate,
                                        mirror=mirror))
        same_bits(whole, parts, name, checked)
        want = [(1 + accumulate) * w for w in oracle(sx[0], sx[1], sg)]
        h = rows_of(whole.host())
        assert rel_c(h[0:2], want[0:2]) < 1e-5, name
        if mirror:
            assert rel_c(h[2:4], want[2:4]) < 1e-5, name
        else:
            assert not h[2].any() and not h[3].any(), (name, "dz* was written")


@pytest.mark.parametrize("accumulate,mirror", [(0, True), (1, False)])
def test_residual_backward_of_a_pair_streaming(gpu, port, accumulate, mirror):
    g4, h4 = pair_planes(13), pair_planes(14)
    g, g2 = ops.Grad.from_host(g4), ops.Grad.from_host(h4)
    checked = 4 if mirror else 2
    for two in (False, True):
        wu, wv, pu, pv = (ops.Grad.empty(ROWS, COLS, zero=True) for _ in range(4))
        for _ in range(1 + accumulate):
            if two:
                ops.residual_bwd_sym2(g, g2, wu, wv, accumulate=accumulate, mirror=mirror)
                in_chunks(lambda r0, r: ops.residual_bwd_sym2(g.rows_from(r0, r), g2.rows_from(r0, r), pu.rows_from(r0, r),
                                                              pv.rows_from(r0, r), accumulate=accumulate, mirror=mirror))
            else:
                ops.residual_bwd_sym(g, wu, wv, accumulate=accumulate, mirror=mirror)
                in_chunks(lambda r0, r: ops.residual_bwd_sym(g.rows_from(r0, r), pu.rows_from(r0, r), pv.rows_from(r0, r),
                                                             accumulate=accumulate, mirror=mirror))
        same_bits(wu, pu, ("du", two), checked); same_bits(wv, pv, ("dv", two), checked)
        # Residual hands the incoming gradient(s) on unchanged (impl/residual.h:54-77 upstream)
        # (an accumulating pass adds the first gradient, then the second: (old + g1) + g2)
        want = [np.zeros((len(SAMPLE), COLS), np.float32) for _ in range(4)]
        for _ in range(1 + accumulate):
            for p, (a, b) in enumerate(zip(rows_of(g4), rows_of(h4))):
                want[p] = ((want[p] + a) + b if two else want[p] + a) if accumulate else (a + b if two else a)
        for got in (wu, wv):
            for p in range(checked):
                assert np.array_equal(got.planes[p].host()[SAMPLE], want[p]), (two, p)


@pytest.mark.parametrize("shared", [False, True])
def test_hadamard_backward_of_a_pair_streaming(gpu, port, shared):
    ur, ui = planes(15, 2)
    g4 = pair_planes(16)
    rng = np.random.default_rng(17)
    vr, vi = [0.7 * rng.standard_normal((1 if shared else ROWS, COLS), dtype=np.float32) for _ in range(2)]
    u, v, g = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi), ops.Grad.from_host(g4)
    su, sg = rows_of([ur, ui]), rows_of(g4)
    sv = [vr[0], vi[0]] if shared else rows_of([vr, vi])
    rv = 1 if shared else ROWS
    du_o, dv_o = port.hadamard_bwd(su[0], su[1], sv[0], sv[1], sg)
    for accumulate in (0, 1):
        wu, pu = ops.Grad.empty(ROWS, COLS, zero=True), ops.Grad.empty(ROWS, COLS, zero=True)
        wv, pv = ops.Grad.empty(rv, COLS, zero=True), ops.Grad.empty(rv, COLS, zero=True)
        for _ in range(1 + accumulate):
            ops.hadamard_bwd_sym(u, v, g, wu, wv, shared, accumulate=accumulate)
            # a shared weight row sums over the batch: the blocks of rows add to the same row one after the other
            in_chunks(lambda r0, r: ops.hadamard_bwd_sym(u.rows_from(r0, r), v if shared else v.rows_from(r0, r), g.rows_from(r0, r),
                                                         pu.rows_from(r0, r), pv if shared else pv.rows_from(r0, r), shared,
                                                         accumulate=1 if shared and r0 else accumulate))
        same_bits(wu, pu, ("du", shared, accumulate))
        against_oracle(wu, [(1 + accumulate) * w for w in du_o], ("du", shared, accumulate), 1e-6)
        if not shared:
            same_bits(wv, pv, ("dv", accumulate))
            against_oracle(wv, [(1 + accumulate) * w for w in dv_o], ("dv", accumulate), 1e-6)
        elif not accumulate:
            # another order of the batch sum than the blocks of rows: close, not equal; and the oracle over the whole batch
            hw, hp = wv.host(), pv.host()
            assert rel_c(hw[0:2], hp[0:2]) < 1e-5 and np.array_equal(hw[0], hw[2]) and np.array_equal(hw[1], -hw[3])
            _, dv_all = port.hadamard_bwd(ur, ui, vr[0], vi[0], g4)
            want = [d.reshape(hw[0].shape) for d in dv_all]
            assert rel_c(hw[0:2], want[0:2]) < 1e-5 and rel_c(hw[2:4], want[2:4]) < 1e-5


@pytest.mark.parametrize("shared", [False, True])
def test_hadamard_with_cgelu_in_one_pass_streaming(gpu, port, shared):
    ur, ui = planes(18, 2, 2.0)
    g4 = pair_planes(19)
    rng = np.random.default_rng(20)
    vr, vi = [0.7 * rng.standard_normal((1 if shared else ROWS, COLS), dtype=np.float32) for _ in range(2)]
    u, v, g = ops.CMat.from_host(ur, ui), ops.CMat.from_host(vr, vi), ops.Grad.from_host(g4)
    rv = 1 if shared else ROWS
    su, sg = rows_of([ur, ui]), rows_of(g4)
    sv = [vr[0], vi[0]] if shared else rows_of([vr, vi])
    wh, wy, ph, py = (ops.CMat.empty(ROWS, COLS) for _ in range(4))
    ops.hadamard_gelu_fwd(u, v, wh, wy, shared)
    in_chunks(lambda r0, r: ops.hadamard_gelu_fwd(u.rows_from(r0, r), v if shared else v.rows_from(r0, r), ph.rows_from(r0, r),
                                                  py.rows_from(r0, r), shared))
    for a, b in ((wh, ph), (wy, py)):
        assert np.array_equal(a.re.host(), b.re.host()) and np.array_equal(a.im.host(), b.im.host())
    hr, hi = port.hadamard_fwd(su[0], su[1], sv[0], sv[1])
    assert rel_c(rows_of(wh.host()), (hr, hi)) < 1e-6 and rel_c(rows_of(wy.host()), port.gelu_fwd(hr, hi)) < 1e-5
    del ph, py, wy
    dh_o = port.gelu_bwd(hr, hi, sg)
    du_o, dv_o = port.hadamard_bwd(su[0], su[1], sv[0], sv[1], dh_o)
    for with_dh in (True, False):
        wu, pu, wdh, pdh = (ops.Grad.empty(ROWS, COLS, zero=True) for _ in range(4))
        wv, pv = ops.Grad.empty(rv, COLS, zero=True), ops.Grad.empty(rv, COLS, zero=True)
        ops.hadamard_gelu_bwd_sym(u, v, g, wdh if with_dh else None, wu, wv, shared)
        in_chunks(lambda r0, r: ops.hadamard_gelu_bwd_sym(u.rows_from(r0, r), v if shared else v.rows_from(r0, r), g.rows_from(r0, r),
                                                          pdh.rows_from(r0, r) if with_dh else None, pu.rows_from(r0, r),
                                                          pv if shared else pv.rows_from(r0, r), shared,
                                                          accumulate=1 if shared and r0 else 0))
        same_bits(wu, pu, ("du", shared, with_dh)); same_bits(wdh, pdh, ("dh", shared, with_dh))
        against_oracle(wu, du_o, ("du", shared, with_dh))
        if with_dh:
            against_oracle(wdh, dh_o, ("dh", shared))
        if not shared:
            same_bits(wv, pv, ("dv", with_dh))
            against_oracle(wv, dv_o, ("dv", with_dh))
        else:
            hw, hp = wv.host(), pv.host()
            assert rel_c(hw[0:2], hp[0:2]) < 1e-5 and np.array_equal(hw[0], hw[2]) and np.array_equal(hw[1], -hw[3])


@pytest.mark.parametrize("two,with_dv,mirror", [(True, True, True), (False, False, True), (True, False, False)])
def test_residual_with_cgelu_backward_in_one_pass_streaming(gpu, port, two, with_dv, mirror):
    g4, k4 = pair_planes(21), pair_planes(22)
    hr, hi = planes(23, 2, 2.0)
    g1, g2, h = ops.Grad.from_host(g4), ops.Grad.from_host(k4), ops.CMat.from_host(hr, hi)
    checked = 4 if mirror else 2
    wu, wv, wh, pu, pv, ph = (ops.Grad.empty(ROWS, COLS, zero=True) for _ in range(6))
    ops.residual_gelu_bwd_sym(g1, g2 if two else None, h, wu, wv if with_dv else None, wh, mirror=mirror)
    in_chunks(lambda r0, r: ops.residual_gelu_bwd_sym(g1.rows_from(r0, r), g2.rows_from(r0, r) if two else None, h.rows_from(r0, r),
                                                      pu.rows_from(r0, r), pv.rows_from(r0, r) if with_dv else None,
                                                      ph.rows_from(r0, r), mirror=mirror))
    same_bits(wu, pu, "du", checked); same_bits(wv, pv, "dv", checked); same_bits(wh, ph, "dh", checked)
    summed = [np.ascontiguousarray((a + b)[SAMPLE] if two else a[SAMPLE]) for a, b in zip(g4, k4)]
    want = port.gelu_bwd(hr[SAMPLE], hi[SAMPLE], summed)
    hh, hu = rows_of(wh.host()), rows_of(wu.host())
    assert rel_c(hh[0:2], want[0:2]) < 1e-5 and np.array_equal(hu[0], summed[0]) and np.array_equal(hu[1], summed[1])
    if mirror:
        assert rel_c(hh[2:4], want[2:4]) < 1e-5 and np.array_equal(hu[2], summed[2]) and np.array_equal(hu[3], summed[3])
    else:
        assert not hh[2].any() and not hu[3].any()
    if with_dv:
        assert np.array_equal(wv.planes[0].host()[SAMPLE], summed[0])


@pytest.mark.parametrize("mirror", [True, False])
def test_loss_backward_of_a_pair_streaming(gpu, port, mirror):
    zr, zi = planes(24, 2)
    z = ops.CMat.from_host(zr, zi)
    checked = 4 if mirror else 2
    for accumulate in (0, 1):
        whole, parts = ops.Grad.empty(ROWS, COLS, zero=True), ops.Grad.empty(ROWS, COLS, zero=True)
        for _ in range(1 + accumulate):
            ops.l2out_bwd_sym(z, whole, accumulate=accumulate, mirror=mirror)
            in_chunks(lambda r0, r: ops.l2out_bwd_sym(z.rows_from(r0, r), parts.rows_from(r0, r), accumulate=accumulate, mirror=mirror))
        same_bits(whole, parts, ("l2out", accumulate), checked)
        want = port.l2out_bwd(zr[SAMPLE], zi[SAMPLE])
        for p in range(checked):
            assert np.array_equal(whole.planes[p].host()[SAMPLE], (1 + accumulate) * want[p]), ("l2out", accumulate, p)
    labels = np.random.default_rng(25).integers(0, COLS, ROWS).astype(np.int32)
    lab, s, loss, am = ops.ints(labels), capi.empty(ROWS), capi.empty(ROWS), capi.empty(ROWS, np.int32)
    ops.cross_entropy_fwd(z, lab, s, loss, am, None)

    class At:
        def __init__(self, arr, first):
            self.ptr = arr.ptr + 4 * first

    whole, parts = ops.Grad.empty(ROWS, COLS, zero=True), ops.Grad.empty(ROWS, COLS, zero=True)
    ops.cross_entropy_bwd_sym(z, s, lab, whole, mirror=mirror)
    in_chunks(lambda r0, r: ops.cross_entropy_bwd_sym(z.rows_from(r0, r), At(s, r0), At(lab, r0), parts.rows_from(r0, r), mirror=mirror))
    same_bits(whole, parts, "cross entropy", checked)
    want = port.crossent_bwd(zr[SAMPLE], zi[SAMPLE], labels[SAMPLE])
    h = rows_of(whole.host())
    assert rel_c(h[0:2], want[0:2]) < 1e-5 and (not mirror or rel_c(h[2:4], want[2:4]) < 1e-5)
    assert mirror or not (h[2].any() or h[3].any())


def test_softmax_streaming(gpu, port):
    """SoftMax rows held in registers (4096 columns) under the streaming policies: forward, backward with both halves and
    of a conjugate pair (upstream testSoftmax / testSoftMaxGradient, tests/gputests.h:138, 691)."""
    zr, zi = planes(26, 2)
    g4 = pair_planes(27)
    z, g = ops.CMat.from_host(zr, zi), ops.Grad.from_host(g4)

    class At:
        def __init__(self, arr, first):
            self.ptr = arr.ptr + 4 * first

    wy, py = ops.CMat.empty(ROWS, COLS), ops.CMat.empty(ROWS, COLS)
    ws, ps = ops.Plane.empty(1, ROWS), ops.Plane.empty(1, ROWS)
    ops.l2norm_fwd(z, wy, ws)
    in_chunks(lambda r0, r: ops.l2norm_fwd(z.rows_from(r0, r), py.rows_from(r0, r), At(ps, r0)))
    assert np.array_equal(wy.re.host(), py.re.host()) and np.array_equal(wy.im.host(), py.im.host())
    assert np.array_equal(ws.host(), ps.host())
    yr, yi, S = port.softmax_fwd(zr[SAMPLE], zi[SAMPLE])
    assert rel_c(rows_of(wy.host()), (yr, yi)) < 1e-6 and rel(ws.host()[0][SAMPLE], S) < 1e-6
    del wy, py
    want = port.softmax_bwd(np.ascontiguousarray(zr[SAMPLE]), np.ascontiguousarray(zi[SAMPLE]), rows_of(g4))
    for accumulate in (0, 1):
        for name, call, mirrors in (("both halves", ops.l2norm_bwd, (None,)), ("pair", ops.l2norm_bwd_sym, (True, False))):
            for mirror in mirrors:
                kw = {} if mirror is None else {"mirror": mirror}
                checked = 2 if mirror is False else 4
                whole, parts = ops.Grad.empty(ROWS, COLS, zero=True), ops.Grad.empty(ROWS, COLS, zero=True)
                for _ in range(1 + accumulate):
                    call(z, ws, g, whole, accumulate=accumulate, **kw)
                    in_chunks(lambda r0, r: call(z.rows_from(r0, r), At(ws, r0), g.rows_from(r0, r), parts.rows_from(r0, r),
                                                 accumulate=accumulate, **kw))
                same_bits(whole, parts, (name, accumulate, mirror), checked)
                h = rows_of(whole.host())
                assert rel_c(h[0:2], [(1 + accumulate) * w for w in want[0:2]]) < 1e-5, (name, accumulate, mirror)
                if checked == 4:
                    assert rel_c(h[2:4], [(1 + accumulate) * w for w in want[2:4]]) < 1e-5, (name, accumulate, mirror)
                else:
                    assert not h[2].any() and not h[3].any()
