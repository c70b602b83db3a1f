"""Backward passes for a conjugate gradient pair (g.dzs == conj(g.dz), as under every real-valued loss).

The *_sym entry points compute the dz product only and write its conjugate to the dz* planes.  On a pair that is
conjugate bit for bit the two-product entry points compute the same sums for dz* as for dz, so the two agree to
rounding (not to the bit: the one-problem launch may take another block shape, which groups the four real products of
an element differently, and a two-problem launch that cuts its last blocks along K cuts only blocks of dz*).  Checked for
whichever kernel the shape takes (block kernels of each shape, cut along K, tail blocks, columns split off, the small-C
kernel with and without slices of K, the scalar-load kernel, the triangular mode), with and without accumulation.
That the loss layers and every backward pass of the CPU twin do produce conjugate pairs is checked on the oracle in
tests/test_oracle_math.py.
"""
import numpy as np
import pytest

from cnet_amd import ops
from tests.gpu_util import gpu, seeded  # noqa: F401

pytestmark = pytest.mark.gpu


def _pair(port, seed, shape):
    """A gradient carrier whose dz* planes are the exact conjugate of its dz planes."""
    re, im = seeded(port, seed, shape), seeded(port, seed + 1, shape)
    return [re, im, re.copy(), -im]


def _same(full, sym, what):
    """The one-product result is an exact conjugate pair and agrees with the two-product result to rounding (relative
    Frobenius distance over the four planes)."""
    f, s = full.host(), sym.host()
    assert np.array_equal(s[0], s[2]) and np.array_equal(s[1], -s[3]), (what, "dz* is not the conjugate of dz")
    num = np.sqrt(sum(float(np.sum((p.astype(np.float64) - q) ** 2)) for p, q in zip(f, s)))
    den = np.sqrt(sum(float(np.sum(p.astype(np.float64) ** 2)) for p in f))
    assert num / max(den, 1e-30) < 2e-6, (what, num / den)


def _prefilled(port, seed, rows, cols):
    """Two copies of a destination that already holds a conjugate pair (what accumulate = 1 adds to)."""
    base = _pair(port, seed, (rows, cols))
    return ops.Grad.from_host(base), ops.Grad.from_host(base)


# B, K (in), N (out)
LINEAR = [(4096, 1024, 1024), (512, 784, 256), (64, 784, 10), (300, 100, 37), (4096, 832, 784), (2048, 544, 544), (4096, 784, 10),
          (16, 16, 16), (2048, 550, 549), (1000, 512, 1000)]
# (2048, 550, 549): odd sizes, scalar-load kernel cut along K; (1000, 512, 1000): both reductions (over out = 1000 and over
# B = 1000) are not a whole number of chunks, so each product is two launches and the second adds to both halves


@pytest.mark.parametrize("B,K,N", LINEAR)
def test_linear_backward_of_a_conjugate_pair(gpu, port, B, K, N):
    g = ops.Grad.from_host(_pair(port, 7 * B + K + N, (B, N)))
    x = ops.CMat.from_host(seeded(port, 1, (B, K)), seeded(port, 2, (B, K)))
    w = ops.CMat.from_host(seeded(port, 3, (N, K)), seeded(port, 4, (N, K)))
    for accumulate in (0, 1):
        dx_full, dx_sym = _prefilled(port, 10, B, K)
        ops.linear_bwd_input(g, w, dx_full, accumulate=accumulate)
        ops.linear_bwd_input_sym(g, w, dx_sym, accumulate=accumulate)
        _same(dx_full, dx_sym, ("dx", accumulate))
        dw_full, dw_sym = _prefilled(port, 20, N, K)
        ops.linear_bwd_weight(g, x, dw_full, accumulate=accumulate)
        ops.linear_bwd_weight_sym(g, x, dw_sym, accumulate=accumulate)
        _same(dw_full, dw_sym, ("dw", accumulate))


@pytest.mark.parametrize("B,n", [(24, 96), (64, 784), (4096, 784), (1024, 1024), (100, 333)])
def test_dft_backward_of_a_conjugate_pair(gpu, port, B, n):
    g = ops.Grad.from_host(_pair(port, B + n, (B, n)))
    for accumulate in (0, 1):
        full, sym = _prefilled(port, 30, B, n)
        ops.dft_bwd(g, full, accumulate=accumulate)
        ops.dft_bwd_sym(g, sym, accumulate=accumulate)
        _same(full, sym, ("dft", accumulate))


@pytest.mark.parametrize("B,n", [(16, 64), (512, 256), (300, 520)])
def test_triangular_dft_backward_of_a_conjugate_pair(gpu, port, B, n):
    g = ops.Grad.from_host(_pair(port, 3 * B + n, (B, n)))
    for accumulate in (0, 1):
        full, sym = _prefilled(port, 40, B, n)
        ops.triang_dft_bwd(g, full, accumulate=accumulate)
        ops.triang_dft_bwd_sym(g, sym, accumulate=accumulate)
        _same(full, sym, ("triangular dft", accumulate))


def _exact(full, sym, what):
    """Elementwise passes use the arithmetic of the general kernel operation for operation: equal bits, not just close."""
    f, s = full.host(), sym.host()
    for p in range(4):
        assert np.array_equal(f[p], s[p]), (what, "plane", p)


def _dz_only(port, call, rows, cols, want, what):
    """The same pass with the dz* planes withheld (NULL): dz as before, the dz* planes of the destination untouched."""
    keep = _pair(port, 99, (rows, cols))
    d = ops.Grad.from_host(keep)
    call(d)
    h, w = d.host(), want.host()
    assert np.array_equal(h[0], w[0]) and np.array_equal(h[1], w[1]), (what, "dz")
    assert np.array_equal(h[2], keep[2]) and np.array_equal(h[3], keep[3]), (what, "dz* was written")


ELEMENTWISE = [(1, 1), (3, 7), (64, 784), (130, 36), (512, 2048), (33, 1028)]


@pytest.mark.parametrize("B,n", ELEMENTWISE)
def test_elementwise_backward_of_a_conjugate_pair(gpu, port, B, n):
    """CGelu, CRelu, Residual and Hadamard (per-row and shared weights): the one-gradient entry points against the general
    ones on an exactly conjugate pair, with and without accumulation, with and without the dz* planes."""
    g = ops.Grad.from_host(_pair(port, 5 * B + n, (B, n)))
    x = ops.CMat.from_host(seeded(port, 1, (B, n), 2.0), seeded(port, 2, (B, n), 2.0))
    v = ops.CMat.from_host(seeded(port, 3, (B, n), 0.05), seeded(port, 4, (B, n), 0.05))
    v1 = ops.CMat.from_host(seeded(port, 5, (1, n), 0.05), seeded(port, 6, (1, n), 0.05))
    for accumulate in (0, 1):
        for name, general, sym in (("gelu", ops.gelu_bwd, ops.gelu_bwd_sym), ("crelu", ops.crelu_bwd, ops.crelu_bwd_sym)):
            full, one = _prefilled(port, 50, B, n)
            general(x, g, full, accumulate=accumulate)
            sym(x, g, one, accumulate=accumulate)
            _exact(full, one, (name, accumulate))
            if not accumulate:
                _dz_only(port, lambda d: sym(x, g, d, mirror=False), B, n, full, name)
        fu, su = _prefilled(port, 60, B, n)
        fv, sv = _prefilled(port, 61, B, n)
        ops.residual_bwd(g, fu, fv, accumulate=accumulate)
        ops.residual_bwd_sym(g, su, sv, accumulate=accumulate)
        _exact(fu, su, ("residual du", accumulate)); _exact(fv, sv, ("residual dv", accumulate))
        # two incoming gradients added in the kernel against two passes, the second accumulating
        g2 = ops.Grad.from_host(_pair(port, 7 * B + n, (B, n)))
        fu, su = _prefilled(port, 62, B, n)
        fv, sv = _prefilled(port, 63, B, n)
        ops.residual_bwd_sym(g, fu, fv, accumulate=accumulate)
        ops.residual_bwd_sym(g2, fu, fv, accumulate=1)
        ops.residual_bwd_sym2(g, g2, su, sv, accumulate=accumulate)
        _exact(fu, su, ("residual, two consumers, du", accumulate)); _exact(fv, sv, ("residual, two consumers, dv", accumulate))
        for shared, vv in ((False, v), (True, v1)):
            fu, su = _prefilled(port, 70, B, n)
            fv, sv = _prefilled(port, 71, 1 if shared else B, n)
            ops.hadamard_bwd(x, vv, g, fu, fv, shared, accumulate=accumulate)
            ops.hadamard_bwd_sym(x, vv, g, su, sv, shared, accumulate=accumulate)
            _exact(fu, su, ("hadamard du", shared, accumulate)); _exact(fv, sv, ("hadamard dv", shared, accumulate))
            if not accumulate:
                keep = ops.Grad.from_host(_pair(port, 98, (1 if shared else B, n)))
                _dz_only(port, lambda d: ops.hadamard_bwd_sym(x, vv, g, d, keep, shared, mirror=False), B, n, fu, "hadamard")
                hk = keep.host()
                assert np.array_equal(hk[0], fv.host()[0]) and np.array_equal(hk[1], fv.host()[1])


@pytest.mark.parametrize("B,n", ELEMENTWISE + [(4096, 784)])
def test_hadamard_followed_by_cgelu_in_one_pass(gpu, port, B, n):
    """cnet_hadamard_cgelu_fwd / _bwd_sym against the two separate calls each way (equal bits: h, y, dh, du, dv), per-row and
    shared weights, with and without accumulation into du / dv, with and without the planes of dh; and against the oracle."""
    from tests.gpu_util import rel_c, TOL
    g = ops.Grad.from_host(_pair(port, 11 * B + n, (B, n)))
    xr, xi = seeded(port, 1, (B, n), 2.0), seeded(port, 2, (B, n), 2.0)
    x = ops.CMat.from_host(xr, xi)
    for shared in (False, True):
        rows_v = 1 if shared else B
        vr, vi = seeded(port, 3, (rows_v, n), 0.7), seeded(port, 4, (rows_v, n), 0.7)
        v = ops.CMat.from_host(vr, vi)
        h0, y0, h1, y1 = (ops.CMat.empty(B, n) for _ in range(4))
        ops.hadamard_fwd(x, v, h0, shared)
        ops.gelu_fwd(h0, y0)
        ops.hadamard_gelu_fwd(x, v, h1, y1, shared)
        for a, b in ((h0, h1), (y0, y1)):
            assert np.array_equal(a.host()[0], b.host()[0]) and np.array_equal(a.host()[1], b.host()[1]), ("forward", shared)
        if B * n <= 1 << 17:  # the oracle, sample by sample
            hr, hi = port.hadamard_fwd(xr, xi, vr if not shared else vr[0], vi if not shared else vi[0])
            assert rel_c(y1.host(), port.gelu_fwd(hr, hi)) < TOL
        for accumulate in (0, 1):
            dh0 = ops.Grad.empty(B, n)
            ops.gelu_bwd_sym(h0, g, dh0)
            fu, su = _prefilled(port, 70, B, n)
            fv, sv = _prefilled(port, 71, rows_v, n)
            ops.hadamard_bwd_sym(x, v, dh0, fu, fv, shared, accumulate=accumulate)
            dh1 = ops.Grad.from_host(_pair(port, 97, (B, n)))
            ops.hadamard_gelu_bwd_sym(x, v, g, dh1, su, sv, shared, accumulate=accumulate)
            _exact(dh0, dh1, ("dh", shared, accumulate))
            _exact(fu, su, ("du", shared, accumulate)); _exact(fv, sv, ("dv", shared, accumulate))
            # without the planes of dh, and without the dz* planes of du and dv
            nu, nv = _prefilled(port, 70, B, n)[0], _prefilled(port, 71, rows_v, n)[0]
            ops.hadamard_gelu_bwd_sym(x, v, g, None, nu, nv, shared, accumulate=accumulate, mirror=False)
            for got, want, keep_seed, r in ((nu, fu, 70, B), (nv, fv, 71, rows_v)):
                hg, hw, keep = got.host(), want.host(), _pair(port, keep_seed, (r, n))
                assert np.array_equal(hg[0], hw[0]) and np.array_equal(hg[1], hw[1]), ("dz", shared, accumulate)
                assert np.array_equal(hg[2], keep[2]) and np.array_equal(hg[3], keep[3]), ("dz* was written", shared)


@pytest.mark.parametrize("B,n", ELEMENTWISE + [(2048, 2048)])
def test_residual_and_cgelu_backward_in_one_pass(gpu, port, B, n):
    """cnet_residual_cgelu_bwd_sym against cnet_residual_bwd_sym2 (or _sym) followed by cnet_cgelu_bwd_sym: equal bits in du, dv
    and dh, with one and two consumers, with and without the planes of dv and the dz* planes."""
    g1 = ops.Grad.from_host(_pair(port, 13 * B + n, (B, n)))
    g2 = ops.Grad.from_host(_pair(port, 17 * B + n, (B, n)))
    h = ops.CMat.from_host(seeded(port, 1, (B, n), 2.0), seeded(port, 2, (B, n), 2.0))
    for two in (True, False):
        fu, fv, fh = (ops.Grad.empty(B, n) for _ in range(3))
        if two:
            ops.residual_bwd_sym2(g1, g2, fu, fv)
        else:
            ops.residual_bwd_sym(g1, fu, fv)
        ops.gelu_bwd_sym(h, fv, fh)
        su, sv, sh = (ops.Grad.from_host(_pair(port, 90 + k, (B, n))) for k in range(3))
        ops.residual_gelu_bwd_sym(g1, g2 if two else None, h, su, sv, sh)
        _exact(fu, su, ("du", two)); _exact(fv, sv, ("dv", two)); _exact(fh, sh, ("dh", two))
        keep = _pair(port, 91, (B, n))
        nu, nh = ops.Grad.from_host(keep), ops.Grad.from_host(keep)
        ops.residual_gelu_bwd_sym(g1, g2 if two else None, h, nu, None, nh, mirror=False)
        for got, want in ((nu, fu), (nh, fh)):
            hg, hw = got.host(), want.host()
            assert np.array_equal(hg[0], hw[0]) and np.array_equal(hg[1], hw[1]), ("dz", two)
            assert np.array_equal(hg[2], keep[2]) and np.array_equal(hg[3], keep[3]), ("dz* was written", two)


@pytest.mark.parametrize("B,n", [(3, 6), (64, 10), (5, 1024), (3, 2048), (4, 3000), (2, 4100), (2, 5001), (2, 32768)])
def test_loss_and_softmax_backward_of_a_conjugate_pair(gpu, port, B, n):
    """SoftMax (every row kernel: registers, two-pass, scalar), L2Out and CrossEntropy: one-gradient entry points against
    the general ones, equal bits."""
    g = ops.Grad.from_host(_pair(port, 9 * B + n, (B, n)))
    zr, zi = seeded(port, 1, (B, n)), seeded(port, 2, (B, n))
    z = ops.CMat.from_host(zr, zi)
    y, s = ops.CMat.empty(B, n), ops.Plane.empty(1, B)
    ops.l2norm_fwd(z, y, s)
    for accumulate in (0, 1):
        full, one = _prefilled(port, 80, B, n)
        ops.l2norm_bwd(z, s, g, full, accumulate=accumulate)
        ops.l2norm_bwd_sym(z, s, g, one, accumulate=accumulate)
        _exact(full, one, ("softmax", accumulate))
        if not accumulate:
            _dz_only(port, lambda d: ops.l2norm_bwd_sym(z, s, g, d, mirror=False), B, n, full, "softmax")
        full, one = _prefilled(port, 81, B, n)
        ops.l2out_bwd(z, full, accumulate=accumulate)
        ops.l2out_bwd_sym(z, one, accumulate=accumulate)
        _exact(full, one, ("l2out", accumulate))
    _dz_only(port, lambda d: ops.l2out_bwd_sym(z, d, mirror=False), B, n, _l2(z, B, n), "l2out")
    labels = ops.ints(port.randint(3, (B,), n))
    from cnet_amd import capi
    S, loss, am = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
    ops.cross_entropy_fwd(z, labels, S, loss, am, None)
    full, one = ops.Grad.empty(B, n), ops.Grad.empty(B, n)
    ops.cross_entropy_bwd(z, S, labels, full)
    ops.cross_entropy_bwd_sym(z, S, labels, one)
    _exact(full, one, "cross entropy")
    _dz_only(port, lambda d: ops.cross_entropy_bwd_sym(z, S, labels, d, mirror=False), B, n, full, "cross entropy")
    # forward pass and gradient in one launch: every result of the two calls, to the bit, with and without the normalised
    # planes and the dz* planes
    norm = ops.CMat.empty(B, n)
    ops.cross_entropy_fwd(z, labels, S, loss, am, norm)
    want = [S.download(), loss.download(), am.download()] + list(norm.host())
    for with_out in (True, False):
        S2, loss2, am2 = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
        norm2, both = ops.CMat.empty(B, n), ops.Grad.from_host(_pair(port, 98, (B, n)))
        ops.cross_entropy_fwd_bwd_sym(z, labels, S2, loss2, am2, both, out=norm2 if with_out else None)
        _exact(full, both, ("cross entropy, one launch", with_out))
        got = [S2.download(), loss2.download(), am2.download()] + (list(norm2.host()) if with_out else [])
        for a, b in zip(got, want):
            assert np.array_equal(a, b), ("cross entropy forward results, one launch", with_out)
        _dz_only(port, lambda d: ops.cross_entropy_fwd_bwd_sym(z, labels, S2, loss2, am2, d, out=norm2 if with_out else None, mirror=False),
                 B, n, full, "cross entropy, one launch")


def _l2(z, B, n):
    d = ops.Grad.empty(B, n)
    ops.l2out_bwd(z, d)
    return d


def test_matrix_products_of_a_conjugate_pair_without_the_mirror_planes(gpu, port):
    """The conjugate-pair products with the dz* planes withheld: dz as with them, nothing else written (block kernel, K
    cut, small-C kernel, DFT and triangular DFT)."""
    for B, K, N in [(512, 256, 256), (64, 784, 10), (4096, 784, 16), (300, 100, 37)]:
        g = ops.Grad.from_host(_pair(port, B + K + N, (B, N)))
        x = ops.CMat.from_host(seeded(port, 1, (B, K)), seeded(port, 2, (B, K)))
        w = ops.CMat.from_host(seeded(port, 3, (N, K)), seeded(port, 4, (N, K)))
        for accumulate in (0, 1):
            with_m, _ = _prefilled(port, 10, B, K)
            ops.linear_bwd_input_sym(g, w, with_m, accumulate=accumulate)
            if not accumulate:
                _dz_only(port, lambda d: ops.linear_bwd_input_sym(g, w, d, mirror=False), B, K, with_m, ("dx", B, K, N))
            with_m, _ = _prefilled(port, 20, N, K)
            ops.linear_bwd_weight_sym(g, x, with_m, accumulate=accumulate)
            if not accumulate:
                _dz_only(port, lambda d: ops.linear_bwd_weight_sym(g, x, d, mirror=False), N, K, with_m, ("dw", B, K, N))
    B, n = 100, 320
    g = ops.Grad.from_host(_pair(port, 5, (B, n)))
    for sym in (ops.dft_bwd_sym, ops.triang_dft_bwd_sym):
        with_m = ops.Grad.empty(B, n)
        sym(g, with_m)
        _dz_only(port, lambda d: sym(g, d, mirror=False), B, n, with_m, sym.__name__)


@pytest.mark.parametrize("overrides", [
    {"CNET_CGEMM_SKINNY": "0"},                            # small products on the block kernels (cut along K)
    {"CNET_CGEMM_TILE": "0", "CNET_CGEMM_COLSPLIT": "0"},  # 128 x 128 blocks (two accumulator sets, negated operand)
    {"CNET_CGEMM_TILE": "3", "CNET_CGEMM_TAIL": "1"},      # 64 x 64 blocks, tail blocks cut along K whenever possible
    {"CNET_CGEMM_TILE": "4"},                              # 64 x 64 blocks with two LDS stages
])
def test_conjugate_pairs_under_other_kernel_choices(gpu, overrides):
    """The tests of this file again, in a process whose tuning overrides (read once per process) send the same shapes to
    other kernels and block shapes: every epilogue and both partial-sum kernels write the conjugate half."""
    import os
    import subprocess
    import sys
    if os.environ.get("CNET_TEST_INNER"):
        pytest.skip("already the inner run")
    env = dict(os.environ, CNET_TEST_INNER="1", **overrides)
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-m", "gpu"], env=env,
                       capture_output=True, text=True, timeout=280, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
