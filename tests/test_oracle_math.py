"""Pins the CPU oracle against what the mathematics fixes, independent of any compiled upstream code:
fp64 closed forms (numpy complex128), DFT identities, finite differences of the real loss, and the
known-answer values held by the upstream tests (tests/test.h:458-471, 491-533; tests/gputests.h:195-198,
1470-1506).  A dropped term, a wrong sign, a transposed operand or a conj in the wrong place fails here.
"""
import numpy as np
import pytest

from oracle import binding as ob


def rel(a, b):
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def cplx(r, i):
    return r.astype(np.float64) + 1j * i.astype(np.float64)


def rnd(seed, *shape):
    return np.random.RandomState(seed).randn(*shape).astype(np.float32)


# ---------------------------------------------------------------- Linear
def test_linear_against_fp64_gemm(port):
    B, K, N = 5, 48, 20
    xr, xi, wr, wi = rnd(1, B, K), rnd(2, B, K), rnd(3, N, K), rnd(4, N, K)
    g4 = [rnd(10 + p, B, N) for p in range(4)]
    X, W, G, Gs = cplx(xr, xi), cplx(wr, wi), cplx(g4[0], g4[1]), cplx(g4[2], g4[3])
    yr, yi = port.linear_fwd(xr, xi, wr, wi)
    assert rel(cplx(yr, yi), X @ W.T) < 1e-6
    dx, dw = port.linear_bwd(xr, xi, wr, wi, g4)
    assert rel(cplx(dx[0], dx[1]), G @ W) < 1e-6
    assert rel(cplx(dx[2], dx[3]), Gs @ W.conj()) < 1e-6
    assert rel(cplx(dw[0], dw[1]), G.T @ X) < 1e-6
    assert rel(cplx(dw[2], dw[3]), Gs.T @ X.conj()) < 1e-6
    # the wrong variants are far away (guards the test itself)
    assert rel(cplx(dx[2], dx[3]), Gs @ W) > 0.5
    assert rel(cplx(yr, yi), X @ W.conj().T) > 0.5


# ---------------------------------------------------------------- Fourier
@pytest.mark.parametrize("n", [1, 2, 4, 8, 12, 100, 512, 784])
def test_dft_forward_is_unitary_dft_with_negative_sign(port, n):
    xr, xi = rnd(n, 3, n), rnd(n + 1, 3, n)
    yr, yi = port.dft_fwd(xr, xi)
    exact = np.fft.fft(cplx(xr, xi), axis=1) / np.sqrt(n)
    assert rel(cplx(yr, yi), exact) < 2e-4  # the float twiddle recurrence costs up to ~1e-4
    wrong = np.fft.ifft(cplx(xr, xi), axis=1) * np.sqrt(n)
    if n > 2:
        assert rel(cplx(yr, yi), wrong) > 0.5
    # unitarity
    assert abs(np.linalg.norm(cplx(yr, yi)) / np.linalg.norm(cplx(xr, xi)) - 1) < 2e-4


def test_dft_small_by_hand(port):
    # n=2: y = [x0+x1, x0-x1]/sqrt2 ; n=4 impulse at 1 -> (1,-i,-1,i)/2
    yr, yi = port.dft_fwd(np.array([[1, 2]], np.float32), np.array([[3, -1]], np.float32))
    assert np.allclose(cplx(yr, yi), np.array([[3 + 2j, -1 + 4j]]) / np.sqrt(2), atol=1e-6)
    e = np.zeros((1, 4), np.float32); e[0, 1] = 1
    yr, yi = port.dft_fwd(e, np.zeros_like(e))
    assert np.allclose(cplx(yr, yi), np.array([[1, -1j, -1, 1j]]) / 2, atol=1e-6)
    # impulse at 0 -> constant 1/sqrt(n)
    e = np.zeros((1, 784), np.float32); e[0, 0] = 1
    yr, yi = port.dft_fwd(e, np.zeros_like(e))
    # chirp-z path in float: ~7e-5 relative is the CPU path's own error at this length
    assert np.allclose(yr, 1 / np.sqrt(784), atol=1e-5) and np.allclose(yi, 0, atol=1e-5)


@pytest.mark.parametrize("n", [8, 100, 512])
def test_dft_backward_against_fp64(port, n):
    g4 = [rnd(20 + p, 2, n) for p in range(4)]
    dx = port.dft_bwd(g4)
    k = np.arange(n)
    F = np.exp(-2j * np.pi * np.outer(k, k) / n) / np.sqrt(n)
    G, Gs = cplx(g4[0], g4[1]), cplx(g4[2], g4[3])
    assert rel(cplx(dx[0], dx[1]), G @ F) < 2e-6
    assert rel(cplx(dx[2], dx[3]), Gs @ F.conj()) < 2e-6
    assert rel(cplx(dx[2], dx[3]), Gs @ F) > 0.5


def test_dft_matrix_reproduces_forward(port):
    n = 100
    fr, fi = port.dft_matrix(n)
    xr, xi = rnd(1, 4, n), rnd(2, 4, n)
    yr, yi = port.dft_fwd(xr, xi)
    assert rel(cplx(xr, xi) @ cplx(fr, fi).T, cplx(yr, yi)) < 1e-6


# ---------------------------------------------------------------- elementwise closed forms
def test_hadamard_residual_closed_forms(port):
    B, n = 3, 17
    ur, ui, vr, vi = rnd(1, B, n), rnd(2, B, n), rnd(3, B, n), rnd(4, B, n)
    g4 = [rnd(30 + p, B, n) for p in range(4)]
    U, V, G, Gs = cplx(ur, ui), cplx(vr, vi), cplx(g4[0], g4[1]), cplx(g4[2], g4[3])
    yr, yi = port.hadamard_fwd(ur, ui, vr, vi)
    assert rel(cplx(yr, yi), U * V) < 1e-6
    du, dv = port.hadamard_bwd(ur, ui, vr, vi, g4)
    assert rel(cplx(du[0], du[1]), G * V) < 1e-6 and rel(cplx(du[2], du[3]), Gs * V.conj()) < 1e-6
    assert rel(cplx(dv[0], dv[1]), G * U) < 1e-6 and rel(cplx(dv[2], dv[3]), Gs * U.conj()) < 1e-6
    # shared second operand: gradient is the sum over rows
    w_r, w_i = vr[0].copy(), vi[0].copy()
    du, dv = port.hadamard_bwd(ur, ui, w_r, w_i, g4)
    assert rel(cplx(dv[2], dv[3]), (Gs * U.conj()).sum(0)) < 1e-6
    assert rel(cplx(dv[0], dv[1]), (G * U).sum(0)) < 1e-6
    yr, yi = port.residual_fwd(ur, ui, vr, vi)
    assert np.array_equal(yr, ur + vr) and np.array_equal(yi, ui + vi)
    du, dv = port.residual_bwd(g4)
    for p in range(4):
        assert np.array_equal(du[p], g4[p]) and np.array_equal(dv[p], g4[p])


def test_gelu_against_fp64_formula(port):
    x = np.linspace(-6, 6, 2001).astype(np.float32).reshape(1, -1)
    y = (x[:, ::-1] * 0.7).copy()
    yr, yi = port.gelu_fwd(x, y)
    c = np.sqrt(2 / np.pi)

    def g(t):
        t = t.astype(np.float64)
        return 0.5 * t * (1 + np.tanh(c * (t + 0.044715 * t ** 3)))

    def gp(t):
        t = t.astype(np.float64)
        a = c * (t + 0.044715 * t ** 3)
        return 0.5 * (1 + np.tanh(a)) + 0.5 * t / np.cosh(a) ** 2 * c * (1 + 3 * 0.044715 * t ** 2)

    assert np.allclose(yr, g(x), atol=2e-6) and np.allclose(yi, g(y), atol=2e-6)
    g4 = [rnd(40 + p, *x.shape) for p in range(4)]
    dx = port.gelu_bwd(x, y, g4)
    G, Gs = cplx(g4[0], g4[1]), cplx(g4[2], g4[3])
    s, d = 0.5 * (gp(x) + gp(y)), 0.5 * (gp(x) - gp(y))
    assert rel(cplx(dx[0], dx[1]), G * s + Gs * d) < 1e-5
    assert rel(cplx(dx[2], dx[3]), G * d + Gs * s) < 1e-5


# ---------------------------------------------------------------- normalisation / losses
def test_softmax_is_l2_normalisation_with_closed_form_gradient(port):
    B, n = 3, 41
    zr, zi = rnd(1, B, n), rnd(2, B, n)
    g4 = [rnd(50 + p, B, n) for p in range(4)]
    Z, G, Gs = cplx(zr, zi), cplx(g4[0], g4[1]), cplx(g4[2], g4[3])
    S = (abs(Z) ** 2).sum(1, keepdims=True)
    yr, yi, S_o = port.softmax_fwd(zr, zi)
    assert rel(cplx(yr, yi), Z / np.sqrt(S)) < 1e-6 and np.allclose(S_o, S[:, 0], rtol=1e-6)
    dz = port.softmax_bwd(zr, zi, g4)
    A = (G * Z).sum(1, keepdims=True) + (Gs * Z.conj()).sum(1, keepdims=True)
    assert rel(cplx(dz[0], dz[1]), G / np.sqrt(S) - Z.conj() * A / (2 * S ** 1.5)) < 1e-5
    assert rel(cplx(dz[2], dz[3]), Gs / np.sqrt(S) - Z * A / (2 * S ** 1.5)) < 1e-5


def test_cross_entropy_properties(port):
    B, n = 6, 10
    zr, zi = rnd(1, B, n), rnd(2, B, n)
    labels = np.array([0, 9, 3, 3, 7, 1], np.int32)
    outr, outi, S, loss, pred = port.crossent_fwd(zr, zi, labels)
    p = outr.astype(np.float64) ** 2 + outi.astype(np.float64) ** 2
    assert np.allclose(p.sum(1), 1, atol=1e-6)
    assert np.allclose(loss, -np.log(p[np.arange(B), labels]), rtol=1e-5)
    assert np.array_equal(pred, np.argmax(zr.astype(np.float64) ** 2 + zi.astype(np.float64) ** 2, 1))
    dz = port.crossent_bwd(zr, zi, labels)
    Z = cplx(zr, zi)
    Sd = (abs(Z) ** 2).sum(1, keepdims=True)
    expect = Z / Sd
    m = abs(Z[np.arange(B), labels]) ** 2
    expect[np.arange(B), labels] = -Z[np.arange(B), labels] * (Sd[:, 0] - m) / (m * Sd[:, 0])
    assert rel(cplx(dz[2], dz[3]), expect) < 1e-5
    assert np.array_equal(dz[0], dz[2]) and np.array_equal(dz[1], -dz[3])  # dz = conj(dz*)
    # planted one-hot: loss 0, gradient at the label 0
    z = np.zeros((1, n), np.float32); z[0, 4] = 3
    _, _, _, l, pr = port.crossent_fwd(z, np.zeros_like(z), np.array([4], np.int32))
    assert l[0] == 0 and pr[0] == 4


def test_cross_entropy_ln2_case_of_upstream_batch_test(port):
    # rows {(1+2i),(1+2i)} padded to 6, label 0 -> p = 5/10 (tests/gputests.h:1470-1506 upstream)
    z_r = np.array([[1, 1, 0, 0, 0, 0], [3, 3, 0, 0, 0, 0], [5, 5, 0, 0, 0, 0]], np.float32)
    z_i = np.array([[2, 2, 0, 0, 0, 0], [4, 4, 0, 0, 0, 0], [6, 6, 0, 0, 0, 0]], np.float32)
    _, _, S, loss, pred = port.crossent_fwd(z_r, z_i, np.array([0, 1, 2], np.int32))
    assert np.allclose(loss[:2], np.log(2), rtol=1e-6)
    assert np.array_equal(S, np.array([10, 50, 122], np.float32))
    assert loss[2] == np.float32(-np.log(np.float32(1e-15)))  # label on a zero entry: clamped
    assert np.array_equal(pred, [0, 0, 0])  # ties: first index wins


def test_l2out_planted_values_of_upstream_test(port):
    # tests/gputests.h:195-198 upstream plants 1+2i and 3+4i
    zr = np.zeros((2, 6), np.float32); zi = np.zeros((2, 6), np.float32)
    zr[0, 0], zi[0, 0], zr[1, 1], zi[1, 1] = 1, 2, 3, 4
    assert np.array_equal(port.l2out_fwd(zr, zi), np.array([5, 25], np.float32))
    dz = port.l2out_bwd(zr, zi)
    assert np.array_equal(dz[0], zr) and np.array_equal(dz[1], -zi)
    assert np.array_equal(dz[2], zr) and np.array_equal(dz[3], zi)


def test_embedding_known_answers_of_upstream_tests(port):
    # tests/test.h:458-471 upstream: dz* (1+2i)+(7+8i) = 8+10i, (3+4i)+(9+10i) = 12+14i at token 2
    net = port.net()
    e = net.add(ob.EMBEDDING, 2, 3, 4)
    a = net.add(ob.L2OUT, 6, inputs=[e])
    b = net.add(ob.L2OUT, 6, inputs=[e])
    net.set_tokens(e, [2])
    net.plane(a, ob.DZS_RE)[:2] = [1, 3]; net.plane(a, ob.DZS_IM)[:2] = [2, 4]
    net.plane(b, ob.DZS_RE)[:2] = [7, 9]; net.plane(b, ob.DZS_IM)[:2] = [8, 10]
    net.node_backward(e)
    assert list(net.plane(e, ob.DZS_RE)[4:6]) == [8, 12] and list(net.plane(e, ob.DZS_IM)[4:6]) == [10, 14]
    assert not net.plane(e, ob.DZS_RE)[:4].any() and not net.plane(e, ob.DZS_RE)[6:].any()
    # tests/test.h:491-533 upstream: gather rows, zero padding
    table = rnd(5, 2, 8)
    net.plane(e, ob.RE)[:] = table[0]; net.plane(e, ob.IM)[:] = table[1]
    for toks in ([1, 3], [0], [2, 2, 2]):
        net.set_tokens(e, toks)
        net.node_forward(e)
        for s in (a, b):
            got = net.plane(s, ob.RE).reshape(3, 2)
            for k, t in enumerate(toks):
                assert np.array_equal(got[k], table[0].reshape(4, 2)[t])
            assert not got[len(toks):].any()
    # batch variant with -1 padding
    tok = np.array([[1, 3, -1], [0, -1, -1], [2, 2, 2]], np.int32)
    yr, yi = port.embedding_fwd(table[0].reshape(4, 2), table[1].reshape(4, 2), tok)
    assert np.array_equal(yr[0, :2], table[0][2:4]) and not yr[0, 4:].any() and not yr[1, 2:].any()
    gs = rnd(6, 2, 3, 6)
    dsr, dsi = port.embedding_bwd(4, 2, tok, gs[0], gs[1])
    want = np.zeros((4, 2)); 
    for b_ in range(3):
        for t_ in range(3):
            if tok[b_, t_] >= 0:
                want[tok[b_, t_]] += gs[0, b_, 2 * t_:2 * t_ + 2]
    assert np.allclose(dsr, want, atol=1e-6)


def test_sgd_update(port):
    zr, zi, dr, di = rnd(1, 50), rnd(2, 50), rnd(3, 50), rnd(4, 50)
    a, b = zr.copy(), zi.copy()
    port.sgd_update(a, b, dr, di, 0.25)
    assert np.array_equal(a, zr - np.float32(0.25) * dr) and np.array_equal(b, zi - np.float32(0.25) * di)


def test_adam_update_closed_forms(port):
    """beta = 0 is plain SGD (m = g, bias correction 1); from m = 0 the first step at any beta is also lr * g,
    because (1 - beta) g / (1 - beta^1) = g; later steps follow the textbook recursion in float64."""
    z, g = rnd(5, 2, 64), rnd(6, 2, 64)
    zr, zi, mr, mi = z[0].copy(), z[1].copy(), rnd(7, 64), rnd(8, 64)
    port.adam_update(zr, zi, mr, mi, g[0], g[1], 0.25, 0.0, 3)
    assert np.array_equal(mr, g[0]) and np.array_equal(mi, g[1])
    assert np.array_equal(zr, z[0] - np.float32(0.25) * g[0]) and np.array_equal(zi, z[1] - np.float32(0.25) * g[1])
    zr, zi, mr, mi = z[0].copy(), z[1].copy(), np.zeros(64, np.float32), np.zeros(64, np.float32)
    z64, m64 = z.astype(np.float64), np.zeros((2, 64))
    for t in range(5):
        gt = rnd(20 + t, 2, 64)
        port.adam_update(zr, zi, mr, mi, gt[0], gt[1], 0.1, 0.9, t)
        m64 = 0.9 * m64 + (1 - 0.9) * gt
        z64 = z64 - 0.1 * m64 / (1 - 0.9 ** (t + 1))
        if t == 0:
            assert np.allclose(zr, z[0] - 0.1 * gt[0], rtol=0, atol=1e-6)
        assert np.allclose(np.stack([mr, mi]), m64, atol=1e-6)
        assert np.allclose(np.stack([zr, zi]), z64, atol=2e-6)


def test_crelu_closed_form(port):
    x = rnd(9, 2, 500)
    x[:, :4] = [[0.0, 1.0, -0.0, 1.0], [1.0, 0.0, 1.0, -1.0]]  # zero parts do not pass (strict >)
    on = (x[0] > 0) & (x[1] > 0)
    yr, yi = port.crelu_fwd(x[0], x[1])
    assert np.array_equal(yr, np.where(on, x[0], 0)) and np.array_equal(yi, np.where(on, x[1], 0))
    assert not on[:4].any() and 50 < on.sum() < 200
    g4 = [rnd(10 + p, 500) for p in range(4)]
    for got, g in zip(port.crelu_bwd(x[0], x[1], g4), g4):
        assert np.array_equal(got, np.where(on, g, 0))


@pytest.mark.parametrize("n", [1, 2, 9, 64, 100])
def test_triang_fourier_is_masked_dft_matrix(port, n):
    """y = x T with T[i][o] = exp(-2 pi i (i o) / n) / sqrt n for i <= o, 0 below; backward is g T^T and g* conj(T)^T."""
    i, o = np.meshgrid(np.arange(n), np.arange(n), indexing="ij")
    T = np.where(i <= o, np.exp(-2j * np.pi * ((i * o) % n) / n) / np.sqrt(n), 0)
    x = rnd(n, 3, n) + 1j * rnd(n + 1, 3, n)
    yr, yi = port.triang_fwd(np.ascontiguousarray(x.real, np.float32), np.ascontiguousarray(x.imag, np.float32))
    assert rel(cplx(yr, yi), x @ T) < 2e-6
    if n > 2:  # the mask is one-sided: the full DFT differs
        F = np.exp(-2j * np.pi * ((i * o) % n) / n) / np.sqrt(n)
        assert rel(cplx(yr, yi), x @ F) > 0.1
    g4 = [rnd(40 + p, 3, n) for p in range(4)]
    dx = port.triang_bwd(g4)
    assert rel(cplx(dx[0], dx[1]), cplx(g4[0], g4[1]) @ T.T) < 2e-6
    assert rel(cplx(dx[2], dx[3]), cplx(g4[2], g4[3]) @ np.conj(T).T) < 2e-6


# ---------------------------------------------------------------- finite differences through whole nets
def _fd_check(port, build, in_len, seed, tol=3e-2, label=-1):
    """d(real loss)/d Re x = 2 Re dz*, d/d Im x = 2 Im dz*; dz = conj(dz*) for a real loss."""
    net, x, out = build(port)
    rng = np.random.RandomState(seed)
    x0 = (rng.randn(2, in_len) * 0.7).astype(np.float32)

    def loss_at(v):
        net.plane(x, ob.RE)[:] = v[0]; net.plane(x, ob.IM)[:] = v[1]
        net.forward()
        return float(net.loss(out, max(label, 0)))

    loss_at(x0)
    net.backward(label)
    dzs = net.plane(x, ob.DZS_RE).copy() + 1j * net.plane(x, ob.DZS_IM).copy()
    eps = 2e-2
    num = np.zeros(in_len, complex)
    for k in range(in_len):
        for part in (0, 1):
            vp, vm = x0.copy(), x0.copy()
            vp[part, k] += eps; vm[part, k] -= eps
            d = (loss_at(vp) - loss_at(vm)) / (2 * eps)
            num[k] += d if part == 0 else 1j * d
    assert rel(2 * dzs, num) < tol, (rel(2 * dzs, num), 2 * dzs[:3], num[:3])


def _chain(kinds):
    def build(lib):
        net = lib.net()
        n = 6
        x = net.add(ob.INPUT, n)
        cur = x
        for kind in kinds:
            if kind == ob.LINEAR:
                w = net.add(ob.INPUT, n * n)
                net.plane(w, ob.RE)[:] = rnd(77, n * n) * 0.4; net.plane(w, ob.IM)[:] = rnd(78, n * n) * 0.4
                cur = net.add(ob.LINEAR, n, n * n, inputs=[cur, w])
            elif kind == ob.HADAMARD:
                w = net.add(ob.INPUT, n)
                net.plane(w, ob.RE)[:] = rnd(79, n); net.plane(w, ob.IM)[:] = rnd(80, n)
                cur = net.add(ob.HADAMARD, n, inputs=[cur, w])
            elif kind == ob.RESIDUAL:
                cur = net.add(ob.RESIDUAL, n, inputs=[x, cur])
            else:
                cur = net.add(kind, n, inputs=[cur])
        return net, x, cur
    return build


@pytest.mark.parametrize("kinds", [
    [ob.L2OUT], [ob.LINEAR, ob.L2OUT], [ob.FOURIER, ob.GELU, ob.L2OUT], [ob.HADAMARD, ob.GELU, ob.L2OUT],
    [ob.GELU, ob.L2OUT], [ob.LINEAR, ob.GELU, ob.RESIDUAL, ob.L2OUT], [ob.SOFTMAX, ob.GELU, ob.L2OUT],
    [ob.FOURIER, ob.HADAMARD, ob.GELU, ob.LINEAR, ob.SOFTMAX, ob.GELU, ob.L2OUT],
    [ob.TRIANG_FOURIER, ob.L2OUT], [ob.LINEAR, ob.TRIANG_FOURIER, ob.GELU, ob.L2OUT],
])
def test_wirtinger_gradients_by_finite_differences(port, kinds):
    _fd_check(port, _chain(kinds), 6, seed=len(kinds))


@pytest.mark.parametrize("kinds", [[ob.CROSSENT], [ob.LINEAR, ob.GELU, ob.CROSSENT], [ob.FOURIER, ob.HADAMARD, ob.CROSSENT]])
def test_cross_entropy_gradient_by_finite_differences(port, kinds):
    _fd_check(port, _chain(kinds), 6, seed=11, label=2)


def _conj_gap(g4):
    a, b = g4[0] + 1j * g4[1], g4[2] + 1j * g4[3]
    return float(np.abs(b - np.conj(a)).max() / max(np.abs(a).max(), 1e-30))


def test_gradient_pairs_are_conjugate_under_a_real_loss(port):
    """The loss of CrossEntropy and L2Out is real, so dL/dz* = conj(dL/dz): the loss layers write such a pair exactly, and
    every backward pass maps a conjugate pair to a conjugate pair (exactly where the dz and dz* formulas mirror each other
    operation by operation, to rounding otherwise).  The *_sym entry points of the device library rest on this."""
    rs = np.random.RandomState(5)
    B, n = 6, 12
    f32 = lambda *s: rs.randn(*s).astype(np.float32)  # noqa: E731
    zr, zi, xr, xi = f32(B, n), f32(B, n), f32(B, n), f32(B, n)
    labels = rs.randint(0, n, B).astype(np.int32)
    sources = {"crossent": port.crossent_bwd(zr, zi, labels), "l2out": port.l2out_bwd(zr, zi)}
    for name, g in sources.items():
        assert _conj_gap(g) == 0.0, name
        g = [np.ascontiguousarray(p) for p in g]
        wr, wi = f32(n, n), f32(n, n)
        dx, dw = port.linear_bwd(xr, xi, wr, wi, g)
        assert _conj_gap(dx) == 0.0 and _conj_gap(dw) == 0.0, name
        assert _conj_gap(port.dft_bwd(g)) < 1e-6, name
        assert _conj_gap(port.triang_bwd(g)) < 1e-6, name
        du, dv = port.hadamard_bwd(xr, xi, zr, zi, g)
        assert _conj_gap(du) < 1e-6 and _conj_gap(dv) < 1e-6, name
        assert _conj_gap(port.gelu_bwd(xr, xi, g)) < 1e-6, name
        assert _conj_gap(port.crelu_bwd(xr, xi, g)) == 0.0, name
        assert _conj_gap(port.softmax_bwd(xr, xi, g)) < 1e-6, name
        for part in port.residual_bwd(g):
            assert _conj_gap(part) == 0.0, name
