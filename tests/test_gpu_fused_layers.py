"""Layers that run as one launch: Linear followed by CGelu (the activation applied to the accumulators of the matrix product
when they are stored).  The fused entry point must give the bits of the two separate calls, whichever kernel the shape takes
(block kernels of each shape, the register-staged kernel for odd sizes, a K that is not a whole number of chunks, the
small-C kernel with and without slices of K, blocks cut along K, tail blocks, columns split off), and agree with the CPU
oracle."""
import os
import subprocess
import sys

import numpy as np
import pytest

from cnet_amd import ops
from tests.gpu_util import gpu, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu

# B, K (in), N (out)
LINEAR = [(4096, 1024, 1024), (2048, 2048, 2048), (512, 784, 256), (64, 784, 10), (64, 784, 784), (300, 100, 37), (4096, 784, 784),
          (2048, 544, 544), (4096, 784, 10), (16, 16, 16), (257, 33, 7), (2048, 550, 549), (1000, 1000, 512), (256, 4096, 64)]


@pytest.mark.parametrize("B,K,N", LINEAR)
def test_linear_followed_by_cgelu_in_one_launch(gpu, port, B, K, N):
    xr, xi = seeded(port, B + K, (B, K)), seeded(port, B + K + 1, (B, K))
    wr, wi = seeded(port, N + 2, (N, K), K ** -0.5), seeded(port, N + 3, (N, K), K ** -0.5)
    x, w = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi)
    base = (seeded(port, 5, (B, N)), seeded(port, 6, (B, N)))
    for accumulate in (0, 1):
        h0, h1 = ops.CMat.from_host(*base), ops.CMat.from_host(*base)
        y0, y1 = ops.CMat.empty(B, N), ops.CMat.from_host(*base)
        ops.linear_fwd(x, w, h0, accumulate=accumulate)
        ops.gelu_fwd(h0, y0)
        ops.linear_gelu_fwd(x, w, h1, y1, accumulate=accumulate)
        for a, b, what in ((h0, h1, "pre-activation"), (y0, y1, "activation")):
            ha, hb = a.host(), b.host()
            assert np.array_equal(ha[0], hb[0]) and np.array_equal(ha[1], hb[1]), (what, accumulate)
    if B * K * N <= 1 << 26:   # the CPU path, sample by sample
        hr, hi = port.linear_fwd(xr, xi, wr, wi)
        ops.linear_gelu_fwd(x, w, h1, y1)
        assert rel_c(h1.host(), (hr, hi)) < TOL / 5
        assert rel_c(y1.host(), port.gelu_fwd(hr, hi)) < TOL / 5


def test_linear_cgelu_into_a_column_window(gpu, port):
    """Both results land in column windows of wider buffers (shared leading dimension) and leave the rest alone."""
    B, K, N, W = 70, 48, 40, 64
    x = ops.CMat.from_host(seeded(port, 1, (B, K)), seeded(port, 2, (B, K)))
    w = ops.CMat.from_host(seeded(port, 3, (N, K)), seeded(port, 4, (N, K)))
    base = seeded(port, 9, (B, W))
    hw = ops.CMat(ops.Plane.from_host(base), ops.Plane.from_host(base))
    yw = ops.CMat(ops.Plane.from_host(base), ops.Plane.from_host(base))
    ops.linear_gelu_fwd(x, w, hw.sub(8, N), yw.sub(8, N))
    h0, y0 = ops.CMat.empty(B, N), ops.CMat.empty(B, N)
    ops.linear_fwd(x, w, h0)
    ops.gelu_fwd(h0, y0)
    mask = np.ones(W, bool); mask[8:8 + N] = False
    for wide, want in ((hw, h0), (yw, y0)):
        for plane, ref in zip((wide.re.owner.download(), wide.im.owner.download()), want.host()):
            assert np.array_equal(plane[:, 8:8 + N], ref) and np.array_equal(plane[:, mask], base[:, mask])


@pytest.mark.parametrize("B,K,N", [(64, 784, 10), (64, 16, 16), (33, 7, 5), (16, 64, 12), (1, 3, 2), (200, 40, 24), (64, 784, 784),
                                   (1024, 256, 256), (4096, 784, 10), (1000, 100, 16), (300, 5, 1), (256, 1030, 3), (513, 260, 7),
                                   (257, 33, 12), (16384, 784, 10)])
def test_both_gradients_of_a_linear_in_one_call(gpu, port, B, K, N):
    """cnet_clinear_bwd_sym against cnet_clinear_bwd_input_sym + cnet_clinear_bwd_weight_sym: same bits, whether the two
    products share a launch (both small and on the same kernel: the first cases) or not, with each accumulate flag and with
    the dz* planes of either result left out.  The cases from (4096, 784, 10) on are narrow layers (few outputs) at batches
    beyond the small-C kernel: a K of 1 .. 16 for the input gradient, a reduction over the whole batch for the weights (at
    16384 rows in slices of 1024, more than two workgroups to a compute unit)."""
    gr, gi = seeded(port, B + 11, (B, N)), seeded(port, B + 12, (B, N))
    g = ops.Grad.from_host([gr, gi, gr, -gi])
    x = ops.CMat.from_host(seeded(port, K + 1, (B, K)), seeded(port, K + 2, (B, K)))
    w = ops.CMat.from_host(seeded(port, N + 3, (N, K)), seeded(port, N + 4, (N, K)))
    bx, bw = [seeded(port, 20 + p, (B, K)) for p in range(4)], [seeded(port, 30 + p, (N, K)) for p in range(4)]
    for acc_x, acc_w, mir_x, mir_w in ((0, 0, True, True), (1, 0, True, False), (0, 1, False, True), (1, 1, True, True)):
        dx0, dw0, dx1, dw1 = ops.Grad.from_host(bx), ops.Grad.from_host(bw), ops.Grad.from_host(bx), ops.Grad.from_host(bw)
        ops.linear_bwd_input_sym(g, w, dx0, accumulate=acc_x, mirror=mir_x)
        ops.linear_bwd_weight_sym(g, x, dw0, accumulate=acc_w, mirror=mir_w)
        ops.linear_bwd_sym(g, x, w, dx1, dw1, accumulate_dx=acc_x, accumulate_dw=acc_w, mirror_dx=mir_x, mirror_dw=mir_w)
        for a, b in ((dx0, dx1), (dw0, dw1)):
            for pa, pb in zip(a.host(), b.host()):
                assert np.array_equal(pa, pb), (acc_x, acc_w, mir_x, mir_w)
    if B * K * N <= 1 << 27:   # the CPU path on the same pair
        (xr, xi), (wr, wi) = x.host(), w.host()
        dxo, dwo = port.linear_bwd(xr, xi, wr, wi, [gr, gi, gr, -gi])
        dx1, dw1 = ops.Grad.empty(B, K), ops.Grad.empty(N, K)
        ops.linear_bwd_sym(g, x, w, dx1, dw1)
        assert rel_c(dx1.host()[0:2], dxo[0:2]) < TOL / 5 and rel_c(dx1.host()[2:4], dxo[2:4]) < TOL / 5
        assert rel_c(dw1.host()[0:2], dwo[0:2]) < TOL / 5 and rel_c(dw1.host()[2:4], dwo[2:4]) < TOL / 5


def test_backward_pass_of_a_narrow_linear_in_windows_of_wider_buffers(gpu):
    """Both gradients of a narrow layer (few outputs, many rows) with every operand a column window of a wider buffer, against
    numpy in complex128; what lies beside the windows stays untouched, and accumulation adds to what the windows held."""
    rs = np.random.RandomState(5)
    for B, K, N in [(700, 300, 10), (256, 7, 16), (1200, 1025, 2)]:
        def wide(rows, cols, pad_l, pad_r):
            buf = rs.randn(rows, pad_l + cols + pad_r).astype(np.float32)
            bufi = rs.randn(rows, pad_l + cols + pad_r).astype(np.float32)
            full = ops.CMat.from_host(buf, bufi)
            return full, full.sub(pad_l, cols), (buf + 1j * bufi)[:, pad_l:pad_l + cols].astype(np.complex128), buf, bufi
        _, g, G, _, _ = wide(B, N, 3, 2)
        _, x, X, _, _ = wide(B, K, 1, 4)
        _, w, W, _, _ = wide(N, K, 5, 0)
        gg = ops.Grad([g.re, g.im, g.re, g.im])   # only the dz planes are read
        for acc in (0, 1):
            dxf, dx, DX0, dxb, dxbi = wide(B, K, 2, 3)
            dwf, dw, DW0, dwb, dwbi = wide(N, K, 4, 1)
            dxs, dws = ops.CMat.empty(B, K, ld=K + 5, zero=True), ops.CMat.empty(N, K, ld=K + 5, zero=True)   # the leading dimension of the windows
            ops.linear_bwd_sym(gg, x, w, ops.Grad([dx.re, dx.im, dxs.re, dxs.im]), ops.Grad([dw.re, dw.im, dws.re, dws.im]),
                               accumulate_dx=acc, accumulate_dw=acc)
            want_dx, want_dw = G @ W + (DX0 if acc else 0), G.T @ X + (DW0 if acc else 0)
            for full, window, want, b_re, b_im, pad_l, cols in ((dxf, dx, want_dx, dxb, dxbi, 2, K), (dwf, dw, want_dw, dwb, dwbi, 4, K)):
                hr, hi = full.re.owner.download(), full.im.owner.download()
                got = (hr + 1j * hi)[:, pad_l:pad_l + cols]
                assert np.linalg.norm(got - want) / np.linalg.norm(want) < 2e-6, (B, K, N, acc)
                mask = np.ones(hr.shape[1], bool); mask[pad_l:pad_l + cols] = False
                assert np.array_equal(hr[:, mask], b_re[:, mask]) and np.array_equal(hi[:, mask], b_im[:, mask])
            # the dz* planes: conjugates of what was added
            (sr, si), (tr, ti) = dxs.host(), dws.host()
            assert np.linalg.norm((sr + 1j * si) - np.conj(G @ W)) / np.linalg.norm(G @ W) < 2e-6
            assert np.linalg.norm((tr + 1j * ti) - np.conj(G.T @ X)) / np.linalg.norm(G.T @ X) < 2e-6


@pytest.mark.parametrize("overrides", [
    {"CNET_CGEMM_SKINNY": "0"},                            # small products on the block kernels (cut along K)
    {"CNET_CGEMM_TILE": "0", "CNET_CGEMM_COLSPLIT": "0"},  # 128 x 128 blocks
    {"CNET_CGEMM_TILE": "3", "CNET_CGEMM_TAIL": "1"},      # 64 x 64 blocks, tail blocks cut along K whenever possible
    {"CNET_CGEMM_TILE": "4", "CNET_CGEMM_TAIL": "1"},      # the same blocks with two LDS stages
    {"CNET_CGEMM_SKINNY_W": "16"},                         # sixteen wavefronts per tile of the small-C kernel (1024 threads a workgroup)
])
def test_fused_layers_under_other_kernel_choices(gpu, overrides):
    """The tests of this file again in a process whose tuning overrides (read once per process) send the same shapes to
    other kernels: every epilogue and both partial-sum kernels apply the activation."""
    if os.environ.get("CNET_TEST_INNER"):
        pytest.skip("already the inner run")
    env = dict(os.environ, CNET_TEST_INNER="1", **overrides)
    r = subprocess.run([sys.executable, "-m", "pytest", os.path.abspath(__file__), "-x", "-q", "-m", "gpu"], env=env,
                       capture_output=True, text=True, timeout=280, cwd=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]


# B, n: small batches take the small-C kernel and one launch; 50 x 2048 (K cut into slices), 4096 x 784 and 1024 x 1024 (block
# kernels) two launches
TRANSFORM_GATE = [(64, 784), (16, 96), (1, 4), (100, 333), (256, 784), (50, 2048), (4096, 784), (1024, 1024)]


@pytest.mark.parametrize("B,n", TRANSFORM_GATE)
def test_transform_gate_and_activation_in_one_call(gpu, port, B, n):
    """cnet_cdft_hadamard_cgelu_fwd (FourierTrans -> Hadamard with a shared weight row -> CGelu, the first three layers of
    upstream's README net) against cnet_cdft_fwd followed by cnet_hadamard_cgelu_fwd: equal bits in all three results, in
    column windows of wider buffers as well; and against the CPU oracle layer by layer (upstream testFfft / testHadamard /
    testGelu, tests/gputests.h:91, 464, 517)."""
    xr, xi = seeded(port, 3 * B + n, (B, n)), seeded(port, 3 * B + n + 1, (B, n))
    vr, vi = seeded(port, n + 7, (1, n), 0.7), seeded(port, n + 8, (1, n), 0.7)
    x, v = ops.CMat.from_host(xr, xi), ops.CMat.from_host(vr, vi)
    y0, h0, a0 = (ops.CMat.empty(B, n) for _ in range(3))
    ops.dft_fwd(x, y0)
    ops.hadamard_gelu_fwd(y0, v, h0, a0, shared=True)
    W = n + 12   # wider buffers: the results land in a window that starts at column 8
    base = seeded(port, 5, (B, W))
    wide = [ops.CMat(ops.Plane.from_host(base), ops.Plane.from_host(base)) for _ in range(3)]
    y1, h1, a1 = (w.sub(8, n) for w in wide)
    ops.dft_hadamard_gelu_fwd(x, v, y1, h1, a1)
    mask = np.ones(W, bool); mask[8:8 + n] = False
    for w, want, what in zip(wide, (y0, h0, a0), ("transform", "gated", "activation")):
        for plane, ref in zip((w.re.owner.download(), w.im.owner.download()), want.host()):
            assert np.array_equal(plane[:, 8:8 + n], ref), (what, B, n)
            assert np.array_equal(plane[:, mask], base[:, mask]), (what, "outside the window")
    if B * n * n <= 1 << 27:
        yr, yi = port.dft_fwd(xr, xi)
        hr, hi = port.hadamard_fwd(yr, yi, vr[0], vi[0])
        assert rel_c(y0.host(), (yr, yi)) < TOL and rel_c(h0.host(), (hr, hi)) < TOL
        assert rel_c(a0.host(), port.gelu_fwd(hr, hi)) < TOL


# B, K, N: narrow heads on the small-C kernel (one launch), a head of 16 logits (the 128-bit row routine), a head that is too
# wide (N = 20) and one whose product is cut along K (K = 4096): two launches
HEADS = [(64, 784, 10), (1, 8, 1), (100, 96, 3), (4096, 784, 10), (64, 64, 16), (50, 300, 12), (64, 128, 20), (32, 4096, 10)]


@pytest.mark.parametrize("B,K,N", HEADS)
def test_linear_head_and_its_loss_in_one_call(gpu, port, B, K, N):
    """cnet_clinear_cross_entropy_fwd_bwd_sym against cnet_clinear_fwd followed by cnet_cross_entropy_fwd_bwd_sym: equal bits
    in the logits, S, loss, argmax, the normalised rows and the gradient, with and without the normalised planes and the dz*
    planes; and against the CPU oracle (upstream testLinear / testCE, tests/gputests.h:317, 266)."""
    from cnet_amd import capi
    xr, xi = seeded(port, B + K, (B, K)), seeded(port, B + K + 1, (B, K))
    wr, wi = seeded(port, N + 2, (N, K), K ** -0.5), seeded(port, N + 3, (N, K), K ** -0.5)
    labels_h = port.randint(B + N, (B,), N)
    x, w, labels = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi), ops.ints(labels_h)
    keep = [seeded(port, 40 + p, (B, N)) for p in range(4)]
    for with_out in (True, False):
        for mirror in (True, False):
            y0, y1 = ops.CMat.empty(B, N), ops.CMat.empty(B, N)
            n0, n1 = ops.CMat.empty(B, N, zero=True), ops.CMat.empty(B, N, zero=True)
            d0, d1 = ops.Grad.from_host(keep), ops.Grad.from_host(keep)
            r0 = [capi.empty(B), capi.empty(B), capi.empty(B, np.int32)]
            r1 = [capi.empty(B), capi.empty(B), capi.empty(B, np.int32)]
            ops.linear_fwd(x, w, y0)
            ops.cross_entropy_fwd_bwd_sym(y0, labels, r0[0], r0[1], r0[2], d0, out=n0 if with_out else None, mirror=mirror)
            ops.linear_cross_entropy_fwd_bwd_sym(x, w, y1, labels, r1[0], r1[1], r1[2], d1, out=n1 if with_out else None, mirror=mirror)
            what = (B, K, N, with_out, mirror)
            for a, b in zip(list(y0.host()) + list(n0.host()) + d0.host(), list(y1.host()) + list(n1.host()) + d1.host()):
                assert np.array_equal(a, b), what
            for a, b in zip(r0, r1):
                assert np.array_equal(a.download(), b.download()), what
            if not mirror:
                assert np.array_equal(d1.host()[2], keep[2]) and np.array_equal(d1.host()[3], keep[3]), (what, "dz* was written")
    if B * K * N <= 1 << 24:
        zr, zi = port.linear_fwd(xr, xi, wr, wi)
        _, _, S, loss, pred = port.crossent_fwd(zr, zi, labels_h)
        assert rel_c(y1.host(), (zr, zi)) < TOL / 5
        assert np.array_equal(r1[2].download(), pred) and np.allclose(r1[1].download(), loss, rtol=2e-5, atol=2e-6)
        want = port.crossent_bwd(zr, zi, labels_h)
        d = ops.Grad.empty(B, N)
        ops.linear_cross_entropy_fwd_bwd_sym(x, w, y1, labels, r1[0], r1[1], r1[2], d)
        h = d.host()
        # (the gradient at a label whose logit is small is large and as ill conditioned as 1 / |z_label|: the bar itself)
        assert rel_c(h[0:2], want[0:2]) < TOL and rel_c(h[2:4], want[2:4]) < TOL


# B, K (hidden width = columns of the gate), N (outputs of the Linear): up to 128 rows with small products take one launch;
# 129 and 200 rows, and 784 outputs (products beyond the small-C kernel) the separate launches
GATED_HEADS = [(64, 784, 10), (1, 4, 1), (3, 20, 2), (16, 96, 16), (100, 333, 12), (128, 784, 10), (127, 130, 5), (129, 784, 10),
               (200, 64, 7), (64, 784, 784), (60, 2052, 10)]


@pytest.mark.parametrize("B,K,N", GATED_HEADS)
def test_backward_pass_of_a_linear_and_the_gate_below_it_in_one_call(gpu, port, B, K, N):
    """cnet_clinear_hadamard_cgelu_bwd_sym against cnet_clinear_bwd_sym followed by cnet_hadamard_cgelu_bwd_sym (shared row):
    same bits in dx, dw, dh, du and dv, with each accumulate flag, with and without the dz* planes, with and without dh; and
    the gradients against the CPU path (Linear, CGelu and Hadamard backward of the oracle on the same conjugate pair)."""
    u = ops.CMat.from_host(seeded(port, K + 1, (B, K)), seeded(port, K + 2, (B, K)))
    v = ops.CMat.from_host(seeded(port, K + 3, (1, K)), seeded(port, K + 4, (1, K)))
    h, x = ops.CMat.empty(B, K), ops.CMat.empty(B, K)
    ops.hadamard_gelu_fwd(u, v, h, x, shared=True)
    w = ops.CMat.from_host(seeded(port, N + 5, (N, K)), seeded(port, N + 6, (N, K)))
    gr, gi = seeded(port, B + 7, (B, N)), seeded(port, B + 8, (B, N))
    g = ops.Grad.from_host([gr, gi, gr, -gi])
    bx, bw, bv = ([seeded(port, s + p, shape) for p in range(4)] for s, shape in ((20, (B, K)), (30, (N, K)), (40, (1, K))))
    cases = ((0, 0, 0, True, True), (1, 0, 1, True, True), (0, 1, 0, False, True), (1, 1, 1, True, False), (0, 0, 1, False, False))
    for acc_x, acc_w, acc_g, mirror, with_dh in cases:
        def planes():
            return (ops.Grad.from_host(bx), ops.Grad.from_host(bw), ops.Grad.from_host(bx) if with_dh else None, ops.Grad.from_host(bx),
                    ops.Grad.from_host(bv))
        dx0, dw0, dh0, du0, dv0 = planes()
        ops.linear_bwd_sym(g, x, w, dx0, dw0, accumulate_dx=acc_x, accumulate_dw=acc_w, mirror_dx=mirror, mirror_dw=mirror)
        ops.hadamard_gelu_bwd_sym(u, v, dx0, dh0, du0, dv0, shared=True, accumulate=acc_g, mirror=mirror)
        dx1, dw1, dh1, du1, dv1 = planes()
        ops.linear_hadamard_gelu_bwd_sym(g, x, w, dx1, dw1, u, v, dh1, du1, dv1, accumulate_dx=acc_x, accumulate_dw=acc_w,
                                         accumulate_gate=acc_g, mirror=mirror)
        for name, a, b in (("dx", dx0, dx1), ("dw", dw0, dw1), ("dh", dh0, dh1), ("du", du0, du1), ("dv", dv0, dv1)):
            if a is None:
                continue
            for pa, pb in zip(a.host(), b.host()):
                assert np.array_equal(pa, pb), (name, acc_x, acc_w, acc_g, mirror, with_dh)
    # the CPU path on the same pair
    (ur, ui), (vr, vi), (hr, hi), (xr, xi), (wr, wi) = u.host(), v.host(), h.host(), x.host(), w.host()
    dxo, dwo = port.linear_bwd(xr, xi, wr, wi, [gr, gi, gr, -gi])
    dho = port.gelu_bwd(hr, hi, dxo)
    duo, dvo = port.hadamard_bwd(ur, ui, np.ascontiguousarray(vr[0]), np.ascontiguousarray(vi[0]), dho)   # shared row: dv summed over the batch
    dx1, dw1, dh1, du1, dv1 = ops.Grad.empty(B, K), ops.Grad.empty(N, K), ops.Grad.empty(B, K), ops.Grad.empty(B, K), ops.Grad.empty(1, K)
    ops.linear_hadamard_gelu_bwd_sym(g, x, w, dx1, dw1, u, v, dh1, du1, dv1)
    for got, want in ((dx1, dxo), (dw1, dwo), (dh1, dho), (du1, duo), (dv1, [p[None, :] for p in dvo])):
        assert rel_c(got.host()[0:2], want[0:2]) < TOL / 5 and rel_c(got.host()[2:4], want[2:4]) < TOL / 5
