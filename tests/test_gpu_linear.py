"""Complex Linear (forward and the four Wirtinger backward products) on the GPU against the CPU oracle.

Mirrors upstream testLinear / testLinearMaxGradient (tests/gputests.h:317, 756): same layer, CPU result as the
reference, but seeded inputs and a relative Frobenius bound (1e-4; observed ~1e-6) instead of a loose absolute one.
"""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu

SHAPES = [  # B, K, N
    (1, 4, 4), (3, 8, 5), (64, 784, 10), (37, 100, 19), (130, 68, 132), (256, 256, 256), (96, 1024, 64), (257, 33, 7),
]


@pytest.fixture(params=[3, 4], ids=["three_products", "four_products"])
def products(request, gpu):
    """Runs a test with the block kernels forming a complex product from four real ones (the default) and from three."""
    lib = capi.load()
    before = lib.cnet_cgemm_get_products()
    capi.call("cnet_cgemm_set_products", request.param)
    yield request.param
    capi.call("cnet_cgemm_set_products", before)


def _case(port, B, K, N, seed):
    xr, xi = seeded(port, seed, (B, K)), seeded(port, seed + 1, (B, K))
    wr, wi = seeded(port, seed + 2, (N, K), 1 / np.sqrt(K)), seeded(port, seed + 3, (N, K), 1 / np.sqrt(K))
    g4 = [seeded(port, seed + 4 + p, (B, N)) for p in range(4)]
    return xr, xi, wr, wi, g4


@pytest.mark.usefixtures("products")
@pytest.mark.parametrize("B,K,N", SHAPES)
def test_linear_forward_and_backward(gpu, port, B, K, N):
    xr, xi, wr, wi, g4 = _case(port, B, K, N, seed=B + K + N)
    yr, yi = port.linear_fwd(xr, xi, wr, wi)
    dx_o, dw_o = port.linear_bwd(xr, xi, wr, wi, g4)

    x, w, g = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi), ops.Grad.from_host(g4)
    y = ops.CMat.empty(B, N)
    ops.linear_fwd(x, w, y)
    assert rel_c(y.host(), (yr, yi)) < TOL / 5
    dx, dw = ops.Grad.empty(B, K), ops.Grad.empty(N, K)
    ops.linear_bwd_input(g, w, dx)
    ops.linear_bwd_weight(g, x, dw)
    hx, hw = dx.host(), dw.host()
    assert rel_c(hx[0:2], dx_o[0:2]) < TOL / 5 and rel_c(hx[2:4], dx_o[2:4]) < TOL / 5
    assert rel_c(hw[0:2], dw_o[0:2]) < TOL / 5 and rel_c(hw[2:4], dw_o[2:4]) < TOL / 5


def test_linear_accumulate_and_leading_dimensions(gpu, port):
    """Outputs land in a column window of a wider buffer (a consumer's concatenated input block) and add to what is there."""
    B, K, N = 48, 40, 24
    xr, xi, wr, wi, g4 = _case(port, B, K, N, seed=9)
    yr, yi = port.linear_fwd(xr, xi, wr, wi)
    dx_o, dw_o = port.linear_bwd(xr, xi, wr, wi, g4)
    base = seeded(port, 77, (B, 100))
    wide = ops.CMat(ops.Plane.from_host(base), ops.Plane.from_host(base))
    x, w, g = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi), ops.Grad.from_host(g4)
    ops.linear_fwd(x, w, wide.sub(12, N), accumulate=1)
    hr, hi = wide.re.owner.download(), wide.im.owner.download()
    assert rel_c((hr[:, 12:12 + N] - base[:, 12:12 + N], hi[:, 12:12 + N] - base[:, 12:12 + N]), (yr, yi)) < 1e-5
    mask = np.ones(100, bool); mask[12:12 + N] = False
    assert np.array_equal(hr[:, mask], base[:, mask]) and np.array_equal(hi[:, mask], base[:, mask])
    # x read from a window of a wider buffer, gradients accumulated twice
    xw = ops.CMat(ops.Plane.from_host(np.concatenate([base[:, :8], xr, base[:, :4]], 1)),
                  ops.Plane.from_host(np.concatenate([base[:, :8], xi, base[:, :4]], 1))).sub(8, K)
    dw = ops.Grad.empty(N, K, zero=True)
    ops.linear_bwd_weight(g, xw, dw, accumulate=1)
    ops.linear_bwd_weight(g, xw, dw, accumulate=1)
    h = dw.host()
    assert rel_c((h[2] / 2, h[3] / 2), dw_o[2:4]) < 1e-5
    dx = ops.Grad.empty(B, K, ld=K + 4, zero=True)
    ops.linear_bwd_input(g, w, dx, accumulate=1)
    assert rel_c(dx.host()[0:2], dx_o[0:2]) < 1e-5


@pytest.mark.usefixtures("products")
def test_cgemm_all_layouts(gpu, port):
    """C = op(A) op(B) for the four storage combinations, with and without conj(B), against numpy complex128."""
    M, N, K = 72, 40, 52
    A = seeded(port, 1, (M, K)) + 1j * seeded(port, 2, (M, K))
    Bm = seeded(port, 3, (K, N)) + 1j * seeded(port, 4, (K, N))
    for a_km in (0, 1):
        for b_km in (0, 1):
            for cj in (0, 1):
                a_h = A.T if a_km else A
                b_h = Bm if b_km else Bm.T
                a = ops.CMat.from_host(np.ascontiguousarray(a_h.real), np.ascontiguousarray(a_h.imag))
                b = ops.CMat.from_host(np.ascontiguousarray(b_h.real), np.ascontiguousarray(b_h.imag))
                c = ops.CMat.empty(M, N)
                ops.cgemm(a, b, c, M, N, K, a_km, b_km, cj)
                want = A @ (Bm.conj() if cj else Bm)
                cr, ci = c.host()
                err = np.linalg.norm(cr + 1j * ci - want) / np.linalg.norm(want)
                assert err < 1e-5, (a_km, b_km, cj, err)


def _check_all_layouts(port, M, N, K):
    """All four layouts, conj(B), accumulation into a window of a wider and taller buffer whose other elements must keep
    their bits, and run-to-run identical results; the expected product is numpy's in complex128."""
    A = seeded(port, 1, (M, K)) + 1j * seeded(port, 2, (M, K))
    Bm = seeded(port, 3, (K, N)) + 1j * seeded(port, 4, (K, N))
    base = seeded(port, 5, (M + 2, N + 9))
    for a_km in (0, 1):
        for b_km in (0, 1):
            a_h = A.T if a_km else A
            b_h = Bm if b_km else Bm.T
            a = ops.CMat.from_host(np.ascontiguousarray(a_h.real), np.ascontiguousarray(a_h.imag))
            b = ops.CMat.from_host(np.ascontiguousarray(b_h.real), np.ascontiguousarray(b_h.imag))
            cj = (a_km + b_km) % 2
            want = A @ (Bm.conj() if cj else Bm)
            c = ops.CMat.empty(M, N)
            ops.cgemm(a, b, c, M, N, K, a_km, b_km, cj)
            first = c.host()
            err = np.linalg.norm(first[0] + 1j * first[1] - want) / np.linalg.norm(want)
            assert err < 1e-5, (a_km, b_km, err)
            ops.cgemm(a, b, c, M, N, K, a_km, b_km, cj)
            again = c.host()
            assert np.array_equal(first[0], again[0]) and np.array_equal(first[1], again[1])
            wide = ops.CMat(ops.Plane.from_host(base), ops.Plane.from_host(base))
            ops.cgemm(a, b, wide.sub(4, N), M, N, K, a_km, b_km, cj, accumulate=1)
            hr, hi = wide.re.owner.download(), wide.im.owner.download()
            got = (hr[:M, 4:4 + N] - base[:M, 4:4 + N]) + 1j * (hi[:M, 4:4 + N] - base[:M, 4:4 + N])
            assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5
            hr[:M, 4:4 + N] = hi[:M, 4:4 + N] = base[:M, 4:4 + N]  # what is left is the frame around the window
            assert np.array_equal(hr, base) and np.array_equal(hi, base)


@pytest.mark.usefixtures("products")
@pytest.mark.parametrize("M,N,K", [(8, 24, 1000), (64, 64, 4096), (40, 100, 333), (64, 784, 784), (3, 5, 2049), (784, 784, 4096),
                                   (64, 64, 100000), (520, 516, 2048)])
def test_cgemm_short_grid_long_reduction(gpu, port, M, N, K):
    """Few blocks of C against a long K.  Up to K = 1024 each 16 x 16 tile of C has a workgroup of its own whose wavefronts
    share K; beyond, the launch of the block kernel is cut along K and the partial blocks are added in a fixed order (also
    when the blocks of C are fewer than two per compute unit, 784 x 784: 169 blocks, and the cost model finds the cut
    cheaper than idle units)."""
    _check_all_layouts(port, M, N, K)


@pytest.mark.usefixtures("products")
@pytest.mark.parametrize("M,N,K", [(4, 4, 16), (132, 200, 64), (260, 68, 48), (700, 388, 32), (1028, 516, 80), (68, 1300, 160),
                                   (4100, 1028, 16), (61, 67, 64), (4096, 784, 256), (1028, 516, 1000), (520, 772, 4092)])
def test_cgemm_blocks_on_the_edge_of_c(gpu, port, M, N, K):
    """K a multiple of 16 with M and N that are not multiples of any block shape: blocks that hang over the edge of C
    read the last valid rows again and must store nothing outside C.  The last shape (784 = 12 x 64 + 16 columns) is one
    the library computes as two products, columns 0..767 by the block kernel and the 16 left over by the small-C kernel;
    the two after it have a K that is not a whole number of 16-long chunks: the whole chunks go to the fast kernel and the
    last 8 / 12 values of k are added by a second launch."""
    _check_all_layouts(port, M, N, K)


def test_cgemm_batched_short_grid(gpu, port):
    """Strided batch of small products with a long K: the batch index and the K split share one grid dimension."""
    nb, M, N, K = 3, 16, 32, 640
    A = seeded(port, 11, (nb, M, K)) + 1j * seeded(port, 12, (nb, M, K))
    Bm = seeded(port, 13, (K, N)) + 1j * seeded(port, 14, (K, N))
    a = ops.CMat.from_host(np.ascontiguousarray(A.real).reshape(nb * M, K), np.ascontiguousarray(A.imag).reshape(nb * M, K))
    b = ops.CMat.from_host(np.ascontiguousarray(Bm.real), np.ascontiguousarray(Bm.imag))
    c = ops.CMat.empty(nb * M, N)
    ops.cgemm_batched(a, M * K, b, 0, c, M * N, M, N, K, nb, a_kmajor=0, b_kmajor=1, conj_a=1)
    cr, ci = c.host()
    want = np.conj(A) @ Bm
    got = (cr + 1j * ci).reshape(nb, M, N)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5


def test_linear_headline_shape_rows_against_oracle(gpu, port):
    """B=4096, 1024->1024 (the benchmark shape).  The oracle computes a 24-row subsample; dW/dW* are compared on a
    batch equal to that subsample, and the full-size run is checked through linearity in the batch:
    dW(all rows) = dW(first half) + dW(second half)."""
    B, K, N, sub = 4096, 1024, 1024, 24
    xr, xi, wr, wi, g4 = _case(port, B, K, N, seed=2024)
    x, w, g = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi), ops.Grad.from_host(g4)
    y, dx, dw = ops.CMat.empty(B, N), ops.Grad.empty(B, K), ops.Grad.empty(N, K)
    ops.linear_fwd(x, w, y)
    ops.linear_bwd_input(g, w, dx)
    ops.linear_bwd_weight(g, x, dw)
    rows = np.linspace(0, B - 1, sub).astype(int)
    sx = (np.ascontiguousarray(xr[rows]), np.ascontiguousarray(xi[rows]))
    sg = [np.ascontiguousarray(p[rows]) for p in g4]
    yr, yi = port.linear_fwd(sx[0], sx[1], wr, wi)
    dx_o, dw_o = port.linear_bwd(sx[0], sx[1], wr, wi, sg)
    hy, hdx = y.host(), dx.host()
    assert rel_c((hy[0][rows], hy[1][rows]), (yr, yi)) < TOL / 5
    assert rel_c((hdx[0][rows], hdx[1][rows]), dx_o[0:2]) < TOL / 5
    assert rel_c((hdx[2][rows], hdx[3][rows]), dx_o[2:4]) < TOL / 5
    # weight gradients on the subsample batch
    dws = ops.Grad.empty(N, K)
    ops.linear_bwd_weight(ops.Grad.from_host(sg), ops.CMat.from_host(*sx), dws)
    h = dws.host()
    assert rel_c(h[0:2], dw_o[0:2]) < TOL / 5 and rel_c(h[2:4], dw_o[2:4]) < TOL / 5
    # full batch: additivity over a split of the batch
    half = B // 2
    acc = ops.Grad.empty(N, K)
    for k, sl in enumerate((slice(0, half), slice(half, B))):
        gs = ops.Grad.from_host([np.ascontiguousarray(p[sl]) for p in g4])
        xs = ops.CMat.from_host(np.ascontiguousarray(xr[sl]), np.ascontiguousarray(xi[sl]))
        ops.linear_bwd_weight(gs, xs, acc, accumulate=k)
    full, parts = dw.host(), acc.host()
    assert rel_c(full[0:2], parts[0:2]) < 1e-5 and rel_c(full[2:4], parts[2:4]) < 1e-5


@pytest.mark.usefixtures("products")
@pytest.mark.parametrize("M,N,K,nb", [(8192, 1024, 64, 1), (192, 256, 48, 2), (4096, 512, 32, 1), (1024, 2048, 32, 1),
                                      (40, 52, 200, 2), (64, 10, 784, 1)])
def test_cgemm_conjugate_combinations(gpu, port, M, N, K, nb):
    """conj(A) and conj(B) in all four combinations, on shapes that take each block shape of the fast path: the signs are
    applied when the block is stored (one- and two-tile wavefronts) or by the choice of the negated operand (four
    tiles), and conj(A) conj(B) negates the imaginary plane on its way out.  The last two shapes have a small C and go
    to the kernel with one 16 x 16 tile per workgroup, which scales the imaginary operands by the signs."""
    A = seeded(port, 21, (nb, M, K)) + 1j * seeded(port, 22, (nb, M, K))
    Bm = seeded(port, 23, (K, N)) + 1j * seeded(port, 24, (K, N))
    a = ops.CMat.from_host(np.ascontiguousarray(A.real).reshape(nb * M, K), np.ascontiguousarray(A.imag).reshape(nb * M, K))
    b = ops.CMat.from_host(np.ascontiguousarray(Bm.real), np.ascontiguousarray(Bm.imag))
    for conj_a in (0, 1):
        for conj_b in (0, 1):
            c = ops.CMat.empty(nb * M, N)
            ops.cgemm_batched(a, M * K, b, 0, c, M * N, M, N, K, nb, a_kmajor=0, b_kmajor=1, conj_a=conj_a, conj_b=conj_b)
            cr, ci = c.host()
            want = (np.conj(A) if conj_a else A) @ (np.conj(Bm) if conj_b else Bm)
            got = (cr + 1j * ci).reshape(nb, M, N)
            assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5, (conj_a, conj_b)


@pytest.mark.usefixtures("products")
def test_cgemm_random_shapes(gpu, port):
    """About a hundred seeded random problems across the paths of the GEMM: aligned and odd shapes, K with and without a whole
    number of chunks, every layout, conj(B), accumulation, leading dimensions wider than the matrix, against numpy in
    complex128."""
    rs = np.random.RandomState(20240)
    for case in range(110):
        M = int(rs.choice([1, 3, 4, 7, 16, 60, 64, 68, 100, 128, 132, 200, 257, 384, 520, 1000, 2048, 4100]))
        N = int(rs.choice([1, 2, 4, 10, 16, 36, 64, 72, 128, 196, 260, 512, 784, 1040, 1300]))
        K = int(rs.choice([1, 2, 5, 16, 32, 48, 33, 64, 100, 128, 160, 784, 1000, 1024, 2044, 2048, 4096]))
        if M * N * K > 3e9:
            continue  # the larger ones are there for the paths that only many blocks take (columns split off, K cuts)
        a_km, b_km, cj, acc = int(rs.randint(2)), int(rs.randint(2)), int(rs.randint(2)), int(rs.randint(2))
        pad_a, pad_b, pad_c = (int(rs.choice([0, 4, 8, 3])) for _ in range(3))
        A = rs.randn(M, K) + 1j * rs.randn(M, K)
        Bm = rs.randn(K, N) + 1j * rs.randn(K, N)
        a_h = A.T if a_km else A
        b_h = Bm if b_km else Bm.T
        def wide(h, pad):  # the matrix sits in the first columns of a wider buffer
            buf = np.zeros((h.shape[0], h.shape[1] + pad), np.complex64)
            buf[:, :h.shape[1]] = h
            full = ops.CMat.from_host(np.ascontiguousarray(buf.real), np.ascontiguousarray(buf.imag))
            return full.sub(0, h.shape[1])
        a, b = wide(a_h, pad_a), wide(b_h, pad_b)
        c0 = (rs.randn(M, N + pad_c) + 1j * rs.randn(M, N + pad_c)).astype(np.complex64)
        cfull = ops.CMat.from_host(np.ascontiguousarray(c0.real), np.ascontiguousarray(c0.imag))
        ops.cgemm(a, b, cfull.sub(0, N), M, N, K, a_km, b_km, cj, accumulate=acc)
        cr, ci = cfull.re.owner.download(), cfull.im.owner.download()
        got = cr + 1j * ci
        a32, b32 = A.astype(np.complex64).astype(np.complex128), Bm.astype(np.complex64).astype(np.complex128)
        want = a32 @ (b32.conj() if cj else b32) + (c0[:, :N] if acc else 0)
        err = np.linalg.norm(got[:, :N] - want) / max(np.linalg.norm(want), 1e-30)
        assert err < 2e-5, (case, M, N, K, a_km, b_km, cj, acc, pad_a, pad_b, pad_c, err)
        assert np.array_equal(got[:, N:], c0[:, N:]), (case, "columns beside C were touched")


@pytest.mark.usefixtures("products")
@pytest.mark.parametrize("M,N,K,a_km,b_km,off_a,off_b", [(640, 512, 1000, 0, 1, 1, 0), (640, 512, 1024, 0, 0, 3, 2), (512, 768, 1000, 1, 1, 0, 1),
                                                        (1024, 520, 2040, 0, 1, 2, 3), (516, 600, 1024, 1, 0, 1, 1), (1001, 1001, 1001, 1, 1, 0, 0),
                                                        (1001, 1001, 1008, 0, 1, 0, 0), (2050, 514, 1024, 1, 0, 0, 2)])
def test_cgemm_large_products_of_misaligned_operands(gpu, port, M, N, K, a_km, b_km, off_a, off_b):
    """Operands whose planes start one to three floats off a 16-byte boundary (column windows of wider buffers, leading
    dimensions that are no multiple of four) in products large enough for the pass that first copies them into aligned
    planes, K with and without a whole number of chunks, every layout, also with M or N that end inside a group of four
    floats (1001, 2050, 514: such a run is padded, or taken as it is where its leading dimension covers the group): against
    numpy in complex128, with and without
    accumulation and conj(B); what lies beside C stays untouched, and CNET_CGEMM_PACK=0 (the register-staged kernel on the
    operands as they are) is checked by the random shapes above at smaller sizes."""
    rs = np.random.RandomState(M + N + K)
    A = (rs.randn(M, K) + 1j * rs.randn(M, K)).astype(np.complex64)
    Bm = (rs.randn(K, N) + 1j * rs.randn(K, N)).astype(np.complex64)
    def window(h, off):   # the matrix sits `off` columns into a buffer 5 columns wider (an odd leading dimension)
        buf = np.zeros((h.shape[0], h.shape[1] + 5), np.complex64)
        buf[:, off:off + h.shape[1]] = h
        return ops.CMat.from_host(np.ascontiguousarray(buf.real), np.ascontiguousarray(buf.imag)).sub(off, h.shape[1])
    a, b = window(A.T if a_km else A, off_a), window(Bm if b_km else Bm.T, off_b)
    for cj, acc in ((0, 0), (1, 1)):
        c0 = (rs.randn(M, N + 4) + 1j * rs.randn(M, N + 4)).astype(np.complex64)
        cfull = ops.CMat.from_host(np.ascontiguousarray(c0.real), np.ascontiguousarray(c0.imag))
        ops.cgemm(a, b, cfull.sub(0, N), M, N, K, a_km, b_km, cj, accumulate=acc)
        got = cfull.re.owner.download() + 1j * cfull.im.owner.download()
        want = A.astype(np.complex128) @ (Bm.conj() if cj else Bm).astype(np.complex128) + (c0[:, :N] if acc else 0)
        assert np.linalg.norm(got[:, :N] - want) / np.linalg.norm(want) < 2e-5, (cj, acc)
        assert np.array_equal(got[:, N:], c0[:, N:])


def test_gradient_pairs_of_a_linear_with_misaligned_operands(gpu, port):
    """Both halves of the input gradient and of the weight gradient (two problems per launch that share one operand) with
    every operand a misaligned column window: against the same calls on aligned copies of the operands."""
    rs = np.random.RandomState(5)
    B, K, N = 1024, 520, 512
    def both(h, off):
        buf = np.zeros((h.shape[0], h.shape[1] + 5), np.float32)
        buf[:, off:off + h.shape[1]] = h
        return buf
    planes = {name: [rs.randn(*shape).astype(np.float32) for _ in range(count)]
              for name, shape, count in (("x", (B, K), 2), ("w", (N, K), 2), ("g", (B, N), 4))}
    def run(off):
        if off is None:
            x, w = ops.CMat.from_host(*planes["x"]), ops.CMat.from_host(*planes["w"])
            g = ops.Grad.from_host(planes["g"])
        else:
            x = ops.CMat.from_host(both(planes["x"][0], off), both(planes["x"][1], off)).sub(off, K)
            w = ops.CMat.from_host(both(planes["w"][0], off), both(planes["w"][1], off)).sub(off, K)
            g = ops.Grad.from_host([both(p, off) for p in planes["g"]]).sub(off, N)
        dx, dw = ops.Grad.empty(B, K), ops.Grad.empty(N, K)
        ops.linear_bwd_input(g, w, dx)
        ops.linear_bwd_weight(g, x, dw)
        return dx.host(), dw.host()
    (dx0, dw0), (dx1, dw1) = run(None), run(3)
    for p in range(0, 4, 2):
        assert rel_c(dx1[p:p + 2], dx0[p:p + 2]) < 2e-6 and rel_c(dw1[p:p + 2], dw0[p:p + 2]) < 2e-6


@pytest.mark.parametrize("tile", ["0", "1", "2", "3", "4", ""])
def test_cgemm_tail_blocks_cut_along_k(gpu, tile):
    """Products whose blocks do not fill a whole number of rounds over the compute units, with the cut of the last round's
    blocks along K switched on for every such launch and each block shape in turn (4: the 64 x 64 block with two LDS stages; and
    the library's own choice)."""
    import os
    import subprocess
    import sys
    env = dict(os.environ, CNET_CGEMM_TAIL="1")
    if tile:
        env["CNET_CGEMM_TILE"] = tile
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpu_tail_blocks_check.py")
    r = subprocess.run([sys.executable, script], env=env, capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "OK" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_three_real_products_per_complex_product(gpu):
    """cnet_cgemm_set_products: the same products with three and with four real products per complex one against complex128,
    on rows of the headline shape and of a long reduction.  Three products stay normwise as accurate (the bound below is
    what they are allowed over four; both are two orders below the parity bar), a product of real operands keeps an
    imaginary plane of exact zeros, and any other count is refused."""
    lib = capi.load()
    before = lib.cnet_cgemm_get_products()
    rs = np.random.RandomState(7)
    try:
        for B, K, N in [(4096, 1024, 1024), (1024, 4096, 2048)]:
            X = (rs.randn(B, K) + 1j * rs.randn(B, K)).astype(np.complex64)
            W = ((rs.randn(N, K) + 1j * rs.randn(N, K)) / np.sqrt(K)).astype(np.complex64)
            x = ops.CMat.from_host(np.ascontiguousarray(X.real), np.ascontiguousarray(X.imag))
            w = ops.CMat.from_host(np.ascontiguousarray(W.real), np.ascontiguousarray(W.imag))
            rows = rs.choice(B, 48, replace=False)
            want = X[rows].astype(np.complex128) @ W.astype(np.complex128).T
            err = {}
            for n in (4, 3):
                capi.call("cnet_cgemm_set_products", n)
                assert lib.cnet_cgemm_get_products() == n
                y = ops.CMat.empty(B, N)
                ops.linear_fwd(x, w, y)
                yr, yi = y.host()
                got = (yr + 1j * yi)[rows]
                err[n] = np.linalg.norm(got - want) / np.linalg.norm(want)
                # each plane on its own as well: neither is traded for the other
                err[n, "re"] = np.linalg.norm(got.real - want.real) / np.linalg.norm(want.real)
                err[n, "im"] = np.linalg.norm(got.imag - want.imag) / np.linalg.norm(want.imag)
            print("B, K, N = %s: relative error against complex128, four products %.2e (re %.2e, im %.2e), three %.2e (re %.2e, im %.2e)"
                  % ((B, K, N), err[4], err[4, "re"], err[4, "im"], err[3], err[3, "re"], err[3, "im"]))
            assert err[4] < 5e-6 and err[3] < 5e-6
            assert err[3] < 3 * err[4] and err[3, "im"] < 4 * err[4, "im"]
        # real operands: T and P are the same sums, Q is zero
        capi.call("cnet_cgemm_set_products", 3)
        B, K, N = 512, 256, 384
        xr, wr = rs.randn(B, K).astype(np.float32), rs.randn(N, K).astype(np.float32)
        x = ops.CMat.from_host(xr, np.zeros_like(xr))
        w = ops.CMat.from_host(wr, np.zeros_like(wr))
        y = ops.CMat.empty(B, N)
        ops.linear_fwd(x, w, y)
        yr, yi = y.host()
        assert not yi.any()
        assert np.linalg.norm(yr - xr.astype(np.float64) @ wr.astype(np.float64).T) / np.linalg.norm(yr) < 1e-6
        for bad in (0, 2, 5, -3):
            assert lib.cnet_cgemm_set_products(bad) == -2  # CNET_ERR_INVALID_ARGUMENT
        assert lib.cnet_cgemm_get_products() == 3
    finally:
        capi.call("cnet_cgemm_set_products", before)
