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


@pytest.mark.parametrize("overrides", [
    {"CNET_CGEMM_SKINNY": "0"},                            # small products on the block kernels (cut along K)
    {"CNET_CGEMM_TILE": "0", "CNET_CGEMM_COLSPLIT": "0"},  # 128 x 128 blocks (two accumulator sets, negated operand)
    {"CNET_CGEMM_TILE": "3", "CNET_CGEMM_TAIL": "1"},      # 64 x 64 blocks, tail blocks cut along K whenever possible
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
