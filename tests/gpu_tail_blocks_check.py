"""Run by tests/test_gpu_linear.py in a process of its own, with CNET_CGEMM_TAIL=1 (and a block shape) in the
environment: the library reads those switches once, when the first product is launched.  With the switch on, every
product whose blocks do not fill a whole number of rounds over the compute units cuts the blocks of the last round
along K; the results are compared with numpy in complex128."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from cnet_amd import capi, ops  # noqa: E402


def main():
    capi.init(0)
    rs = np.random.RandomState(7)
    worst = 0.0
    for (M, N, K) in ((1300, 840, 256), (4096, 784, 784), (2048, 1100, 128), (1028, 2052, 64)):
        A = (rs.randn(M, K) + 1j * rs.randn(M, K)).astype(np.complex64)
        Bm = (rs.randn(K, N) + 1j * rs.randn(K, N)).astype(np.complex64)
        want = A.astype(np.complex128) @ Bm.astype(np.complex128)
        for a_km in (0, 1):
            for b_km in (0, 1):
                a_h = A.T if a_km else A
                b_h = Bm if b_km else Bm.T
                a = ops.CMat.from_host(np.ascontiguousarray(a_h.real), np.ascontiguousarray(a_h.imag))
                b = ops.CMat.from_host(np.ascontiguousarray(b_h.real), np.ascontiguousarray(b_h.imag))
                cj = (a_km + b_km) % 2
                w = want if not cj else A.astype(np.complex128) @ Bm.astype(np.complex128).conj()
                base = rs.randn(M, N).astype(np.float32)
                c = ops.CMat.from_host(base.copy(), base.copy())
                ops.cgemm(a, b, c, M, N, K, a_km, b_km, cj, accumulate=1)
                cr, ci = c.host()
                err = np.linalg.norm((cr - base) + 1j * (ci - base) - w) / np.linalg.norm(w)
                worst = max(worst, err)
                if err > 2e-5:
                    print("FAIL", M, N, K, a_km, b_km, cj, err)
                    return 1
    # two problems in one launch (dz and dz* of a Linear backward)
    B, Kin, Nout = 1300, 840, 256
    g4 = [rs.randn(B, Nout).astype(np.float32) for _ in range(4)]
    wr, wi = rs.randn(Nout, Kin).astype(np.float32), rs.randn(Nout, Kin).astype(np.float32)
    g, w = ops.Grad.from_host(g4), ops.CMat.from_host(wr, wi)
    dx = ops.Grad.empty(B, Kin)
    ops.linear_bwd_input(g, w, dx)
    h = dx.host()
    W = wr.astype(np.float64) + 1j * wi
    want_dz = (g4[0].astype(np.float64) + 1j * g4[1]) @ W
    want_dzs = (g4[2].astype(np.float64) + 1j * g4[3]) @ W.conj()
    for got, want2 in ((h[0] + 1j * h[1], want_dz), (h[2] + 1j * h[3], want_dzs)):
        err = np.linalg.norm(got - want2) / np.linalg.norm(want2)
        worst = max(worst, err)
        if err > 2e-5:
            print("FAIL linear_bwd_input", err)
            return 1
    print("OK worst relative error %.2e" % worst)
    return 0


if __name__ == "__main__":
    sys.exit(main())
