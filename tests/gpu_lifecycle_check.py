"""Run by tests/test_gpu_abi_errors.py in a process of its own: cnet_init / work / cnet_shutdown, twice over.  After a
shutdown every entry point reports CNET_ERR_NOT_INITIALIZED instead of touching the device, and a second initialisation
rebuilds what the first one owned (streams, twiddle planes, workspace) and gives the same results."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from cnet_amd import capi, ops  # noqa: E402


def work():
    rs = np.random.RandomState(3)
    B, n = 24, 96
    xr, xi = rs.randn(B, n).astype(np.float32), rs.randn(B, n).astype(np.float32)
    x, y = ops.CMat.from_host(xr, xi), ops.CMat.empty(B, n)
    ops.dft_fwd(x, y)                                   # twiddle planes
    A = ops.CMat.from_host(rs.randn(8, 2048).astype(np.float32), rs.randn(8, 2048).astype(np.float32))
    Bm = ops.CMat.from_host(rs.randn(2048, 24).astype(np.float32), rs.randn(2048, 24).astype(np.float32))
    c = ops.CMat.empty(8, 24)
    ops.cgemm(A, Bm, c, 8, 24, 2048, 0, 1)              # cut along K: workspace
    out = [np.concatenate([p.ravel() for p in y.host()]), np.concatenate([p.ravel() for p in c.host()])]
    del x, y, A, Bm, c                                   # device arrays are freed while the library is still up
    return out


def main():
    lib = capi.load()
    if lib.cnet_sync() != -1 or "cnet_init" not in lib.cnet_last_error().decode():
        print("FAIL: an entry point did not report the missing cnet_init")
        return 1
    capi.init(0)
    first = work()
    capi.call("cnet_shutdown")
    if lib.cnet_sync() != -1:
        print("FAIL: cnet_sync did not report the missing initialisation after cnet_shutdown")
        return 1
    if lib.cnet_shutdown() != 0:
        print("FAIL: a second cnet_shutdown is not a no-op")
        return 1
    capi.init(0)
    second = work()
    for a, b in zip(first, second):
        if not np.array_equal(a, b):
            print("FAIL: results differ after re-initialisation")
            return 1
    capi.call("cnet_shutdown")
    print("OK")
    return 0


if __name__ == "__main__":
    sys.exit(main())
