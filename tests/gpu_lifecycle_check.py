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
    # a shutdown with a recording left alive and another one still open: the open one is dropped, the live one destroyed
    # with the library's buffers, and the next initialisation starts clean
    import ctypes as C
    x = ops.CMat.from_host(np.ones((4, 8), np.float32), np.ones((4, 8), np.float32))
    y = ops.CMat.empty(4, 8)
    ops.gelu_fwd(x, y)
    capi.call("cnet_graph_begin")
    ops.gelu_fwd(x, y)
    exe = C.c_void_p()
    capi.call("cnet_graph_end", C.byref(exe))
    capi.call("cnet_graph_launch", exe)
    capi.call("cnet_graph_begin")
    ops.gelu_fwd(x, y)
    if lib.cnet_shutdown() != 0:
        print("FAIL: cnet_shutdown with a live and an open recording: " + lib.cnet_last_error().decode())
        return 1
    capi.init(0)
    del x, y   # the device allocations outlive the library's own state
    if lib.cnet_graph_launch(exe) != -2:
        print("FAIL: a recording from before the shutdown was accepted")
        return 1
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
