"""Error behaviour of the C ABI on the device: every entry point returns a status and leaves a message in
cnet_last_error(); nothing aborts the process (upstream's gpuErrchk prints and exits, gpu/allocator.h:37-57).
Also the graph recording rules: calls that allocate or wait are refused while recording and the recording can
be dropped cleanly; a recorded sequence replays with the same bits as the eager calls."""
import ctypes as C

import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, seeded  # noqa: F401

pytestmark = pytest.mark.gpu

INVALID, UNSUPPORTED = -2, -5


def _status(name, *args):
    return getattr(capi.load(), name)(*args)


def _msg():
    return capi.load().cnet_last_error().decode()


def test_invalid_arguments_are_reported_not_fatal(gpu, port):
    x = ops.CMat.from_host(seeded(port, 1, (4, 8)), seeded(port, 2, (4, 8)))
    y = ops.CMat.empty(4, 8)
    # leading dimension shorter than the row
    assert _status("cnet_cgelu_fwd", *x.p(), 4, *y.p(), 8, 4, 8) == INVALID and "cnet_cgelu_fwd" in _msg()
    # null operand
    assert _status("cnet_cgelu_fwd", None, x.im.ptr, 8, *y.p(), 8, 4, 8) == INVALID
    # negative shape, K = 0
    assert _status("cnet_cgemm", 0, 0, 0, -1, 8, 8, *x.p(), 8, *x.p(), 8, *y.p(), 8, 0) == INVALID
    assert _status("cnet_cgemm", 0, 0, 0, 4, 8, 0, *x.p(), 8, *x.p(), 8, *y.p(), 8, 0) == INVALID
    # empty problems are fine and touch nothing
    before = y.host()
    assert _status("cnet_cgemm", 0, 0, 0, 0, 8, 8, *x.p(), 8, *x.p(), 8, *y.p(), 8, 0) == 0
    assert _status("cnet_cgelu_fwd", *x.p(), 8, *y.p(), 8, 0, 8) == 0
    after = y.host()
    assert np.array_equal(before[0], after[0])
    # DFT length beyond the int exponent range of the reference, Adam with a negative step, unknown marker
    assert _status("cnet_cdft_plan", 50000) == INVALID
    assert _status("cnet_adam_update", x.re.ptr, x.im.ptr, y.re.ptr, y.im.ptr, y.re.ptr, y.im.ptr, 32, 0.1, 0.9, -1, 1) == INVALID
    assert _status("cnet_mark_compute", 8) == INVALID and _status("cnet_upload_wait_marker", -1) == INVALID
    # a second init on the same device is idempotent, on another device it is refused
    assert _status("cnet_init", 0) == 0
    assert _status("cnet_init", 3) == INVALID
    # the library still works
    ops.gelu_fwd(x, y)
    yr, yi = port.gelu_fwd(*x.host())
    assert np.allclose(y.host()[0], yr, atol=1e-6)


def test_graph_recording_rules_and_replay(gpu, port):
    B, K, N = 32, 64, 48
    xr, xi = seeded(port, 3, (B, K)), seeded(port, 4, (B, K))
    wr, wi = seeded(port, 5, (N, K), 0.2), seeded(port, 6, (N, K), 0.2)
    x, w = ops.CMat.from_host(xr, xi), ops.CMat.from_host(wr, wi)
    y, z = ops.CMat.empty(B, N), ops.CMat.empty(B, N)
    ops.linear_fwd(x, w, y)   # eager: also sizes whatever the library needs
    ops.gelu_fwd(y, z)
    eager = z.host()
    assert _status("cnet_graph_end", None) == INVALID  # nothing is being recorded
    # calls that wait or allocate are refused while recording, and the recording can be dropped
    capi.call("cnet_graph_begin")
    p = C.c_void_p()
    assert _status("cnet_alloc", 1024, C.byref(p)) == UNSUPPORTED and "cnet_graph_begin" in _msg()
    assert _status("cnet_sync") == UNSUPPORTED
    assert _status("cnet_cdft_plan", 96) == UNSUPPORTED  # a new transform length needs memory
    assert _status("cnet_graph_begin") == UNSUPPORTED
    capi.call("cnet_graph_end", None)
    capi.sync()
    # record forward + activation + clearing of a buffer, replay three times with eager work and syncs in between
    scratch = capi.to_device(np.ones(1000, np.float32))
    capi.call("cnet_graph_begin")
    ops.linear_fwd(x, w, y)
    ops.gelu_fwd(y, z)
    capi.call("cnet_memset_zero", scratch.ptr + 4, 4 * 500)
    exe = C.c_void_p()
    capi.call("cnet_graph_end", C.byref(exe))
    assert exe.value
    for k in range(3):
        y.re.owner.zero(); z.re.owner.zero(); z.im.owner.zero()
        scratch.upload(np.ones(1000, np.float32))
        capi.call("cnet_graph_launch", exe)
        got = z.host()
        assert np.array_equal(got[0], eager[0]) and np.array_equal(got[1], eager[1]), k
        h = scratch.download()
        assert h[0] == 1 and not h[1:501].any() and h[501] == 1
        ops.residual_fwd(y, y, z)  # unrelated eager work between replays
        capi.sync()
    capi.call("cnet_graph_destroy", exe)
    capi.call("cnet_graph_destroy", None)
