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
    # the entry points for conjugate gradient pairs check their operands like the two-product ones
    g = ops.Grad.empty(4, 8)
    w = ops.CMat.from_host(seeded(port, 3, (8, 8)), seeded(port, 4, (8, 8)))
    dx = ops.Grad.empty(4, 8)
    assert _status("cnet_clinear_bwd_input_sym", g.p()[0], None, 8, *w.p(), 8, *dx.p(), 8, 4, 8, 8, 0) == INVALID
    assert _status("cnet_clinear_bwd_input_sym", *g.p()[:2], 4, *w.p(), 8, *dx.p(), 8, 4, 8, 8, 0) == INVALID      # ldg < N
    assert _status("cnet_clinear_bwd_weight_sym", *g.p()[:2], 8, *x.p(), 8, dx.p()[0], dx.p()[1], dx.p()[2], None, 8, 4, 8, 8, 0) == INVALID
    dw = ops.Grad.empty(8, 8)
    assert _status("cnet_clinear_bwd_sym", *g.p()[:2], 8, *x.p(), 8, *w.p(), 8, *dx.p(), 8, 0, dw.p()[0], dw.p()[1], None, dw.p()[3], 8, 0,
                   4, 8, 8) == INVALID                                                                                # half a pair of dz* planes
    assert _status("cnet_clinear_bwd_sym", *g.p()[:2], 8, *x.p(), 4, *w.p(), 8, *dx.p(), 8, 0, *dw.p(), 8, 0, 4, 8, 8) == INVALID   # ldx < K
    assert _status("cnet_clinear_bwd_sym", *g.p()[:2], 8, *x.p(), 8, *w.p(), 8, *dx.p(), 8, 0, *dw.p(), 8, 0, 0, 8, 8) == INVALID   # no rows
    assert _status("cnet_cdft_bwd_sym", *g.p()[:2], 8, *dx.p(), 4, 4, 8, 0) == INVALID                               # lddx < n
    assert _status("cnet_ctriang_dft_bwd_sym", *g.p()[:2], 8, *dx.p(), 8, 4, 50000, 0) == INVALID
    assert _status("cnet_cdft_bwd_sym", *g.p()[:2], 8, *dx.p(), 8, 0, 8, 0) == 0                                     # no rows: nothing to do
    # the fused pairs of layers check theirs too
    h = ops.CMat.empty(4, 8)
    assert _status("cnet_hadamard_cgelu_fwd", *x.p(), 8, *x.p(), 8, h.re.ptr, None, 8, *y.p(), 8, 4, 8) == INVALID        # a plane of h missing
    assert _status("cnet_hadamard_cgelu_fwd", *x.p(), 8, *x.p(), 8, *h.p(), 4, *y.p(), 8, 4, 8) == INVALID                # ldh < cols
    assert _status("cnet_hadamard_cgelu_fwd", *x.p(), 8, *x.p(), 8, *h.p(), 8, *y.p(), 8, 0, 8) == 0
    none4 = (None,) * 4
    assert _status("cnet_hadamard_cgelu_bwd_sym", *x.p(), 8, *x.p(), 8, *g.p()[:2], 8, *none4, 0, *dx.p(), 8, *dx.p(), 8, 4, 8, 0) == 0   # dh not wanted
    assert _status("cnet_hadamard_cgelu_bwd_sym", *x.p(), 8, *x.p(), 8, *g.p()[:2], 8, g.p()[0], None, None, None, 8, *dx.p(), 8, *dx.p(), 8,
                   4, 8, 0) == INVALID                                                                                    # half a dh
    assert _status("cnet_hadamard_cgelu_bwd_sym", *x.p(), 8, *x.p(), 8, *g.p()[:2], 8, *g.p(), 4, *dx.p(), 8, *dx.p(), 8, 4, 8, 0) == INVALID  # lddh < cols
    assert _status("cnet_residual_cgelu_bwd_sym", *g.p()[:2], 8, g.p()[0], None, 8, *x.p(), 8, *dx.p(), 8, *none4, 0, *dx.p(), 8, 4, 8) == INVALID  # half a g2
    assert _status("cnet_residual_cgelu_bwd_sym", *g.p()[:2], 8, None, None, 0, *x.p(), 8, *dx.p(), 8, None, dx.p()[1], None, None, 8,
                   *dx.p(), 8, 4, 8) == INVALID                                                                           # half a dv
    assert _status("cnet_residual_cgelu_bwd_sym", *g.p()[:2], 8, None, None, 0, *x.p(), 8, *dx.p(), 8, *none4, 0, *none4, 8, 4, 8) == INVALID  # no dh
    assert _status("cnet_residual_cgelu_bwd_sym", *g.p()[:2], 8, None, None, 0, *x.p(), 4, *dx.p(), 8, *none4, 0, *dx.p(), 8, 4, 8) == INVALID  # ldh < cols
    assert _status("cnet_clinear_cgelu_fwd", *x.p(), 8, *w.p(), 8, *h.p(), y.re.ptr, None, 8, 4, 8, 8, 0) == INVALID      # a plane of y missing
    assert _status("cnet_clinear_cgelu_fwd", *x.p(), 8, *w.p(), 8, *h.p(), *y.p(), 4, 4, 8, 8, 0) == INVALID              # ldy < N
    assert _status("cnet_clinear_cgelu_fwd", *x.p(), 8, *w.p(), 8, *h.p(), *y.p(), 8, 0, 8, 8, 0) == 0
    # the calls that carry a layer and what follows it in one launch at small batches hand a bad argument to the separate calls,
    # which name it
    v1 = ops.CMat.from_host(seeded(port, 5, (1, 8)), seeded(port, 6, (1, 8)))
    a8 = ops.CMat.empty(4, 8)
    du, dv, dh = ops.Grad.empty(4, 8), ops.Grad.empty(1, 8), ops.Grad.empty(4, 8)

    def gated(g_im=g.p()[1], ldx=8, dw_dzs_im=dw.p()[3], u_im=x.im.ptr, lddu=8, dh4=dh.p(), B=4):
        return _status("cnet_clinear_hadamard_cgelu_bwd_sym", g.p()[0], g_im, 8, *a8.p(), ldx, *w.p(), 8, *dx.p(), 8, 0, *dw.p()[:3], dw_dzs_im,
                       8, 0, x.re.ptr, u_im, 8, *v1.p(), *dh4, 8, *du.p(), lddu, *dv.p(), 0, B, 8, 8)
    assert gated() == 0 and gated(dh4=none4) == 0
    assert gated(g_im=None) == INVALID and gated(ldx=4) == INVALID and gated(dw_dzs_im=None) == INVALID
    assert gated(u_im=None) == INVALID and gated(lddu=4) == INVALID and gated(dh4=(dh.p()[0], None, None, None)) == INVALID
    assert gated(B=0) == INVALID   # as cnet_clinear_bwd_sym: no rows
    assert _status("cnet_cdft_plan", 8) == 0
    assert _status("cnet_cdft_hadamard_cgelu_fwd", *x.p(), 8, *v1.p(), *y.p(), *h.p(), *a8.p(), 8, 4, 8) == 0
    assert _status("cnet_cdft_hadamard_cgelu_fwd", *x.p(), 8, v1.re.ptr, None, *y.p(), *h.p(), *a8.p(), 8, 4, 8) == INVALID   # half a gate
    assert _status("cnet_cdft_hadamard_cgelu_fwd", *x.p(), 8, *v1.p(), *y.p(), *h.p(), *a8.p(), 4, 4, 8) == INVALID           # ld < n
    lab = ops.ints(np.zeros(4, np.int32))
    s4, l4, am4 = capi.empty(4), capi.empty(4), capi.empty(4, np.int32)

    def head(w_im=w.im.ptr, ldy=8, labels=lab.ptr, dz_im=dx.p()[1]):
        return _status("cnet_clinear_cross_entropy_fwd_bwd_sym", *x.p(), 8, w.re.ptr, w_im, 8, *y.p(), ldy, labels, None, None, 0, s4.ptr,
                       l4.ptr, am4.ptr, dx.p()[0], dz_im, None, None, 8, 4, 8, 8)
    assert head() == 0
    assert head(w_im=None) == INVALID and head(ldy=4) == INVALID and head(labels=None) == INVALID and head(dz_im=None) == INVALID
    # DFT length beyond the int exponent range of the reference, Adam with a negative step, unknown marker
    assert _status("cnet_cdft_plan", 50000) == INVALID
    assert _status("cnet_adam_update", x.re.ptr, x.im.ptr, y.re.ptr, y.im.ptr, y.re.ptr, y.im.ptr, 32, 0.1, 0.9, -1, 1) == INVALID
    assert _status("cnet_mark_compute", 8) == INVALID and _status("cnet_upload_wait_marker", -1) == INVALID
    assert _status("cnet_mark_upload", 8) == INVALID and _status("cnet_compute_wait_upload_marker", -1) == INVALID
    assert _status("cnet_mark_upload", 3) == 0 and _status("cnet_compute_wait_upload_marker", 3) == 0
    assert _status("cnet_compute_wait_upload_marker", 5) == 0   # never set: holds nothing back
    # copy tickets: one per stream, waited for one by one; a ticket that was never issued is refused
    t0, t1 = C.c_int64(-1), C.c_int64(-1)
    assert _status("cnet_copy_ticket", 0, C.byref(t0)) == 0 and _status("cnet_copy_ticket", 1, C.byref(t1)) == 0
    assert t0.value >= 0 and t1.value >= 0 and t0.value % 2 == 0 and t1.value % 2 == 1
    assert _status("cnet_copy_wait", t1.value) == 0 and _status("cnet_copy_wait", t0.value) == 0
    assert _status("cnet_copy_wait", t1.value + 2) == INVALID and _status("cnet_copy_wait", -1) == INVALID
    assert _status("cnet_copy_ticket", 0, None) == INVALID
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
    assert _status("cnet_cdft_plan", 3331) == UNSUPPORTED  # a new transform length needs memory (no other test plans this one)
    assert _status("cnet_graph_begin") == UNSUPPORTED
    assert _status("cnet_mark_compute", 0) == UNSUPPORTED and _status("cnet_compute_wait_upload") == UNSUPPORTED
    assert _status("cnet_mark_upload", 0) == UNSUPPORTED and _status("cnet_compute_wait_upload_marker", 0) == UNSUPPORTED
    t = C.c_int64(-1)
    assert _status("cnet_copy_ticket", 0, C.byref(t)) == UNSUPPORTED
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
    # a recording cannot be destroyed while another one is being recorded (the call waits for the stream)
    capi.call("cnet_graph_begin")
    assert _status("cnet_graph_destroy", exe) == UNSUPPORTED and "cnet_graph_begin" in _msg()
    capi.call("cnet_graph_end", None)
    capi.call("cnet_graph_launch", exe)   # ... and is still whole
    capi.sync()
    capi.call("cnet_graph_destroy", exe)
    capi.call("cnet_graph_destroy", None)
    # a handle that is not a live recording is refused, not handed to the runtime
    assert _status("cnet_graph_launch", exe) == INVALID and _status("cnet_graph_destroy", exe) == INVALID


def test_sgd_update_of_more_tensors_than_one_launch_takes_steps_each_once(gpu, port):
    """Ten tensors, one of them empty, gradients kept (zero_grad = 0): every tensor is stepped exactly once (a launch takes
    eight table entries; the empty one must not shift the next launch's window)."""
    sizes = [16, 12, 0, 8, 5, 64, 7, 9, 33, 4]
    zs, ds, want = [], [], []
    for k, n in enumerate(sizes):
        m = max(n, 1)
        zr, zi, dr, di = [seeded(port, 100 + 4 * k + j, (1, m)) for j in range(4)]
        zs.append(ops.CMat.from_host(zr, zi)); ds.append((ops.Plane.from_host(dr), ops.Plane.from_host(di)))
        a, b = zr.copy(), zi.copy()
        if n:
            port.sgd_update(a, b, dr.copy(), di.copy(), 0.5)
        want.append((a, b, dr, di))
    arr = lambda ptrs: (C.c_void_p * len(ptrs))(*ptrs)
    lens = (C.c_int64 * len(sizes))(*sizes)
    capi.call("cnet_sgd_update_multi", len(sizes), arr([z.re.ptr for z in zs]), arr([z.im.ptr for z in zs]),
              arr([d[0].ptr for d in ds]), arr([d[1].ptr for d in ds]), lens, 0.5, 0)
    for n, z, d, (a, b, dr, di) in zip(sizes, zs, ds, want):
        h = z.host()
        assert np.array_equal(h[0], a) and np.array_equal(h[1], b), n
        assert np.array_equal(d[0].host(), dr) and np.array_equal(d[1].host(), di), n


def test_operand_rows_further_apart_than_32_bit_offsets_reach(gpu):
    """A K-contiguous operand whose rows lie 8.4 M floats apart: inside a 128-row block the byte offset of the last rows
    passes 2^32, which the kernel that moves tiles straight into LDS cannot address.  Such a product must take the kernel
    with 64-bit offsets and give the same result (4.3 GB of device memory per plane, written row by row)."""
    M, N, K = 128, 64, 32
    ld = (1 << 32) // 4 // 127 + 8        # 127 * ld * 4 > 2^32
    assert ld % 4 == 0 and 127 * ld * 4 >= 1 << 32
    rng = np.random.default_rng(11)
    ar, ai = rng.standard_normal((M, K), dtype=np.float32), rng.standard_normal((M, K), dtype=np.float32)
    br, bi = rng.standard_normal((N, K), dtype=np.float32), rng.standard_normal((N, K), dtype=np.float32)
    bytes_plane = ((M - 1) * ld + K) * 4
    pa = [C.c_void_p(), C.c_void_p()]
    for p in pa:
        capi.call("cnet_alloc", bytes_plane, C.byref(p))
    try:
        for p, host in zip(pa, (ar, ai)):
            for r in range(M):
                row = np.ascontiguousarray(host[r])
                capi.call("cnet_memcpy_h2d", C.c_void_p(p.value + 4 * r * ld), row.ctypes.data_as(C.c_void_p), 4 * K)
        Bm, c = ops.CMat.from_host(br, bi), ops.CMat.empty(M, N)
        capi.call("cnet_cgemm", 0, 0, 0, M, N, K, pa[0], pa[1], ld, *Bm.p(), Bm.ld, *c.p(), c.ld, 0)
        want = (ar.astype(np.float64) + 1j * ai) @ (br.astype(np.float64) + 1j * bi).T
        got = c.host()
        err = np.linalg.norm(got[0] + 1j * got[1] - want) / np.linalg.norm(want)
        assert err < 1e-6, err
    finally:
        for p in pa:
            capi.call("cnet_free", p)


def test_out_of_range_labels_and_token_ids_touch_nothing_outside_their_operands(gpu, port):
    """Upstream indexes with a label or a token id unchecked (impl/crossent.h:62-72, impl/embed.h:113-118; its host side
    asserts).  On the device a wrong index must not become a wild access: the loss of such a row is NaN, such a token
    is padding, and the rows with valid indices are unaffected."""
    B, n = 4, 24
    zr, zi = seeded(port, 7, (B, n)), seeded(port, 8, (B, n))
    good = np.array([3, 0, 23, 5], np.int32)
    bad = good.copy(); bad[1], bad[3] = n, -7
    _, _, S, loss, pred = port.crossent_fwd(zr, zi, good)
    z = ops.CMat.from_host(zr, zi)
    s, l, am = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
    ops.cross_entropy_fwd(z, ops.ints(bad), s, l, am, None)
    got = l.download()
    assert np.isnan(got[[1, 3]]).all() and np.allclose(got[[0, 2]], loss[[0, 2]], rtol=2e-6)
    assert np.array_equal(am.download(), pred)
    dz = ops.Grad.empty(B, n)
    ops.cross_entropy_bwd(z, s, ops.ints(bad), dz)    # rows 1 and 3: every entry is a non-label entry, z / S
    h = dz.host()
    assert np.allclose(h[2][1], zr[1] / S[1], rtol=1e-6) and np.isfinite(h[2]).all()

    V, D, T = 6, 4, 3
    tr, ti = seeded(port, 9, (V, D)), seeded(port, 10, (V, D))
    tok = np.array([[1, 2, V], [5, V + 100, -1]], np.int32)   # padding only at the tail of a row, as upstream has it
    as_padding = np.where(tok >= V, -1, tok).astype(np.int32)
    yr, yi = port.embedding_fwd(tr, ti, as_padding)
    y = ops.CMat.empty(2, T * D)
    ops.embedding_fwd(ops.CMat.from_host(tr, ti), ops.ints(tok), y, T)
    hy = y.host()
    assert np.array_equal(hy[0], yr) and np.array_equal(hy[1], yi)
    gs = [seeded(port, 11 + p, (2, T * D)) for p in range(2)]
    dsr, dsi = port.embedding_bwd(V, D, as_padding, gs[0], gs[1])
    d_re, d_im = ops.Plane.empty(V, D), ops.Plane.empty(V, D)
    ops.embedding_bwd(ops.ints(tok), ops.Plane.from_host(gs[0]), ops.Plane.from_host(gs[1]), d_re, d_im, D, V, 2, T)
    assert np.array_equal(d_re.host(), dsr) and np.array_equal(d_im.host(), dsi)


def test_recorded_graph_survives_growth_of_the_workspace(gpu, port):
    """A recording holds the address of the library workspace it was made with (here: the partial blocks of a product
    that is cut along K).  A later, larger request makes the workspace grow; the old one must stay alive for the replay."""
    M, N, K = 8, 24, 2048
    A = seeded(port, 41, (M, K)) + 1j * seeded(port, 42, (M, K))
    Bm = seeded(port, 43, (K, N)) + 1j * seeded(port, 44, (K, N))
    a = ops.CMat.from_host(np.ascontiguousarray(A.real), np.ascontiguousarray(A.imag))
    b = ops.CMat.from_host(np.ascontiguousarray(Bm.real), np.ascontiguousarray(Bm.imag))
    c = ops.CMat.empty(M, N)
    ops.cgemm(a, b, c, M, N, K, 0, 1)      # eager: sizes the workspace for this product
    eager = c.host()
    capi.call("cnet_graph_begin")
    ops.cgemm(a, b, c, M, N, K, 0, 1)
    exe = C.c_void_p()
    capi.call("cnet_graph_end", C.byref(exe))
    # a much larger cut product: the workspace has to grow
    M2, N2, K2 = 128, 512, 8192
    a2, b2, c2 = ops.CMat.empty(M2, K2, zero=True), ops.CMat.empty(K2, N2, zero=True), ops.CMat.empty(M2, N2)
    ops.cgemm(a2, b2, c2, M2, N2, K2, 0, 1)
    capi.sync()
    for _ in range(2):
        c.re.owner.zero(); c.im.owner.zero()
        capi.call("cnet_graph_launch", exe)
        got = c.host()
        assert np.array_equal(got[0], eager[0]) and np.array_equal(got[1], eager[1])
        ops.cgemm(a2, b2, c2, M2, N2, K2, 0, 1)   # eager work on the new workspace in between
        capi.sync()
    capi.call("cnet_graph_destroy", exe)


def test_init_shutdown_init(gpu):
    """Lifetime of the library in a process of its own: nothing works before cnet_init or after cnet_shutdown (a status,
    not a crash), shutdown is idempotent, and a second initialisation gives the same results as the first."""
    import os
    import subprocess
    import sys
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpu_lifecycle_check.py")
    r = subprocess.run([sys.executable, script], capture_output=True, text=True, timeout=280)
    assert r.returncode == 0 and "OK" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_device_copy_caller_stream_and_upload_ordering(gpu, port):
    """cnet_memcpy_d2d, cnet_set_stream (the library launches on a stream the caller owns, here one made with
    hipStreamCreate through the HIP runtime the library itself is linked against) and cnet_upload_wait_compute (an upload
    that must not overtake the kernels queued before it)."""
    hip = C.CDLL("libamdhip64.so")
    src = capi.to_device(seeded(port, 51, (33, 17)))
    dst = capi.zeros((33, 17))
    capi.call("cnet_memcpy_d2d", dst.ptr, src.ptr, src.nbytes)
    capi.sync()
    assert np.array_equal(dst.download(), src.download())

    xr, xi = seeded(port, 52, (40, 64)), seeded(port, 53, (40, 64))
    x, y = ops.CMat.from_host(xr, xi), ops.CMat.empty(40, 64)
    ops.gelu_fwd(x, y)
    want = y.host()
    own = capi.load().cnet_stream()
    ts = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(ts)) == 0
    capi.call("cnet_set_stream", ts)
    assert capi.load().cnet_stream() == ts.value
    y2 = ops.CMat.empty(40, 64)
    ops.gelu_fwd(x, y2)
    assert hip.hipStreamSynchronize(ts) == 0   # the caller's own wait is enough: the kernel ran on its stream
    got = y2.host()
    capi.call("cnet_set_stream", None)     # back to the library's stream
    assert capi.load().cnet_stream() == own
    assert hip.hipStreamDestroy(ts) == 0
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])

    # upload stream held back behind the compute stream: the kernel reads the old contents, then the upload lands
    n = 1 << 20
    host = C.c_void_p()
    capi.call("cnet_host_alloc", 4 * n, C.byref(host))
    pinned = np.ctypeslib.as_array((C.c_float * n).from_address(host.value))
    pinned[:] = 7.0
    a = capi.to_device(np.ones(n, np.float32))
    b = capi.zeros((n,))
    for _ in range(20):                    # some queued work in front
        capi.call("cnet_copy2d", a.ptr, n, b.ptr, n, 1, n)
    capi.call("cnet_upload_wait_compute")
    capi.call("cnet_upload_async", a.ptr, host, 4 * n)
    capi.call("cnet_upload_sync")
    capi.sync()
    assert (b.download() == 1.0).all() and (a.download() == 7.0).all()

    # the way back without a blocking call: copy to page-locked memory on the compute stream, valid once a ticket taken
    # after the copy has been waited for (what reading the loss of a step one step later is built on)
    pinned[:] = -1.0
    capi.call("cnet_copy2d", a.ptr, n, b.ptr, n, 1, n)          # b <- 7 on the compute stream, in front of the copy
    capi.call("cnet_memcpy_d2h_async", host, b.ptr, 4 * n)
    t = C.c_int64(-1)
    capi.call("cnet_copy_ticket", 0, C.byref(t))
    capi.call("cnet_copy_wait", t)
    assert (pinned == 7.0).all()
    assert _status("cnet_memcpy_d2h_async", None, b.ptr, 16) == INVALID
    capi.call("cnet_graph_begin")
    assert _status("cnet_memcpy_d2h_async", host, b.ptr, 4 * n) == UNSUPPORTED
    assert _status("cnet_upload_zero", b.ptr, 16) == UNSUPPORTED
    capi.call("cnet_graph_end", None)
    # clearing on the upload stream, in order with the copies queued there: copy 7s, clear the first half, copy 7s to the end
    assert _status("cnet_upload_zero", None, 16) == INVALID and _status("cnet_upload_zero", None, 0) == 0
    pinned[:] = 7.0
    capi.call("cnet_upload_async", a.ptr, host, 4 * n)
    capi.call("cnet_upload_zero", a.ptr, 2 * n)
    capi.call("cnet_upload_async", a.ptr + 3 * n, host, n)
    capi.call("cnet_upload_sync")
    got = a.download()
    assert (got[: n // 2] == 0.0).all() and (got[n // 2:] == 7.0).all()
    # two regions in one call: a small pair travels in one kernel launch that reads the page-locked memory, a large one as two
    # queued copies; either way the compute stream can wait for the ticket taken behind them
    pinned[:] = np.arange(n, dtype=np.float32)
    for words0, words1, off in ((50176, 64, 0), (50176, 64, 1), (3, 0, 0), (0, 5, 0), (n - 1024, 512, 0)):
        capi.call("cnet_memset_zero", a.ptr, 4 * n)
        capi.call("cnet_memset_zero", b.ptr, 4 * n)
        capi.call("cnet_upload_wait_compute")                    # the upload starts behind the clearing
        capi.call("cnet_upload_pair", a.ptr + 4 * off, host.value + 4 * off, 4 * words0, b.ptr, host.value + 4 * (n - 1024), 4 * words1)
        t = C.c_int64(-1)
        capi.call("cnet_copy_ticket", 1, C.byref(t))
        capi.call("cnet_compute_wait_ticket", t)
        c = capi.zeros((n,))
        capi.call("cnet_copy2d", a.ptr, n, c.ptr, n, 1, n)       # on the compute stream, behind the wait
        capi.sync()
        want = np.zeros(n, np.float32)
        want[off:off + words0] = np.arange(off, off + words0)
        assert np.array_equal(c.download(), want), (words0, words1, off)
        got1 = b.download()
        assert np.array_equal(got1[:words1], np.arange(n - 1024, n - 1024 + words1)) and (got1[words1:] == 0).all()
    # a source that does not come from cnet_host_alloc (pageable memory) is not handed to a kernel: it goes through the runtime's copy
    pageable = np.arange(1000, 1512, dtype=np.float32)
    capi.call("cnet_upload_wait_compute")
    capi.call("cnet_upload_pair", a.ptr, pageable.ctypes.data, pageable.nbytes, b.ptr, host.value, 16)
    capi.call("cnet_upload_sync")
    assert np.array_equal(a.download()[:512], pageable) and np.array_equal(b.download()[:4], pinned[:4])
    assert _status("cnet_upload_pair", a.ptr, host, 6, b.ptr, host, 4) == INVALID        # not whole words
    assert _status("cnet_upload_pair", None, host, 8, b.ptr, host, 4) == INVALID
    assert _status("cnet_upload_pair", None, None, 0, None, None, 0) == 0
    t0 = C.c_int64(-1)
    capi.call("cnet_copy_ticket", 0, C.byref(t0))
    assert _status("cnet_compute_wait_ticket", t0.value) == INVALID                      # a point of the compute stream itself
    assert _status("cnet_compute_wait_ticket", t.value + 2) == INVALID and _status("cnet_compute_wait_ticket", -1) == INVALID
    capi.call("cnet_graph_begin")
    assert _status("cnet_upload_pair", a.ptr, host, 8, b.ptr, host, 4) == UNSUPPORTED
    assert _status("cnet_compute_wait_ticket", t.value) == UNSUPPORTED
    capi.call("cnet_graph_end", None)
    del pinned
    capi.call("cnet_host_free", host)


def test_rows_of_a_table_on_the_device_into_a_batch_buffer(gpu):
    """cnet_upload_gather_rows: rows and labels named by indices in page-locked memory, one and two planes, aligned and odd
    widths, a window of a wider buffer; indices outside the table, in pageable memory, or a label array without its twin are
    refused with an error code."""
    import ctypes as C
    lib = capi.load()
    rs = np.random.RandomState(3)
    for count, dim, rows, planes, pad in [(50, 784, 64, 1, 0), (37, 33, 8, 2, 3), (4, 4, 1, 2, 0), (300, 128, 4096, 2, 4)]:
        table = rs.randn(planes, count, dim).astype(np.float32)
        labels = rs.randint(0, 10, count).astype(np.int32)
        d_table, d_labels = capi.to_device(table), capi.to_device(labels)
        ld = dim + pad
        d_out = capi.to_device(np.full((planes, rows, ld), -7.0, np.float32))
        d_lab = capi.to_device(np.full(rows, -1, np.int32))
        hp = C.c_void_p()
        capi.call("cnet_host_alloc", rows * 4, C.byref(hp))
        idx = np.ctypeslib.as_array(C.cast(hp, C.POINTER(C.c_int32)), shape=(rows,))
        idx[:] = rs.randint(0, count, rows)
        capi.call("cnet_upload_wait_compute")   # the fills above ran on the compute stream
        capi.call("cnet_upload_gather_rows", d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab.ptr,
                  d_labels.ptr, rows, dim)
        capi.call("cnet_upload_sync")
        out = d_out.download()
        assert np.array_equal(out[:, :, :dim], table[:, idx, :])
        assert (out[:, :, dim:] == -7.0).all()
        assert np.array_equal(d_lab.download(), labels[idx])
        # samples only
        capi.call("cnet_upload_gather_rows", d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, 1, count, hp, None, None, rows, dim)
        capi.call("cnet_upload_sync")
        # the twin on the compute stream
        d_out2 = capi.to_device(np.full((planes, rows, ld), -7.0, np.float32))
        d_lab2 = capi.to_device(np.full(rows, -1, np.int32))
        capi.call("cnet_gather_rows", d_out2.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab2.ptr, d_labels.ptr, rows, dim)
        assert np.array_equal(d_out2.download(), out) and np.array_equal(d_lab2.download(), labels[idx])
        assert lib.cnet_gather_rows(d_out2.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, 3, count, hp, d_lab2.ptr, d_labels.ptr, rows, dim) == -2
        assert "cnet_gather_rows" in _msg()
        # refused: an index outside the table, a lone label array, indices in pageable memory
        keep = int(idx[0])
        idx[0] = count
        assert lib.cnet_upload_gather_rows(d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab.ptr, d_labels.ptr, rows, dim) == -2
        idx[0] = -1
        assert lib.cnet_upload_gather_rows(d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab.ptr, d_labels.ptr, rows, dim) == -2
        idx[0] = keep
        assert lib.cnet_upload_gather_rows(d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab.ptr, None, rows, dim) == -2
        pageable = np.zeros(rows, np.int32)
        assert lib.cnet_upload_gather_rows(d_out.ptr, ld, rows * ld, d_table.ptr, dim, count * dim, planes, count, pageable.ctypes.data, d_lab.ptr,
                                           d_labels.ptr, rows, dim) == -2
        assert lib.cnet_upload_gather_rows(d_out.ptr, dim - 1, rows * ld, d_table.ptr, dim, count * dim, planes, count, hp, d_lab.ptr, d_labels.ptr, rows, dim) == -2
        assert "cnet_upload_gather_rows" in _msg()
        capi.call("cnet_upload_sync")
        capi.call("cnet_host_free", hp)
