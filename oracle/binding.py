"""ctypes binding of the CPU oracle libraries (TEST INFRASTRUCTURE ONLY).

Two shared objects export the same ``cno_net_*`` graph API:

* ``oracle/liboracle.so``        -- the restatement (``cnet_oracle.hpp``), plus batch loops;
* ``oracle/_ref/libcnet_ref.so`` -- the upstream CNet CPU classes compiled from the upstream tree.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this module; it is the checker, never the product path.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
PORT_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libcnet_ref.so")

# node kinds (numeric ids of impl/cnet.h:31-42 upstream)
HADAMARD, EMBEDDING, LINEAR, FOURIER, CROSSENT, RESIDUAL, SOFTMAX, INPUT, GELU, L2OUT = 1, 2, 3, 4, 5, 6, 7, 8, 10, 11
CRELU, TRIANG_FOURIER = 9, 12
# plane ids of a node's input block
RE, IM, DZ_RE, DZ_IM, DZS_RE, DZS_IM, OUT_RE, OUT_IM = range(8)

_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int)


def _fp(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f32p)


def _ip(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_i32p)


def _p4(planes):
    arr = (_f32p * 4)(*[_fp(p) for p in planes])
    return arr


class OracleLib:
    """One loaded oracle backend ("port" or "reference")."""

    def __init__(self, path):
        self.path = path
        self.lib = C.CDLL(path)
        L = self.lib
        L.cno_backend.restype = C.c_char_p
        L.cno_threads.restype = C.c_int
        L.cno_net_new.restype = C.c_void_p
        L.cno_net_free.argtypes = [C.c_void_p]
        L.cno_net_add.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _i32p, C.c_int]
        L.cno_net_add.restype = C.c_int
        L.cno_net_len.argtypes = [C.c_void_p, C.c_int]
        L.cno_net_len.restype = C.c_int
        L.cno_net_plane.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.cno_net_plane.restype = _f32p
        L.cno_net_set_tokens.argtypes = [C.c_void_p, C.c_int, _i32p, C.c_int]
        L.cno_net_forward.argtypes = [C.c_void_p]
        L.cno_net_backward.argtypes = [C.c_void_p, C.c_int]
        L.cno_net_update.argtypes = [C.c_void_p, C.c_float, C.c_int]
        L.cno_net_save.argtypes = [C.c_void_p, C.c_char_p, C.c_long]
        L.cno_net_save.restype = C.c_long
        L.cno_net_restore.argtypes = [C.c_void_p, C.c_char_p, C.c_long]
        L.cno_net_count.argtypes = [C.c_void_p]
        L.cno_net_uid_at.argtypes = [C.c_void_p, C.c_int]
        L.cno_net_kind.argtypes = [C.c_void_p, C.c_int]
        L.cno_net_adam_update.argtypes = [C.c_void_p, C.c_float, C.c_int, C.c_float, C.c_int]
        L.cno_net_loss.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.cno_net_loss.restype = C.c_float
        L.cno_net_prediction.argtypes = [C.c_void_p, C.c_int]
        L.cno_net_prediction.restype = C.c_int
        L.cno_node_forward.argtypes = [C.c_void_p, C.c_int]
        L.cno_node_backward.argtypes = [C.c_void_p, C.c_int, C.c_int]
        L.cno_node_zero_gradients.argtypes = [C.c_void_p, C.c_int]
        L.cno_fill_normal.argtypes = [C.c_uint64, C.c_long, C.c_double, C.c_double, _f32p]
        L.cno_fill_uniform.argtypes = [C.c_uint64, C.c_long, C.c_double, C.c_double, _f32p]
        self.backend = L.cno_backend().decode()
        self.threads = L.cno_threads()

    # -------------------------------------------------------------- generators
    def normal(self, seed, shape, mu=0.0, sig=1.0):
        out = np.empty(shape, np.float32)
        self.lib.cno_fill_normal(seed, out.size, mu, sig, _fp(out))
        return out

    def uniform(self, seed, shape, lo=0.0, hi=1.0):
        out = np.empty(shape, np.float32)
        self.lib.cno_fill_uniform(seed, out.size, lo, hi, _fp(out))
        return out

    def randint(self, seed, shape, high):
        out = np.empty(shape, np.int32)
        self.lib.cno_fill_int.argtypes = [C.c_uint64, C.c_long, C.c_int, _i32p]
        self.lib.cno_fill_int(seed, out.size, high, _ip(out))
        return out

    def net(self):
        return Net(self)

    # -------------------------------------------------------------- batch loops (port only)
    def linear_fwd(self, xr, xi, wr, wi):
        B, K = xr.shape
        N = wr.shape[0]
        yr = np.empty((B, N), np.float32)
        yi = np.empty((B, N), np.float32)
        self.lib.cno_linear_fwd(B, K, N, _fp(xr), _fp(xi), _fp(wr), _fp(wi), _fp(yr), _fp(yi))
        return yr, yi

    def linear_bwd(self, xr, xi, wr, wi, g4):
        B, K = xr.shape
        N = wr.shape[0]
        dx = [np.empty((B, K), np.float32) for _ in range(4)]
        dw = [np.empty((N, K), np.float32) for _ in range(4)]
        self.lib.cno_linear_bwd(B, K, N, _fp(xr), _fp(xi), _fp(wr), _fp(wi), _p4(g4), _p4(dx), _p4(dw))
        return dx, dw

    def dft_fwd(self, xr, xi):
        B, n = xr.shape
        yr, yi = np.empty_like(xr), np.empty_like(xi)
        self.lib.cno_dft_fwd(B, n, _fp(xr), _fp(xi), _fp(yr), _fp(yi))
        return yr, yi

    def dft_bwd(self, g4):
        B, n = g4[0].shape
        dx = [np.empty((B, n), np.float32) for _ in range(4)]
        self.lib.cno_dft_bwd(B, n, _p4(g4), _p4(dx))
        return dx

    def dft_matrix(self, n):
        fr = np.empty((n, n), np.float32)
        fi = np.empty((n, n), np.float32)
        self.lib.cno_dft_matrix(n, _fp(fr), _fp(fi))
        return fr, fi

    def hadamard_fwd(self, ur, ui, vr, vi):
        B, n = ur.shape
        shared = int(vr.ndim == 1)
        yr, yi = np.empty_like(ur), np.empty_like(ui)
        self.lib.cno_hadamard_fwd(B, n, _fp(ur), _fp(ui), _fp(vr), _fp(vi), shared, _fp(yr), _fp(yi))
        return yr, yi

    def hadamard_bwd(self, ur, ui, vr, vi, g4):
        B, n = ur.shape
        shared = int(vr.ndim == 1)
        du = [np.empty((B, n), np.float32) for _ in range(4)]
        dv = [np.empty(vr.shape, np.float32) for _ in range(4)]
        self.lib.cno_hadamard_bwd(B, n, _fp(ur), _fp(ui), _fp(vr), _fp(vi), shared, _p4(g4), _p4(du), _p4(dv))
        return du, dv

    def gelu_fwd(self, xr, xi):
        yr, yi = np.empty_like(xr), np.empty_like(xi)
        self.lib.cno_gelu_fwd(C.c_long(xr.size), _fp(xr), _fp(xi), _fp(yr), _fp(yi))
        return yr, yi

    def gelu_bwd(self, xr, xi, g4):
        dx = [np.empty_like(xr) for _ in range(4)]
        self.lib.cno_gelu_bwd(C.c_long(xr.size), _fp(xr), _fp(xi), _p4(g4), _p4(dx))
        return dx

    def crelu_fwd(self, xr, xi):
        yr, yi = np.empty_like(xr), np.empty_like(xi)
        self.lib.cno_crelu_fwd(C.c_long(xr.size), _fp(xr), _fp(xi), _fp(yr), _fp(yi))
        return yr, yi

    def crelu_bwd(self, xr, xi, g4):
        dx = [np.empty_like(xr) for _ in range(4)]
        self.lib.cno_crelu_bwd(C.c_long(xr.size), _fp(xr), _fp(xi), _p4(g4), _p4(dx))
        return dx

    def triang_fwd(self, xr, xi):
        B, n = xr.shape
        yr, yi = np.empty_like(xr), np.empty_like(xi)
        self.lib.cno_triang_fwd(B, n, _fp(xr), _fp(xi), _fp(yr), _fp(yi))
        return yr, yi

    def triang_bwd(self, g4):
        B, n = g4[0].shape
        dx = [np.empty((B, n), np.float32) for _ in range(4)]
        self.lib.cno_triang_bwd(B, n, _p4(g4), _p4(dx))
        return dx

    def residual_fwd(self, ur, ui, vr, vi):
        yr, yi = np.empty_like(ur), np.empty_like(ui)
        self.lib.cno_residual_fwd(C.c_long(ur.size), _fp(ur), _fp(ui), _fp(vr), _fp(vi), _fp(yr), _fp(yi))
        return yr, yi

    def residual_bwd(self, g4):
        du = [np.empty_like(g4[0]) for _ in range(4)]
        dv = [np.empty_like(g4[0]) for _ in range(4)]
        self.lib.cno_residual_bwd(C.c_long(g4[0].size), _p4(g4), _p4(du), _p4(dv))
        return du, dv

    def softmax_fwd(self, zr, zi):
        B, n = zr.shape
        yr, yi = np.empty_like(zr), np.empty_like(zi)
        S = np.empty(B, np.float32)
        self.lib.cno_softmax_fwd(B, n, _fp(zr), _fp(zi), _fp(yr), _fp(yi), _fp(S))
        return yr, yi, S

    def softmax_bwd(self, zr, zi, g4):
        B, n = zr.shape
        dz = [np.empty_like(zr) for _ in range(4)]
        self.lib.cno_softmax_bwd(B, n, _fp(zr), _fp(zi), _p4(g4), _p4(dz))
        return dz

    def crossent_fwd(self, zr, zi, labels):
        B, n = zr.shape
        outr, outi = np.empty_like(zr), np.empty_like(zi)
        S = np.empty(B, np.float32)
        loss = np.empty(B, np.float32)
        pred = np.empty(B, np.int32)
        self.lib.cno_crossent_fwd(B, n, _fp(zr), _fp(zi), _ip(labels), _fp(outr), _fp(outi), _fp(S), _fp(loss),
                                  _ip(pred))
        return outr, outi, S, loss, pred

    def crossent_bwd(self, zr, zi, labels):
        B, n = zr.shape
        dz = [np.zeros_like(zr) for _ in range(4)]
        self.lib.cno_crossent_bwd(B, n, _fp(zr), _fp(zi), _ip(labels), _p4(dz))
        return dz

    def l2out_fwd(self, zr, zi):
        B, n = zr.shape
        loss = np.empty(B, np.float32)
        self.lib.cno_l2out_fwd(B, n, _fp(zr), _fp(zi), _fp(loss))
        return loss

    def l2out_bwd(self, zr, zi):
        B, n = zr.shape
        dz = [np.empty_like(zr) for _ in range(4)]
        self.lib.cno_l2out_bwd(B, n, _fp(zr), _fp(zi), _p4(dz))
        return dz

    def embedding_fwd(self, tr, ti, tokens):
        B, T = tokens.shape
        V, D = tr.shape
        yr = np.empty((B, T * D), np.float32)
        yi = np.empty((B, T * D), np.float32)
        self.lib.cno_embedding_fwd(B, T, D, _fp(tr), _fp(ti), _ip(tokens), _fp(yr), _fp(yi))
        return yr, yi

    def embedding_bwd(self, V, D, tokens, gsr, gsi):
        B, T = tokens.shape
        dsr = np.empty((V, D), np.float32)
        dsi = np.empty((V, D), np.float32)
        self.lib.cno_embedding_bwd(B, T, D, V, _ip(tokens), _fp(gsr), _fp(gsi), _fp(dsr), _fp(dsi))
        return dsr, dsi

    def sgd_update(self, zr, zi, dsr, dsi, lr):
        self.lib.cno_sgd_update(C.c_long(zr.size), _fp(zr), _fp(zi), _fp(dsr), _fp(dsi), C.c_float(lr))

    def adam_update(self, zr, zi, mr, mi, dsr, dsi, lr, beta, t):
        """In place on z and m (first moment); dsr/dsi are left as they are."""
        self.lib.cno_adam_update(C.c_long(zr.size), _fp(zr), _fp(zi), _fp(mr), _fp(mi), _fp(dsr), _fp(dsi), C.c_float(lr),
                                 C.c_float(beta), C.c_int(t))


class Net:
    """Per-sample graph with the upstream step semantics; mirrors ComplexNet's add/forward/backward/update."""

    def __init__(self, lib):
        self.o = lib
        self.h = C.c_void_p(lib.lib.cno_net_new())
        self.kind = {}

    def __del__(self):
        try:
            self.o.lib.cno_net_free(self.h)
        except Exception:
            pass

    def add(self, kind, p0, p1=0, p2=0, inputs=()):
        ins = np.asarray(list(inputs), np.int32)
        uid = self.o.lib.cno_net_add(self.h, kind, p0, p1, p2, _ip(ins) if ins.size else None, int(ins.size))
        assert uid > 0
        self.kind[uid] = kind
        return uid

    def plane(self, uid, plane):
        """numpy view (no copy) of one plane of a node's input block (or output block for plane 6/7)."""
        n = self.o.lib.cno_net_len(self.h, uid)
        if plane >= 6:  # output block: CrossEntropy keeps n normalised values, L2Out one loss value
            n = n if self.kind[uid] == CROSSENT else 1
        ptr = self.o.lib.cno_net_plane(self.h, uid, plane)
        assert ptr, "no such plane"
        return np.ctypeslib.as_array(ptr, shape=(n,))

    def set_tokens(self, uid, tokens):
        t = np.asarray(tokens, np.int32)
        self.o.lib.cno_net_set_tokens(self.h, uid, _ip(t), int(t.size))

    def forward(self):
        self.o.lib.cno_net_forward(self.h)

    def backward(self, label=-1):
        self.o.lib.cno_net_backward(self.h, label)

    def update(self, lr, batch=1):
        self.o.lib.cno_net_update(self.h, C.c_float(lr), batch)

    def save(self):
        """The .mod record stream of this net (bytes)."""
        n = self.o.lib.cno_net_save(self.h, None, 0)
        buf = C.create_string_buffer(n)
        assert self.o.lib.cno_net_save(self.h, buf, n) == n
        return buf.raw

    def restore(self, blob):
        """Append the functions stored in a .mod stream; returns False when the stream is refused."""
        ok = bool(self.o.lib.cno_net_restore(self.h, blob, len(blob)))
        if ok:
            for uid in self.uids():
                self.kind[uid] = self.o.lib.cno_net_kind(self.h, uid)
        return ok

    def uids(self):
        return [self.o.lib.cno_net_uid_at(self.h, k) for k in range(self.o.lib.cno_net_count(self.h))]

    def adam_update(self, lr, batch, beta, t):
        self.o.lib.cno_net_adam_update(self.h, C.c_float(lr), batch, C.c_float(beta), t)

    def loss(self, uid, label=0):
        return self.o.lib.cno_net_loss(self.h, uid, label)

    def prediction(self, uid):
        return self.o.lib.cno_net_prediction(self.h, uid)

    def node_forward(self, uid):
        self.o.lib.cno_node_forward(self.h, uid)

    def node_backward(self, uid, label=-1):
        self.o.lib.cno_node_backward(self.h, uid, label)

    def zero_gradients(self, uid):
        self.o.lib.cno_node_zero_gradients(self.h, uid)


_cache = {}


def load_port():
    if "port" not in _cache:
        if not os.path.exists(PORT_SO):
            raise RuntimeError("oracle/liboracle.so is not built (run `make -C oracle`)")
        _cache["port"] = OracleLib(PORT_SO)
    return _cache["port"]


def load_ref():
    """The compiled upstream classes, or None when oracle/_ref was not built."""
    if "ref" not in _cache:
        _cache["ref"] = OracleLib(REF_SO) if os.path.exists(REF_SO) else None
    return _cache["ref"]
