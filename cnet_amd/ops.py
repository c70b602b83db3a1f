"""Thin Python call wrappers over the C-ABI layer entry points (argument marshalling only; used by tests and bench).

A complex matrix on the device is a `CMat`: two planes (re, im) of one DevArray pair with a leading dimension.
A gradient carrier is a `Grad`: four planes.  `sub(col0, cols)` selects a column window without copying, which is
how a producer writes into its slot of a consumer's concatenated input block.
"""
import numpy as np

from . import capi
from .capi import call


class Plane:
    """One fp32 plane: device pointer, logical shape, leading dimension (elements)."""

    def __init__(self, ptr, rows, cols, ld, owner=None):
        self.ptr, self.rows, self.cols, self.ld, self.owner = ptr, rows, cols, ld, owner

    @staticmethod
    def from_host(a):
        a = np.ascontiguousarray(a, np.float32)
        if a.ndim == 1:
            a = a.reshape(1, -1)
        d = capi.to_device(a)
        return Plane(d.ptr, a.shape[0], a.shape[1], a.shape[1], d)

    @staticmethod
    def empty(rows, cols, ld=None, zero=False):
        ld = ld or cols
        d = capi.DevArray((rows, ld))
        if zero:
            d.zero()
        return Plane(d.ptr, rows, cols, ld, d)

    def sub(self, col0, cols):
        return Plane(self.ptr + 4 * col0, self.rows, cols, self.ld, self.owner)

    def rows_from(self, row0, rows):
        """rows row0 .. row0 + rows of the same columns, without copying"""
        return Plane(self.ptr + 4 * row0 * self.ld, rows, self.cols, self.ld, self.owner)

    def host(self):
        full = self.owner.download().reshape(-1)
        base = (self.ptr - self.owner.ptr) // 4
        if self.ld == self.cols:
            return full[base:base + self.rows * self.cols].reshape(self.rows, self.cols)
        idx = base + np.arange(self.rows)[:, None] * self.ld + np.arange(self.cols)[None, :]
        return full[idx]


class CMat:
    def __init__(self, re, im):
        self.re, self.im = re, im
        self.rows, self.cols, self.ld = re.rows, re.cols, re.ld
        assert im.ld == re.ld and im.cols == re.cols

    @staticmethod
    def from_host(re, im):
        return CMat(Plane.from_host(re), Plane.from_host(im))

    @staticmethod
    def empty(rows, cols, ld=None, zero=False):
        return CMat(Plane.empty(rows, cols, ld, zero), Plane.empty(rows, cols, ld, zero))

    def sub(self, col0, cols):
        return CMat(self.re.sub(col0, cols), self.im.sub(col0, cols))

    def rows_from(self, row0, rows):
        return CMat(self.re.rows_from(row0, rows), self.im.rows_from(row0, rows))

    def host(self):
        return self.re.host(), self.im.host()

    def p(self):
        return (self.re.ptr, self.im.ptr)


class Grad:
    def __init__(self, planes):
        self.planes = list(planes)
        self.rows, self.cols, self.ld = planes[0].rows, planes[0].cols, planes[0].ld

    @staticmethod
    def from_host(four):
        return Grad([Plane.from_host(a) for a in four])

    @staticmethod
    def empty(rows, cols, ld=None, zero=False):
        return Grad([Plane.empty(rows, cols, ld, zero) for _ in range(4)])

    def sub(self, col0, cols):
        return Grad([p.sub(col0, cols) for p in self.planes])

    def rows_from(self, row0, rows):
        return Grad([p.rows_from(row0, rows) for p in self.planes])

    def host(self):
        return [p.host() for p in self.planes]

    def p(self):
        return tuple(p.ptr for p in self.planes)


def ints(a):
    return capi.to_device(np.ascontiguousarray(a, np.int32))


# ------------------------------------------------------------------------------------------------- GEMM family
def cgemm(A, Bm, Cm, M, N, K, a_kmajor=0, b_kmajor=0, conj_b=0, accumulate=0):
    call("cnet_cgemm", a_kmajor, b_kmajor, conj_b, M, N, K, *A.p(), A.ld, *Bm.p(), Bm.ld, *Cm.p(), Cm.ld, accumulate)


def cgemm_batched(A, stride_a, Bm, stride_b, Cm, stride_c, M, N, K, batch, a_kmajor=0, b_kmajor=0, conj_a=0, conj_b=0,
                  accumulate=0):
    call("cnet_cgemm_batched", a_kmajor, b_kmajor, conj_a, conj_b, M, N, K, *A.p(), A.ld, stride_a, *Bm.p(), Bm.ld, stride_b,
         *Cm.p(), Cm.ld, stride_c, batch, accumulate)


def linear_fwd(x, w, y, accumulate=0):
    call("cnet_clinear_fwd", *x.p(), x.ld, *w.p(), w.ld, *y.p(), y.ld, x.rows, x.cols, w.rows, accumulate)


def linear_gelu_fwd(x, w, h, y, accumulate=0):
    assert h.ld == y.ld
    call("cnet_clinear_cgelu_fwd", *x.p(), x.ld, *w.p(), w.ld, *h.p(), *y.p(), y.ld, x.rows, x.cols, w.rows, accumulate)


def linear_bwd_input(g, w, dx, accumulate=0):
    call("cnet_clinear_bwd_input", *g.p(), g.ld, *w.p(), w.ld, *dx.p(), dx.ld, g.rows, w.cols, w.rows, accumulate)


def linear_bwd_weight(g, x, dw, accumulate=0):
    call("cnet_clinear_bwd_weight", *g.p(), g.ld, *x.p(), x.ld, *dw.p(), dw.ld, g.rows, x.cols, g.cols, accumulate)


def _mirrored(d, mirror):
    p = d.p()
    return (p[0], p[1], p[2] if mirror else None, p[3] if mirror else None)


def linear_bwd_input_sym(g, w, dx, accumulate=0, mirror=True):
    """g is a Grad whose dz* planes are the conjugate of its dz planes; only the dz planes are read.  mirror=False: the
    dz* planes of the result are not written."""
    call("cnet_clinear_bwd_input_sym", *g.p()[:2], g.ld, *w.p(), w.ld, *_mirrored(dx, mirror), dx.ld, g.rows, w.cols, w.rows,
         accumulate)


def linear_bwd_weight_sym(g, x, dw, accumulate=0, mirror=True):
    call("cnet_clinear_bwd_weight_sym", *g.p()[:2], g.ld, *x.p(), x.ld, *_mirrored(dw, mirror), dw.ld, g.rows, x.cols, g.cols,
         accumulate)


def linear_bwd_sym(g, x, w, dx, dw, accumulate_dx=0, accumulate_dw=0, mirror_dx=True, mirror_dw=True):
    """Both gradients of a Linear in one call (one launch when both products are small)."""
    call("cnet_clinear_bwd_sym", *g.p()[:2], g.ld, *x.p(), x.ld, *w.p(), w.ld, *_mirrored(dx, mirror_dx), dx.ld, accumulate_dx,
         *_mirrored(dw, mirror_dw), dw.ld, accumulate_dw, g.rows, w.cols, w.rows)


def linear_hadamard_gelu_bwd_sym(g, x, w, dx, dw, u, v, dh, du, dv, accumulate_dx=0, accumulate_dw=0, accumulate_gate=0, mirror=True):
    """linear_bwd_sym, then hadamard_gelu_bwd_sym with a shared row v on dx, in one call (one launch at small batches)."""
    ph = _pair(dh, mirror) if dh is not None else (None,) * 4
    call("cnet_clinear_hadamard_cgelu_bwd_sym", *g.p()[:2], g.ld, *x.p(), x.ld, *w.p(), w.ld, *_mirrored(dx, mirror), dx.ld, accumulate_dx,
         *_mirrored(dw, mirror), dw.ld, accumulate_dw, *u.p(), u.ld, *v.p(), *ph, dh.ld if dh is not None else 0, *_pair(du, mirror), du.ld,
         *_pair(dv, mirror), accumulate_gate, g.rows, w.cols, w.rows)


def dft_fwd(x, y, accumulate=0):
    call("cnet_cdft_fwd", *x.p(), x.ld, *y.p(), y.ld, x.rows, x.cols, accumulate)


def dft_fwd_real_input(x, y):
    """x holds real samples: its imaginary plane is all +0."""
    call("cnet_cdft_fwd_real_input", *x.p(), x.ld, *y.p(), y.ld, x.rows, x.cols)


def dft_hadamard_gelu_fwd(x, v, y, h, a):
    """y = x F, h = y .* v (v: one shared row), a = gelu(h); y, h and a share a leading dimension."""
    assert y.ld == h.ld == a.ld
    call("cnet_cdft_hadamard_cgelu_fwd", *x.p(), x.ld, *v.p(), *y.p(), *h.p(), *a.p(), y.ld, x.rows, x.cols)


def dft_bwd(g, dx, accumulate=0):
    call("cnet_cdft_bwd", *g.p(), g.ld, *dx.p(), dx.ld, g.rows, g.cols, accumulate)


def dft_bwd_sym(g, dx, accumulate=0, mirror=True):
    call("cnet_cdft_bwd_sym", *g.p()[:2], g.ld, *_mirrored(dx, mirror), dx.ld, g.rows, g.cols, accumulate)


def triang_dft_bwd_sym(g, dx, accumulate=0, mirror=True):
    call("cnet_ctriang_dft_bwd_sym", *g.p()[:2], g.ld, *_mirrored(dx, mirror), dx.ld, g.rows, g.cols, accumulate)


def triang_dft_fwd(x, y, accumulate=0):
    call("cnet_ctriang_dft_fwd", *x.p(), x.ld, *y.p(), y.ld, x.rows, x.cols, accumulate)


def triang_dft_bwd(g, dx, accumulate=0):
    call("cnet_ctriang_dft_bwd", *g.p(), g.ld, *dx.p(), dx.ld, g.rows, g.cols, accumulate)


# ------------------------------------------------------------------------------------------------- elementwise
def hadamard_fwd(u, v, y, shared=False):
    call("cnet_hadamard_fwd", *u.p(), u.ld, *v.p(), 0 if shared else v.ld, *y.p(), y.ld, u.rows, u.cols)


def hadamard_bwd(u, v, g, du, dv, shared=False, accumulate=0):
    call("cnet_hadamard_bwd", *u.p(), u.ld, *v.p(), 0 if shared else v.ld, *g.p(), g.ld, *du.p(), du.ld, *dv.p(),
         dv.ld, u.rows, u.cols, accumulate)


def gelu_fwd(x, y):
    call("cnet_cgelu_fwd", *x.p(), x.ld, *y.p(), y.ld, x.rows, x.cols)


def gelu_bwd(x, g, dx, accumulate=0):
    call("cnet_cgelu_bwd", *x.p(), x.ld, *g.p(), g.ld, *dx.p(), dx.ld, x.rows, x.cols, accumulate)


def crelu_fwd(x, y):
    call("cnet_crelu_fwd", *x.p(), x.ld, *y.p(), y.ld, x.rows, x.cols)


def crelu_bwd(x, g, dx, accumulate=0):
    call("cnet_crelu_bwd", *x.p(), x.ld, *g.p(), g.ld, *dx.p(), dx.ld, x.rows, x.cols, accumulate)


def residual_fwd(u, v, y):
    call("cnet_residual_fwd", *u.p(), u.ld, *v.p(), v.ld, *y.p(), y.ld, u.rows, u.cols)


def residual_bwd(g, du, dv, accumulate=0):
    call("cnet_residual_bwd", *g.p(), g.ld, *du.p(), du.ld, *dv.p(), dv.ld, g.rows, g.cols, accumulate)


def l2norm_fwd(z, y, s):
    call("cnet_l2norm_fwd", *z.p(), z.ld, *y.p(), y.ld, s.ptr, z.rows, z.cols)


def l2norm_bwd(z, s, g, dz, accumulate=0):
    call("cnet_l2norm_bwd", *z.p(), z.ld, s.ptr, *g.p(), g.ld, *dz.p(), dz.ld, z.rows, z.cols, accumulate)


def cross_entropy_fwd(z, labels, s, loss, argmax, out=None):
    o = out.p() if out is not None else (None, None)
    call("cnet_cross_entropy_fwd", *z.p(), z.ld, labels.ptr, o[0], o[1], out.ld if out is not None else 0, s.ptr,
         loss.ptr, argmax.ptr, z.rows, z.cols)


def cross_entropy_bwd(z, s, labels, dz):
    call("cnet_cross_entropy_bwd", *z.p(), z.ld, s.ptr, labels.ptr, *dz.p(), dz.ld, z.rows, z.cols)


def l2out_fwd(z, loss):
    call("cnet_l2out_fwd", *z.p(), z.ld, loss.ptr, z.rows, z.cols)


def l2out_bwd(z, dz, accumulate=0):
    call("cnet_l2out_bwd", *z.p(), z.ld, *dz.p(), dz.ld, z.rows, z.cols, accumulate)


# Backward passes for a conjugate gradient pair: `g` is a Grad whose dz* planes are the conjugate of its dz planes (only the
# dz planes are read); mirror=False leaves the dz* planes of the results untouched (NULL pointers at the C ABI).
def _pair(d, mirror):
    p = d.p()
    return (p[0], p[1], p[2] if mirror else None, p[3] if mirror else None)


def hadamard_bwd_sym(u, v, g, du, dv, shared=False, accumulate=0, mirror=True):
    call("cnet_hadamard_bwd_sym", *u.p(), u.ld, *v.p(), 0 if shared else v.ld, *g.p()[:2], g.ld, *_pair(du, mirror), du.ld,
         *_pair(dv, mirror), dv.ld, u.rows, u.cols, accumulate)


def gelu_bwd_sym(x, g, dx, accumulate=0, mirror=True):
    call("cnet_cgelu_bwd_sym", *x.p(), x.ld, *g.p()[:2], g.ld, *_pair(dx, mirror), dx.ld, x.rows, x.cols, accumulate)


def hadamard_gelu_fwd(u, v, h, y, shared=False):
    call("cnet_hadamard_cgelu_fwd", *u.p(), u.ld, *v.p(), 0 if shared else v.ld, *h.p(), h.ld, *y.p(), y.ld, u.rows, u.cols)


def hadamard_gelu_bwd_sym(u, v, g, dh, du, dv, shared=False, accumulate=0, mirror=True):
    """g: the gradient pair that reaches the CGelu; dh (a Grad or None) receives the CGelu's gradient."""
    ph = _pair(dh, mirror) if dh is not None else (None,) * 4
    call("cnet_hadamard_cgelu_bwd_sym", *u.p(), u.ld, *v.p(), 0 if shared else v.ld, *g.p()[:2], g.ld, *ph,
         dh.ld if dh is not None else 0, *_pair(du, mirror), du.ld, *_pair(dv, mirror), dv.ld, u.rows, u.cols, accumulate)


def crelu_bwd_sym(x, g, dx, accumulate=0, mirror=True):
    call("cnet_crelu_bwd_sym", *x.p(), x.ld, *g.p()[:2], g.ld, *_pair(dx, mirror), dx.ld, x.rows, x.cols, accumulate)


def residual_bwd_sym(g, du, dv, accumulate=0, mirror=True):
    call("cnet_residual_bwd_sym", *g.p()[:2], g.ld, *_pair(du, mirror), du.ld, *_pair(dv, mirror), dv.ld, g.rows, g.cols,
         accumulate)


def residual_bwd_sym2(g1, g2, du, dv, accumulate=0, mirror=True):
    call("cnet_residual_bwd_sym2", *g1.p()[:2], g1.ld, *g2.p()[:2], g2.ld, *_pair(du, mirror), du.ld, *_pair(dv, mirror), dv.ld,
         g1.rows, g1.cols, accumulate)


def residual_gelu_bwd_sym(g1, g2, h, du, dv, dh, mirror=True):
    """g2 and dv may be None (one consumer; the gradient of the CGelu's result not wanted)."""
    p2 = g2.p()[:2] if g2 is not None else (None, None)
    pv = _pair(dv, mirror) if dv is not None else (None,) * 4
    call("cnet_residual_cgelu_bwd_sym", *g1.p()[:2], g1.ld, *p2, g2.ld if g2 is not None else 0, *h.p(), h.ld, *_pair(du, mirror),
         du.ld, *pv, dv.ld if dv is not None else 0, *_pair(dh, mirror), dh.ld, g1.rows, g1.cols)


def l2norm_bwd_sym(z, s, g, dz, accumulate=0, mirror=True):
    call("cnet_l2norm_bwd_sym", *z.p(), z.ld, s.ptr, *g.p()[:2], g.ld, *_pair(dz, mirror), dz.ld, z.rows, z.cols, accumulate)


def l2out_bwd_sym(z, dz, accumulate=0, mirror=True):
    call("cnet_l2out_bwd_sym", *z.p(), z.ld, *_pair(dz, mirror), dz.ld, z.rows, z.cols, accumulate)


def cross_entropy_bwd_sym(z, s, labels, dz, mirror=True):
    call("cnet_cross_entropy_bwd_sym", *z.p(), z.ld, s.ptr, labels.ptr, *_pair(dz, mirror), dz.ld, z.rows, z.cols)


def copy2d(src, dst):
    call("cnet_copy2d", src.ptr, src.ld, dst.ptr, dst.ld, src.rows, src.cols)


def add2d(src, dst):
    call("cnet_add2d", src.ptr, src.ld, dst.ptr, dst.ld, src.rows, src.cols)


def batch_sum(src, dst, accumulate=0):
    call("cnet_batch_sum", src.ptr, src.ld, dst.ptr, src.rows, src.cols, accumulate)


def sgd_update(z, dzs_re, dzs_im, lr, zero_grad=1):
    call("cnet_sgd_update", z.re.ptr, z.im.ptr, dzs_re.ptr, dzs_im.ptr, z.rows * z.cols, lr, zero_grad)


def adam_update(z, m_re, m_im, dzs_re, dzs_im, lr, beta, t, zero_grad=1):
    call("cnet_adam_update", z.re.ptr, z.im.ptr, m_re.ptr, m_im.ptr, dzs_re.ptr, dzs_im.ptr, z.rows * z.cols, lr, beta, t, zero_grad)


def embedding_fwd(table, tokens, y, slots):
    call("cnet_embedding_fwd", *table.p(), table.cols, table.rows, tokens.ptr, *y.p(), y.ld, y.rows, slots)


def embedding_bwd(tokens, gs_re, gs_im, dtab_re, dtab_im, dim, vocab, rows, slots, accumulate=0):
    call("cnet_embedding_bwd", tokens.ptr, gs_re.ptr, gs_im.ptr, gs_re.ld, dtab_re.ptr, dtab_im.ptr, dim, vocab, rows,
         slots, accumulate)


def cross_entropy_fwd_bwd_sym(z, labels, s, loss, argmax, dz, out=None, mirror=True):
    """Forward pass and gradient of the loss in one launch."""
    o = out.p() if out is not None else (None, None)
    call("cnet_cross_entropy_fwd_bwd_sym", *z.p(), z.ld, labels.ptr, o[0], o[1], out.ld if out is not None else 0, s.ptr,
         loss.ptr, argmax.ptr, *_pair(dz, mirror), dz.ld, z.rows, z.cols)


def linear_cross_entropy_fwd_bwd_sym(x, w, y, labels, s, loss, argmax, dz, out=None, mirror=True):
    """y = x w^T, then the loss over the rows of y and its gradient (one launch for a narrow head)."""
    o = out.p() if out is not None else (None, None)
    call("cnet_clinear_cross_entropy_fwd_bwd_sym", *x.p(), x.ld, *w.p(), w.ld, *y.p(), y.ld, labels.ptr, o[0], o[1],
         out.ld if out is not None else 0, s.ptr, loss.ptr, argmax.ptr, *_pair(dz, mirror), dz.ld, x.rows, x.cols, w.rows)
