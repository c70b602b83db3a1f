"""Every elementwise, one-gradient (`*_sym`), fused and row-normalising entry point that picks a cache policy for its 128-bit
accesses, run on fixed inputs; `results()` returns every output array by name, `digests()` a hash of each.

tests/test_gpu_stream_policies.py runs this file in processes of their own with CNET_STREAM_MIN_MB=0 (every launch counts as
streaming) and CNET_STREAM_POLICY = 1, 2, 3 (the library reads both once per process), and compares the digests printed
here with those of the plain instantiations: the hinted loads and the hand-written hinted stores must move the same bits.
The inputs come from numpy's generator, so every process sees the same operands.
"""
import hashlib
import json
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from cnet_amd import capi, ops  # noqa: E402

# all column counts are multiples of four (the 128-bit kernels); 2052 and 4100 columns take the four-wavefront row kernels
SHAPES = [(64, 784), (33, 1028), (130, 36), (6, 2052), (3, 4100)]


def _rng(*key):
    return np.random.default_rng(list(key))


def _planes(key, shape, count, sig=1.0):
    r = _rng(*key)
    return [(sig * r.standard_normal(shape)).astype(np.float32) for _ in range(count)]


def _pair(key, shape):
    re, im = _planes(key, shape, 2)
    return [re, im, re.copy(), -im]


def results(shapes=SHAPES):
    """name -> list of host arrays, for every policy-carrying entry point over `shapes`."""
    out = {}

    def keep(name, *objs):
        arrs = []
        for o in objs:
            if isinstance(o, (ops.CMat, ops.Grad)):
                arrs += list(o.host())
            elif isinstance(o, ops.Plane):
                arrs.append(o.host())
            else:
                arrs.append(o.download())
        assert name not in out, name
        out[name] = arrs

    for B, n in shapes:
        tag = "%dx%d" % (B, n)
        xr, xi = _planes((1, B, n), (B, n), 2, 2.0)
        x = ops.CMat.from_host(xr, xi)
        g = ops.Grad.from_host(_planes((2, B, n), (B, n), 4))
        gp = ops.Grad.from_host(_pair((3, B, n), (B, n)))
        gp2 = ops.Grad.from_host(_pair((4, B, n), (B, n)))
        v = ops.CMat.from_host(*_planes((5, B, n), (B, n), 2, 0.7))
        v1 = ops.CMat.from_host(*_planes((6, B, n), (1, n), 2, 0.7))
        base = _pair((7, B, n), (B, n))
        base1 = _pair((8, B, n), (1, n))

        def dest(rows=B):
            return ops.Grad.from_host(base if rows == B else base1)

        # ---- forward passes
        y, h = ops.CMat.empty(B, n), ops.CMat.empty(B, n)
        ops.gelu_fwd(x, y); keep(tag + " gelu_fwd", y)
        ops.crelu_fwd(x, y); keep(tag + " crelu_fwd", y)
        ops.residual_fwd(x, v, y); keep(tag + " residual_fwd", y)
        for shared, vv in ((0, v), (1, v1)):
            ops.hadamard_fwd(x, vv, y, shared); keep(tag + " hadamard_fwd shared=%d" % shared, y)
            ops.hadamard_gelu_fwd(x, vv, h, y, shared); keep(tag + " hadamard_gelu_fwd shared=%d" % shared, h, y)
        s = ops.Plane.empty(1, B)
        ops.l2norm_fwd(x, y, s); keep(tag + " l2norm_fwd", y, s)
        # ---- both halves of every gradient pair
        for acc in (0, 1):
            a = " acc=%d" % acc
            d = dest(); ops.gelu_bwd(x, g, d, accumulate=acc); keep(tag + " gelu_bwd" + a, d)
            d = dest(); ops.crelu_bwd(x, g, d, accumulate=acc); keep(tag + " crelu_bwd" + a, d)
            d, e = dest(), dest(); ops.residual_bwd(g, d, e, accumulate=acc); keep(tag + " residual_bwd" + a, d, e)
            d = dest(); ops.l2out_bwd(x, d, accumulate=acc); keep(tag + " l2out_bwd" + a, d)
            d = dest(); ops.l2norm_bwd(x, s, g, d, accumulate=acc); keep(tag + " l2norm_bwd" + a, d)
            for shared, vv in ((0, v), (1, v1)):
                d, e = dest(), dest(1 if shared else B)
                ops.hadamard_bwd(x, vv, g, d, e, shared, accumulate=acc)
                keep(tag + " hadamard_bwd shared=%d" % shared + a, d, e)
            # ---- one gradient of a conjugate pair, with and without the planes of its conjugate
            for mirror in (True, False):
                m = a + " mirror=%d" % mirror
                d = dest(); ops.gelu_bwd_sym(x, gp, d, accumulate=acc, mirror=mirror); keep(tag + " gelu_bwd_sym" + m, d)
                d = dest(); ops.crelu_bwd_sym(x, gp, d, accumulate=acc, mirror=mirror); keep(tag + " crelu_bwd_sym" + m, d)
                d, e = dest(), dest(); ops.residual_bwd_sym(gp, d, e, accumulate=acc, mirror=mirror)
                keep(tag + " residual_bwd_sym" + m, d, e)
                d, e = dest(), dest(); ops.residual_bwd_sym2(gp, gp2, d, e, accumulate=acc, mirror=mirror)
                keep(tag + " residual_bwd_sym2" + m, d, e)
                d = dest(); ops.l2out_bwd_sym(x, d, accumulate=acc, mirror=mirror); keep(tag + " l2out_bwd_sym" + m, d)
                d = dest(); ops.l2norm_bwd_sym(x, s, gp, d, accumulate=acc, mirror=mirror); keep(tag + " l2norm_bwd_sym" + m, d)
                for shared, vv in ((0, v), (1, v1)):
                    sh = " shared=%d" % shared
                    d, e = dest(), dest(1 if shared else B)
                    ops.hadamard_bwd_sym(x, vv, gp, d, e, shared, accumulate=acc, mirror=mirror)
                    keep(tag + " hadamard_bwd_sym" + sh + m, d, e)
                    for with_dh in (True, False):
                        d, e, dh = dest(), dest(1 if shared else B), dest()
                        ops.hadamard_gelu_bwd_sym(x, vv, gp, dh if with_dh else None, d, e, shared, accumulate=acc, mirror=mirror)
                        keep(tag + " hadamard_gelu_bwd_sym dh=%d" % with_dh + sh + m, d, e, dh)
        for mirror in (True, False):
            m = " mirror=%d" % mirror
            for two in (True, False):
                for with_dv in (True, False):
                    d, e, dh = dest(), dest(), dest()
                    ops.residual_gelu_bwd_sym(gp, gp2 if two else None, x, d, e if with_dv else None, dh, mirror=mirror)
                    keep(tag + " residual_gelu_bwd_sym two=%d dv=%d" % (two, with_dv) + m, d, e, dh)
        # ---- CrossEntropy
        labels = ops.ints(_rng(9, B, n).integers(0, n, B).astype(np.int32))
        S, loss, am = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
        norm = ops.CMat.empty(B, n)
        ops.cross_entropy_fwd(x, labels, S, loss, am, norm); keep(tag + " cross_entropy_fwd", S, loss, am, norm)
        S1, loss1, am1 = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)   # the pass that only reads
        ops.cross_entropy_fwd(x, labels, S1, loss1, am1, None); keep(tag + " cross_entropy_fwd, no planes", S1, loss1, am1)
        ops.l2out_fwd(x, loss1); keep(tag + " l2out_fwd", loss1)
        d = dest(); ops.cross_entropy_bwd(x, S, labels, d); keep(tag + " cross_entropy_bwd", d)
        for mirror in (True, False):
            d = dest(); ops.cross_entropy_bwd_sym(x, S, labels, d, mirror=mirror); keep(tag + " cross_entropy_bwd_sym mirror=%d" % mirror, d)
            d = dest(); S2, loss2, am2 = capi.empty(B), capi.empty(B), capi.empty(B, np.int32)
            ops.cross_entropy_fwd_bwd_sym(x, labels, S2, loss2, am2, d, out=norm, mirror=mirror)
            keep(tag + " cross_entropy_fwd_bwd_sym mirror=%d" % mirror, S2, loss2, am2, norm, d)
        # ---- copies and parameter steps
        d = dest(); ops.copy2d(x.re, d.planes[0]); ops.add2d(x.im, d.planes[1]); keep(tag + " copy2d add2d", d)
        z = ops.CMat.from_host(xr, xi); gr, gi = (ops.Plane.from_host(p) for p in base[:2])
        ops.sgd_update(z, gr, gi, 0.01, zero_grad=1); keep(tag + " sgd_update", z, gr, gi)
        z = ops.CMat.from_host(xr, xi); gr, gi, mr, mi = (ops.Plane.from_host(p) for p in _planes((10, B, n), (B, n), 4))
        ops.adam_update(z, mr, mi, gr, gi, 0.01, 0.9, 3); keep(tag + " adam_update", z, mr, mi, gr, gi)
    return out


def digest(arrs):
    hsh = hashlib.sha256()
    for a in arrs:
        hsh.update(np.ascontiguousarray(a).tobytes())
    return hsh.hexdigest()


def digests(shapes=SHAPES):
    return {k: digest(v) for k, v in results(shapes).items()}


if __name__ == "__main__":
    capi.init(0)
    print("DIGESTS " + json.dumps(digests()), flush=True)
