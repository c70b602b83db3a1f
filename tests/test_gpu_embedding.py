"""CEmbedding gather and dzs scatter-add on the GPU against the CPU oracle and the upstream known answers
(tests/test.h:458-471, 491-533; upstream testEmbedding, tests/gputests.h:594, 1075, 1206)."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from tests.gpu_util import gpu, rel, seeded  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,D,V", [(1, 3, 2, 4), (5, 7, 6, 11), (16, 512, 64, 1000), (4, 33, 1024, 50)])
def test_embedding(gpu, port, B, T, D, V):
    tr, ti = seeded(port, 1, (V, D)), seeded(port, 2, (V, D))
    tok = port.randint(3, (B, T), V)
    for b in range(B):      # ragged rows: -1 padding at the tail
        cut = (b * 3) % T
        if cut:
            tok[b, T - cut:] = -1
    gs = [seeded(port, 4 + p, (B, T * D)) for p in range(2)]
    yr, yi = port.embedding_fwd(tr, ti, tok)
    dsr, dsi = port.embedding_bwd(V, D, tok, gs[0], gs[1])
    table, tokens = ops.CMat.from_host(tr, ti), ops.ints(tok)
    y = ops.CMat.empty(B, T * D)
    ops.embedding_fwd(table, tokens, y, T)
    hy = y.host()
    assert np.array_equal(hy[0], yr) and np.array_equal(hy[1], yi)
    d_re, d_im = ops.Plane.empty(V, D), ops.Plane.empty(V, D)
    ops.embedding_bwd(tokens, ops.Plane.from_host(gs[0]), ops.Plane.from_host(gs[1]), d_re, d_im, D, V, B, T)
    # same summation order as the CPU path (row, slot): identical floats
    assert np.array_equal(d_re.host(), dsr) and np.array_equal(d_im.host(), dsi)
    ops.embedding_bwd(tokens, ops.Plane.from_host(gs[0]), ops.Plane.from_host(gs[1]), d_re, d_im, D, V, B, T, accumulate=1)
    assert rel(d_re.host(), 2 * dsr) < 1e-6


def test_embedding_known_answers(gpu):
    # dz* (1+2i)+(7+8i) and (3+4i)+(9+10i) land on token 2 (tests/test.h:458-471 upstream, two consumers = two rows here)
    tok = ops.ints(np.array([[2], [2]], np.int32))
    gr = ops.Plane.from_host(np.array([[1, 3], [7, 9]], np.float32))
    gi = ops.Plane.from_host(np.array([[2, 4], [8, 10]], np.float32))
    d_re, d_im = ops.Plane.empty(4, 2), ops.Plane.empty(4, 2)
    ops.embedding_bwd(tok, gr, gi, d_re, d_im, 2, 4, 2, 1)
    want_r = np.zeros((4, 2), np.float32); want_r[2] = [8, 12]
    want_i = np.zeros((4, 2), np.float32); want_i[2] = [10, 14]
    assert np.array_equal(d_re.host(), want_r) and np.array_equal(d_im.host(), want_i)
