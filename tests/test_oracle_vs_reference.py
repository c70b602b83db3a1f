"""The restatement in oracle/cnet_oracle.hpp against the compiled upstream CPU classes (oracle/_ref).

Both libraries export the same per-sample graph API, so each case builds the same small net twice, feeds the
same seeded planes and compares every plane bit for bit (np.array_equal), as the upstream GPU-vs-CPU tests
compare mappings (tests/gputests.h upstream), but exact.  Skipped where oracle/_ref is not built; the golden
fixtures written from the same library (tests/golden/) cover that case.
"""
import numpy as np
import pytest

from oracle import binding as ob


def _fill(net, uid, plane, data):
    net.plane(uid, plane)[:] = data


def _same(a, b, what):
    assert a.shape == b.shape
    if not np.array_equal(a, b):
        bad = np.flatnonzero(a != b)
        raise AssertionError("%s differs at %d of %d entries, first %d: %r vs %r"
                             % (what, bad.size, a.size, bad[0], a[bad[0]], b[bad[0]]))


def _layer_case(port, ref, kind, params, in_sizes, seed, consumers=1, label=-1):
    """inputs (CInput per in_size) -> layer -> `consumers` L2Out sinks; returns nothing, asserts equality."""
    nets = []
    for lib in (port, ref):
        net = lib.net()
        ins = [net.add(ob.INPUT, s) for s in in_sizes]
        lay = net.add(kind, *params, inputs=ins)
        out_len = None
        sinks = []
        nets.append((net, ins, lay, sinks))
    # out size from the port restatement
    rng = np.random.RandomState(seed)
    data = [(rng.randn(s).astype(np.float32), rng.randn(s).astype(np.float32)) for s in in_sizes]
    out_size = {ob.LINEAR: lambda: params[1] // params[0]}.get(kind, lambda: params[0])()
    g = [[rng.randn(out_size).astype(np.float32) for _ in range(4)] for _ in range(consumers)]
    results = []
    for (net, ins, lay, sinks) in nets:
        for _ in range(consumers):
            sinks.append(net.add(ob.L2OUT, out_size, inputs=[lay]))
        for uid, (re, im) in zip(ins, data):
            _fill(net, uid, ob.RE, re)
            _fill(net, uid, ob.IM, im)
            net.node_forward(uid)
        net.node_forward(lay)
        fwd = [np.concatenate([net.plane(s, ob.RE), net.plane(s, ob.IM)]).copy() for s in sinks]
        for s, gs in zip(sinks, g):
            for p, arr in zip((ob.DZ_RE, ob.DZ_IM, ob.DZS_RE, ob.DZS_IM), gs):
                _fill(net, s, p, arr)
        net.node_backward(lay, label)
        grads = np.concatenate([net.plane(lay, p) for p in (ob.DZ_RE, ob.DZ_IM, ob.DZS_RE, ob.DZS_IM)]).copy()
        for uid in ins:
            net.node_backward(uid)
        pin = [np.concatenate([net.plane(uid, ob.DZS_RE), net.plane(uid, ob.DZS_IM)]).copy() for uid in ins]
        results.append((fwd, grads, pin))
    (f0, g0, p0), (f1, g1, p1) = results
    for a, b in zip(f0, f1):
        _same(a, b, "forward")
    _same(g0, g1, "layer input gradients")
    for a, b in zip(p0, p1):
        _same(a, b, "gathered dz*")
    assert np.all(np.isfinite(g0))


@pytest.mark.parametrize("K,N", [(1, 1), (3, 5), (16, 8), (64, 32), (257, 19)])
def test_linear(port, ref, K, N):
    _layer_case(port, ref, ob.LINEAR, (K, K * N), [K, K * N], seed=K * 100 + N)


def test_linear_two_consumers(port, ref):
    _layer_case(port, ref, ob.LINEAR, (12, 12 * 7), [12, 12 * 7], seed=5, consumers=2)


@pytest.mark.parametrize("n", [1, 2, 4, 8, 64, 512, 3, 6, 12, 100, 784])
def test_fourier(port, ref, n):
    _layer_case(port, ref, ob.FOURIER, (n,), [n], seed=n)


def test_fourier_4096(port, ref):
    _layer_case(port, ref, ob.FOURIER, (4096,), [4096], seed=4096)


@pytest.mark.parametrize("n", [1, 6, 784])
def test_hadamard(port, ref, n):
    _layer_case(port, ref, ob.HADAMARD, (n,), [n, n], seed=n, consumers=2)


@pytest.mark.parametrize("n", [1, 6, 1000])
def test_gelu(port, ref, n):
    _layer_case(port, ref, ob.GELU, (n,), [n], seed=n)


@pytest.mark.parametrize("n", [1, 6, 1000])
def test_crelu(port, ref, n):
    _layer_case(port, ref, ob.CRELU, (n,), [n], seed=n, consumers=2)


@pytest.mark.parametrize("n", [1, 2, 7, 64, 100])
def test_triang_fourier(port, ref, n):
    _layer_case(port, ref, ob.TRIANG_FOURIER, (n,), [n], seed=n, consumers=2)


@pytest.mark.parametrize("n", [1, 6, 300])
def test_residual(port, ref, n):
    _layer_case(port, ref, ob.RESIDUAL, (n,), [n, n], seed=n, consumers=2)


@pytest.mark.parametrize("n", [1, 2, 6, 97])
def test_softmax(port, ref, n):
    _layer_case(port, ref, ob.SOFTMAX, (n,), [n], seed=n)


@pytest.mark.parametrize("n", [1, 2, 10, 333])
def test_cross_entropy_and_l2(port, ref, n):
    rng = np.random.RandomState(n)
    z = rng.randn(2, n).astype(np.float32)
    if n == 333:
        z[:, 5] = 0  # a zero entry; the label below lands on it -> clamp path
    out = []
    for lib in (port, ref):
        net = lib.net()
        i = net.add(ob.INPUT, n)
        ce = net.add(ob.CROSSENT, n, inputs=[i])
        j = net.add(ob.INPUT, n)
        l2 = net.add(ob.L2OUT, n, inputs=[j])
        for u in (i, j):
            _fill(net, u, ob.RE, z[0])
            _fill(net, u, ob.IM, z[1])
        net.forward()
        label = 5 % n
        rec = [net.plane(ce, ob.OUT_RE).copy(), net.plane(ce, ob.OUT_IM).copy(),
               np.float32(net.loss(ce, label)), np.int32(net.prediction(ce)), np.float32(net.loss(l2, 0))]
        net.backward(label)
        for u in (ce, l2, i, j):
            rec += [net.plane(u, p).copy() for p in range(2, 6)]
        out.append(rec)
    for k, (a, b) in enumerate(zip(*out)):
        _same(np.atleast_1d(a), np.atleast_1d(b), "record %d" % k)


def test_cross_entropy_all_zero_input(port, ref):
    out = []
    for lib in (port, ref):
        net = lib.net()
        i = net.add(ob.INPUT, 4)
        ce = net.add(ob.CROSSENT, 4, inputs=[i])
        net.forward()
        rec = [np.float32(net.loss(ce, 1)), np.int32(net.prediction(ce))]
        net.backward(1)
        rec += [net.plane(ce, p).copy() for p in range(2, 6)]
        out.append(rec)
    for a, b in zip(*out):
        _same(np.atleast_1d(a), np.atleast_1d(b), "zero-input CE")


def test_embedding(port, ref):
    dim, slots, vocab = 5, 4, 9
    rng = np.random.RandomState(3)
    table = rng.randn(2, vocab * dim).astype(np.float32)
    g = rng.randn(2, 2, slots * dim).astype(np.float32)
    out = []
    for lib in (port, ref):
        net = lib.net()
        e = net.add(ob.EMBEDDING, dim, slots, vocab)
        s1 = net.add(ob.L2OUT, slots * dim, inputs=[e])
        s2 = net.add(ob.L2OUT, slots * dim, inputs=[e])
        _fill(net, e, ob.RE, table[0])
        _fill(net, e, ob.IM, table[1])
        rec = []
        for toks in ([1, 3], [0], [2, 2, 2], [8, 2, 8, 0]):
            net.set_tokens(e, toks)
            net.node_forward(e)
            rec += [net.plane(s1, ob.RE).copy(), net.plane(s2, ob.IM).copy()]
            for k, s in enumerate((s1, s2)):
                _fill(net, s, ob.DZS_RE, g[k, 0])
                _fill(net, s, ob.DZS_IM, g[k, 1])
            net.node_backward(e)
            rec += [net.plane(e, ob.DZS_RE).copy(), net.plane(e, ob.DZS_IM).copy()]
        out.append(rec)
    for a, b in zip(*out):
        _same(a, b, "embedding")


def _mnist_like(lib, n, classes):
    """The README net: FourierTrans -> Hadamard(w) -> CGelu -> Linear(W) -> CrossEntropy."""
    net = lib.net()
    x = net.add(ob.INPUT, n)
    f = net.add(ob.FOURIER, n, inputs=[x])
    hw = net.add(ob.INPUT, n)
    h = net.add(ob.HADAMARD, n, inputs=[f, hw])
    g = net.add(ob.GELU, n, inputs=[h])
    lw = net.add(ob.INPUT, n * classes)
    lin = net.add(ob.LINEAR, n, n * classes, inputs=[g, lw])
    ce = net.add(ob.CROSSENT, classes, inputs=[lin])
    return net, dict(x=x, f=f, hw=hw, h=h, g=g, lw=lw, lin=lin, ce=ce)


@pytest.mark.parametrize("n", [16, 784])
def test_training_steps_readme_net(port, ref, n):
    """Three samples, update after the second (gradient accumulation across samples) and after the third."""
    classes = 10
    xs = port.uniform(7, (3, n))
    hw = port.normal(8, (2, n), 0.0, 0.05)
    lw = port.normal(9, (2, n * classes), 0.0, 1.0 / np.sqrt(n))
    labels = [3, 0, 9]
    out = []
    for lib in (port, ref):
        net, u = _mnist_like(lib, n, classes)
        _fill(net, u["hw"], ob.RE, hw[0]); _fill(net, u["hw"], ob.IM, hw[1])
        _fill(net, u["lw"], ob.RE, lw[0]); _fill(net, u["lw"], ob.IM, lw[1])
        rec = []
        for s in range(3):
            _fill(net, u["x"], ob.RE, xs[s]); _fill(net, u["x"], ob.IM, 0)
            net.forward()
            rec.append(np.float32(net.loss(u["ce"], labels[s])))
            rec.append(np.int32(net.prediction(u["ce"])))
            net.backward(labels[s])
            for name in ("f", "h", "g", "lin", "ce", "hw", "lw", "x"):
                rec += [net.plane(u[name], p).copy() for p in range(6)]
            if s >= 1:
                net.update(0.05, 1)
                rec += [net.plane(u[name], p).copy() for name in ("hw", "lw", "x") for p in range(6)]
        out.append(rec)
    for k, (a, b) in enumerate(zip(*out)):
        _same(np.atleast_1d(a), np.atleast_1d(b), "record %d" % k)


def test_residual_block_with_fanout(port, ref):
    """x feeds both a Linear and the Residual that closes the block (fan-out 2), L2Out on top."""
    n = 24
    x = port.normal(1, (2, n))
    w = port.normal(2, (2, n * n), 0, 1 / np.sqrt(n))
    out = []
    for lib in (port, ref):
        net = lib.net()
        xi = net.add(ob.INPUT, n)
        wi = net.add(ob.INPUT, n * n)
        sm = net.add(ob.SOFTMAX, n, inputs=[xi])
        lin = net.add(ob.LINEAR, n, n * n, inputs=[sm, wi])
        ge = net.add(ob.GELU, n, inputs=[lin])
        rs = net.add(ob.RESIDUAL, n, inputs=[sm, ge])
        l2 = net.add(ob.L2OUT, n, inputs=[rs])
        _fill(net, xi, ob.RE, x[0]); _fill(net, xi, ob.IM, x[1])
        _fill(net, wi, ob.RE, w[0]); _fill(net, wi, ob.IM, w[1])
        rec = []
        for step in range(2):
            net.forward()
            rec.append(np.float32(net.loss(l2, 0)))
            net.backward()
            for uid in (sm, lin, ge, rs, l2, xi, wi):
                rec += [net.plane(uid, p).copy() for p in range(6)]
            net.update(0.01, 1)
        out.append(rec)
    for k, (a, b) in enumerate(zip(*out)):
        _same(np.atleast_1d(a), np.atleast_1d(b), "record %d" % k)


def test_adam_steps_triang_crelu_net(port, ref):
    """x -> TriangFourier -> Hadamard(w) -> CRelu -> Linear(W) -> CrossEntropy, four Adam-style steps (t = 0..3) with
    the first moment carried in the inputs' dz planes (upstream tests/gputests.h:1377-1378 drives the same call)."""
    n, classes = 24, 5
    xs = port.uniform(17, (4, n))
    hw = port.normal(18, (2, n), 0.5, 0.3)
    lw = port.normal(19, (2, n * classes), 0.0, 1.0 / np.sqrt(n))
    labels = [3, 0, 4, 1]
    out = []
    for lib in (port, ref):
        net = lib.net()
        x = net.add(ob.INPUT, n)
        f = net.add(ob.TRIANG_FOURIER, n, inputs=[x])
        hwi = net.add(ob.INPUT, n)
        h = net.add(ob.HADAMARD, n, inputs=[f, hwi])
        r = net.add(ob.CRELU, n, inputs=[h])
        lwi = net.add(ob.INPUT, n * classes)
        lin = net.add(ob.LINEAR, n, n * classes, inputs=[r, lwi])
        ce = net.add(ob.CROSSENT, classes, inputs=[lin])
        _fill(net, hwi, ob.RE, hw[0]); _fill(net, hwi, ob.IM, hw[1])
        _fill(net, lwi, ob.RE, lw[0]); _fill(net, lwi, ob.IM, lw[1])
        rec = []
        for t in range(4):
            _fill(net, x, ob.RE, xs[t]); _fill(net, x, ob.IM, xs[(t + 1) % 4])
            net.forward()
            rec.append(np.float32(net.loss(ce, labels[t])))
            net.backward(labels[t])
            for uid in (f, h, r, lin):
                rec += [net.plane(uid, p).copy() for p in range(6)]
            net.adam_update(0.1, 2, 0.9, t)
            rec += [net.plane(uid, p).copy() for uid in (hwi, lwi, x) for p in range(6)]
        out.append(rec)
    assert any(np.any(a != 0) for a in out[0][-18:])
    for k, (a, b) in enumerate(zip(*out)):
        _same(np.atleast_1d(a), np.atleast_1d(b), "record %d" % k)


def test_generators(port, ref):
    for seed in (0, 1, 12345):
        _same(port.normal(seed, 1001, 0.5, 2.0), ref.normal(seed, 1001, 0.5, 2.0), "normal")
        _same(port.uniform(seed, 1001, -1, 3), ref.uniform(seed, 1001, -1, 3), "uniform")
