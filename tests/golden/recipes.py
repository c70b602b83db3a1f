"""Seeded scenarios run against an oracle backend through the per-sample graph API.

`make_golden.py` runs them on the compiled upstream classes (oracle/_ref) and stores inputs + outputs in
`golden.npz`; `tests/test_oracle_golden.py` replays them on the restatement and compares.  Every scenario
returns a flat dict name -> ndarray.
"""
import numpy as np

from oracle import binding as ob

GRAD = (ob.DZ_RE, ob.DZ_IM, ob.DZS_RE, ob.DZS_IM)


def _rand(seed, *shape):
    return np.random.RandomState(seed).randn(*shape).astype(np.float32)


def _layer(lib, kind, params, in_sizes, out_size, seed, consumers=1):
    net = lib.net()
    ins = [net.add(ob.INPUT, s) for s in in_sizes]
    lay = net.add(kind, *params, inputs=ins)
    sinks = [net.add(ob.L2OUT, out_size, inputs=[lay]) for _ in range(consumers)]
    rec = {}
    for k, (uid, s) in enumerate(zip(ins, in_sizes)):
        re, im = _rand(seed + 10 * k, s), _rand(seed + 10 * k + 1, s)
        rec["in%d_re" % k], rec["in%d_im" % k] = re, im
        net.plane(uid, ob.RE)[:] = re
        net.plane(uid, ob.IM)[:] = im
        net.node_forward(uid)
    net.node_forward(lay)
    rec["out_re"], rec["out_im"] = net.plane(sinks[0], ob.RE).copy(), net.plane(sinks[0], ob.IM).copy()
    for c, s in enumerate(sinks):
        for p in GRAD:
            g = _rand(seed + 100 + 10 * c + p, out_size)
            rec["g%d_%d" % (c, p)] = g
            net.plane(s, p)[:] = g
    net.node_backward(lay)
    for p in GRAD:
        rec["grad_%d" % p] = net.plane(lay, p).copy()
    return rec


def linear(lib):
    return _layer(lib, ob.LINEAR, (24, 24 * 7), [24, 24 * 7], 7, seed=1)


def linear_fanout(lib):
    return _layer(lib, ob.LINEAR, (5, 5 * 3), [5, 5 * 3], 3, seed=2, consumers=2)


def fourier_pow2(lib):
    return _layer(lib, ob.FOURIER, (64,), [64], 64, seed=3)


def fourier_784(lib):
    return _layer(lib, ob.FOURIER, (784,), [784], 784, seed=4)


def fourier_12(lib):
    return _layer(lib, ob.FOURIER, (12,), [12], 12, seed=5)


def hadamard(lib):
    return _layer(lib, ob.HADAMARD, (33,), [33, 33], 33, seed=6)


def gelu(lib):
    return _layer(lib, ob.GELU, (257,), [257], 257, seed=7)


def residual(lib):
    return _layer(lib, ob.RESIDUAL, (9,), [9, 9], 9, seed=8, consumers=2)


def crelu(lib):
    return _layer(lib, ob.CRELU, (129,), [129], 129, seed=21, consumers=2)


def triang_fourier(lib):
    return _layer(lib, ob.TRIANG_FOURIER, (50,), [50], 50, seed=22)


def adam_training(lib, n=20, classes=4, steps=4):
    """TriangFourier -> Hadamard(w) -> CRelu -> Linear(W) -> CrossEntropy with the Adam-style step, t = 0..steps-1."""
    net = lib.net()
    x = net.add(ob.INPUT, n)
    f = net.add(ob.TRIANG_FOURIER, n, inputs=[x])
    hw = net.add(ob.INPUT, n)
    h = net.add(ob.HADAMARD, n, inputs=[f, hw])
    r = net.add(ob.CRELU, n, inputs=[h])
    lw = net.add(ob.INPUT, n * classes)
    lin = net.add(ob.LINEAR, n, n * classes, inputs=[r, lw])
    ce = net.add(ob.CROSSENT, classes, inputs=[lin])
    rec = dict(hw0=_rand(31, 2, n) * 0.3 + 0.5, lw0=_rand(32, 2, n * classes) / np.float32(np.sqrt(n)), xs=_rand(33, steps, 2, n),
               labels=np.arange(steps, dtype=np.int32) % classes)
    rec["hw0"] = rec["hw0"].astype(np.float32)
    net.plane(hw, ob.RE)[:] = rec["hw0"][0]; net.plane(hw, ob.IM)[:] = rec["hw0"][1]
    net.plane(lw, ob.RE)[:] = rec["lw0"][0]; net.plane(lw, ob.IM)[:] = rec["lw0"][1]
    for t in range(steps):
        net.plane(x, ob.RE)[:] = rec["xs"][t, 0]; net.plane(x, ob.IM)[:] = rec["xs"][t, 1]
        net.forward()
        rec["loss%d" % t] = np.float32(net.loss(ce, int(rec["labels"][t])))
        net.backward(int(rec["labels"][t]))
        net.adam_update(0.05, 1, 0.9, t)
        for name, uid in (("hw", hw), ("lw", lw)):
            rec["%s_step%d" % (name, t)] = np.stack([net.plane(uid, p).copy() for p in range(4)])
    return rec


def softmax(lib):
    return _layer(lib, ob.SOFTMAX, (31,), [31], 31, seed=9)


def fourier_rows_4096(lib):
    """Rows of the CPU forward operator at n=4096: images of e_1, e_5, e_4095 and of one random vector."""
    n = 4096
    net = lib.net()
    x = net.add(ob.INPUT, n)
    f = net.add(ob.FOURIER, n, inputs=[x])
    s = net.add(ob.L2OUT, n, inputs=[f])
    rec = {}
    for q in (1, 5, 4095):
        net.plane(x, ob.RE)[:] = 0
        net.plane(x, ob.IM)[:] = 0
        net.plane(x, ob.RE)[q] = 1
        net.node_forward(x)
        net.node_forward(f)
        rec["e%d_re" % q], rec["e%d_im" % q] = net.plane(s, ob.RE).copy(), net.plane(s, ob.IM).copy()
    re, im = _rand(40, n), _rand(41, n)
    rec["x_re"], rec["x_im"] = re, im
    net.plane(x, ob.RE)[:] = re
    net.plane(x, ob.IM)[:] = im
    net.node_forward(x)
    net.node_forward(f)
    rec["y_re"], rec["y_im"] = net.plane(s, ob.RE).copy(), net.plane(s, ob.IM).copy()
    return rec


def losses(lib):
    n = 10
    net = lib.net()
    i = net.add(ob.INPUT, n)
    ce = net.add(ob.CROSSENT, n, inputs=[i])
    j = net.add(ob.INPUT, n)
    l2 = net.add(ob.L2OUT, n, inputs=[j])
    rec = {}
    for t, label in enumerate((0, 7, 3)):
        re, im = _rand(50 + t, n), _rand(60 + t, n)
        if t == 2:
            re[3] = im[3] = 0  # label on an exactly-zero logit: both clamps
        rec["z%d_re" % t], rec["z%d_im" % t] = re, im
        for u in (i, j):
            net.plane(u, ob.RE)[:] = re
            net.plane(u, ob.IM)[:] = im
        net.forward()
        rec["ce%d_out_re" % t] = net.plane(ce, ob.OUT_RE).copy()
        rec["ce%d_out_im" % t] = net.plane(ce, ob.OUT_IM).copy()
        rec["ce%d_loss" % t] = np.float32(net.loss(ce, label))
        rec["ce%d_pred" % t] = np.int32(net.prediction(ce))
        rec["l2%d_loss" % t] = np.float32(net.loss(l2, 0))
        net.backward(label)
        for p in GRAD:
            rec["ce%d_grad_%d" % (t, p)] = net.plane(ce, p).copy()
            rec["l2%d_grad_%d" % (t, p)] = net.plane(l2, p).copy()
    return rec


def readme_net_training(lib, n=100, classes=10, steps=4):
    """FourierTrans -> Hadamard(w) -> CGelu -> Linear(W) -> CrossEntropy (the README net, upstream README.md:19-30),
    per-sample SGD with an update every second sample: pins accumulation across samples and the step on the
    data input."""
    net = lib.net()
    x = net.add(ob.INPUT, n)
    f = net.add(ob.FOURIER, n, inputs=[x])
    hw = net.add(ob.INPUT, n)
    h = net.add(ob.HADAMARD, n, inputs=[f, hw])
    g = net.add(ob.GELU, n, inputs=[h])
    lw = net.add(ob.INPUT, n * classes)
    lin = net.add(ob.LINEAR, n, n * classes, inputs=[g, lw])
    ce = net.add(ob.CROSSENT, classes, inputs=[lin])
    rs = np.random.RandomState(123)
    xs = rs.rand(steps, n).astype(np.float32)
    w_h = (rs.randn(2, n) * 0.05).astype(np.float32)
    w_l = (rs.randn(2, n * classes) / np.sqrt(n)).astype(np.float32)
    labels = rs.randint(0, classes, steps).astype(np.int32)
    rec = dict(xs=xs, w_h=w_h, w_l=w_l, labels=labels)
    net.plane(hw, ob.RE)[:] = w_h[0]
    net.plane(hw, ob.IM)[:] = w_h[1]
    net.plane(lw, ob.RE)[:] = w_l[0]
    net.plane(lw, ob.IM)[:] = w_l[1]
    for s in range(steps):
        net.plane(x, ob.RE)[:] = xs[s]
        net.plane(x, ob.IM)[:] = 0
        net.forward()
        rec["loss%d" % s] = np.float32(net.loss(ce, int(labels[s])))
        rec["pred%d" % s] = np.int32(net.prediction(ce))
        net.backward(int(labels[s]))
        rec["lin_in%d" % s] = np.stack([net.plane(lin, p)[:n].copy() for p in range(6)])
        rec["x_dzs%d" % s] = np.stack([net.plane(x, ob.DZS_RE).copy(), net.plane(x, ob.DZS_IM).copy()])
        rec["hw_dzs%d" % s] = np.stack([net.plane(hw, ob.DZS_RE).copy(), net.plane(hw, ob.DZS_IM).copy()])
        if s % 2 == 1:
            net.update(0.05, 1)
            rec["hw_after%d" % s] = np.stack([net.plane(hw, ob.RE).copy(), net.plane(hw, ob.IM).copy()])
            rec["lw_after%d" % s] = np.stack([net.plane(lw, ob.RE).copy(), net.plane(lw, ob.IM).copy()])
            rec["x_after%d" % s] = np.stack([net.plane(x, ob.RE).copy(), net.plane(x, ob.IM).copy()])
    return rec


def residual_block_training(lib, n=16, steps=3):
    """Linear -> CGelu -> Residual(x, .) -> L2Out with fan-out on x; label-free backward; SGD on W and x."""
    net = lib.net()
    x = net.add(ob.INPUT, n)
    w = net.add(ob.INPUT, n * n)
    lin = net.add(ob.LINEAR, n, n * n, inputs=[x, w])
    ge = net.add(ob.GELU, n, inputs=[lin])
    rs_ = net.add(ob.RESIDUAL, n, inputs=[x, ge])
    l2 = net.add(ob.L2OUT, n, inputs=[rs_])
    r = np.random.RandomState(77)
    x0 = r.randn(2, n).astype(np.float32)
    w0 = (r.randn(2, n * n) / np.sqrt(n)).astype(np.float32)
    rec = dict(x0=x0, w0=w0)
    net.plane(x, ob.RE)[:] = x0[0]
    net.plane(x, ob.IM)[:] = x0[1]
    net.plane(w, ob.RE)[:] = w0[0]
    net.plane(w, ob.IM)[:] = w0[1]
    for s in range(steps):
        net.forward()
        rec["loss%d" % s] = np.float32(net.loss(l2, 0))
        net.backward()
        rec["lin%d" % s] = np.stack([net.plane(lin, p)[:n].copy() for p in range(6)])
        rec["x_dzs%d" % s] = np.stack([net.plane(x, ob.DZS_RE).copy(), net.plane(x, ob.DZS_IM).copy()])
        net.update(0.01, 1)
        rec["w_after%d" % s] = np.stack([net.plane(w, ob.RE).copy(), net.plane(w, ob.IM).copy()])
    return rec


def embedding(lib):
    dim, slots, vocab = 4, 3, 6
    net = lib.net()
    e = net.add(ob.EMBEDDING, dim, slots, vocab)
    s1 = net.add(ob.L2OUT, slots * dim, inputs=[e])
    s2 = net.add(ob.L2OUT, slots * dim, inputs=[e])
    table = _rand(90, 2, vocab * dim)
    rec = dict(table=table)
    net.plane(e, ob.RE)[:] = table[0]
    net.plane(e, ob.IM)[:] = table[1]
    for t, toks in enumerate(([1, 3], [0], [2, 2, 2], [5, 2, 5])):
        net.set_tokens(e, toks)
        net.node_forward(e)
        rec["out%d" % t] = np.stack([net.plane(s1, ob.RE).copy(), net.plane(s1, ob.IM).copy()])
        for c, s in enumerate((s1, s2)):
            g = _rand(91 + 2 * t + c, 2, slots * dim)
            rec["g%d_%d" % (t, c)] = g
            net.plane(s, ob.DZS_RE)[:] = g[0]
            net.plane(s, ob.DZS_IM)[:] = g[1]
        net.node_backward(e)
        rec["dzs%d" % t] = np.stack([net.plane(e, ob.DZS_RE).copy(), net.plane(e, ob.DZS_IM).copy()])
    return rec


def _mod_readme_net(lib, n=100, classes=10):
    net = lib.net()
    x = net.add(ob.INPUT, n)
    f = net.add(ob.FOURIER, n, inputs=[x])
    hw = net.add(ob.INPUT, n)
    h = net.add(ob.HADAMARD, n, inputs=[f, hw])
    g = net.add(ob.GELU, n, inputs=[h])
    lw = net.add(ob.INPUT, n * classes)
    lin = net.add(ob.LINEAR, n, n * classes, inputs=[g, lw])
    ce = net.add(ob.CROSSENT, classes, inputs=[lin])
    net.plane(hw, ob.RE)[:] = _rand(41, n) * 0.3 + 1; net.plane(hw, ob.IM)[:] = _rand(42, n) * 0.3
    net.plane(lw, ob.RE)[:] = _rand(43, n * classes) * 0.1; net.plane(lw, ob.IM)[:] = _rand(44, n * classes) * 0.1
    return net, x, ce


def _mod_token_net(lib, dim=4, slots=6, vocab=19):
    """Every remaining function kind in one graph: embedding + positional input -> Residual -> TriangFourier -> Linear ->
    Residual -> SoftMax -> CRelu -> Hadamard -> logits Linear -> CrossEntropy, with an L2Out side branch."""
    size = dim * slots
    net = lib.net()
    emb = net.add(ob.EMBEDDING, dim, slots, vocab)
    pos = net.add(ob.INPUT, size)
    r0 = net.add(ob.RESIDUAL, size, inputs=[emb, pos])
    tf = net.add(ob.TRIANG_FOURIER, size, inputs=[r0])
    w1 = net.add(ob.INPUT, size * size)
    l1 = net.add(ob.LINEAR, size, size * size, inputs=[tf, w1])
    r1 = net.add(ob.RESIDUAL, size, inputs=[tf, l1])
    sm = net.add(ob.SOFTMAX, size, inputs=[r1])
    cr = net.add(ob.CRELU, size, inputs=[sm])
    hd = net.add(ob.INPUT, size)
    h = net.add(ob.HADAMARD, size, inputs=[cr, hd])
    w2 = net.add(ob.INPUT, size * vocab)
    l2 = net.add(ob.LINEAR, size, size * vocab, inputs=[h, w2])
    ce = net.add(ob.CROSSENT, vocab, inputs=[l2])
    side = net.add(ob.L2OUT, size, inputs=[sm])
    for k, uid in enumerate((emb, pos, w1, hd, w2)):
        n = net.plane(uid, ob.RE).size
        net.plane(uid, ob.RE)[:] = _rand(50 + 2 * k, n) * 0.5 + 0.3
        net.plane(uid, ob.IM)[:] = _rand(51 + 2 * k, n) * 0.5 + 0.3
    return net, emb, ce, side


def model_files(lib):
    """.mod streams as the backend writes them, and what a net restored from each computes on seeded inputs."""
    rec = {}
    net, x, ce = _mod_readme_net(lib)
    blob = net.save()
    rec["readme_mod"] = np.frombuffer(blob, np.uint8).copy()
    back = lib.net()
    assert back.restore(blob)
    rec["readme_uids"] = np.asarray(back.uids(), np.int32)
    rec["readme_x"] = np.abs(_rand(45, 3, 100))
    for k in range(3):
        back.plane(x, ob.RE)[:] = rec["readme_x"][k]; back.plane(x, ob.IM)[:] = 0
        back.forward()
        rec["readme_out%d" % k] = np.stack([back.plane(ce, ob.OUT_RE).copy(), back.plane(ce, ob.OUT_IM).copy()])
        rec["readme_loss%d" % k] = np.float32(back.loss(ce, k))
        rec["readme_pred%d" % k] = np.int32(back.prediction(ce))
    net, emb, ce, side = _mod_token_net(lib)
    blob = net.save()
    rec["token_mod"] = np.frombuffer(blob, np.uint8).copy()
    back = lib.net()
    assert back.restore(blob)
    rec["token_uids"] = np.asarray(back.uids(), np.int32)
    rec["token_tokens"] = np.asarray([[3, 18, 0, 7, 7, 2], [5, 1, 4, -1, -1, -1]], np.int32)
    for k in range(2):
        row = rec["token_tokens"][k]
        back.set_tokens(emb, row[row >= 0])
        back.forward()
        rec["token_out%d" % k] = np.stack([back.plane(ce, ob.OUT_RE).copy(), back.plane(ce, ob.OUT_IM).copy()])
        rec["token_l2_%d" % k] = np.float32(back.loss(side, 0))
        back.backward(int(row[0]))
        rec["token_table_dzs%d" % k] = np.stack([back.plane(emb, ob.DZS_RE).copy(), back.plane(emb, ob.DZS_IM).copy()])
    return rec


def generators(lib):
    return dict(normal=lib.normal(2024, 257, 0.0, 1.0), uniform=lib.uniform(2024, 257, 0.0, 1.0))


SCENARIOS = [linear, linear_fanout, fourier_pow2, fourier_784, fourier_12, hadamard, gelu, residual, softmax, crelu,
             triang_fourier, adam_training, model_files,
             fourier_rows_4096, losses, readme_net_training, residual_block_training, embedding, generators]
