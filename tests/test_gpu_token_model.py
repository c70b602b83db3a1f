"""The complex token model of the fifth configuration at reduced size, forward and backward on the GPU against the CPU
oracle composed layer by layer (the sequence-axis transform = the oracle's FourierTrans applied to every column)."""
import numpy as np
import pytest

from cnet_amd import capi, ops
from cnet_amd.workloads import TokenModel
from tests.gpu_util import gpu, rel, rel_c, seeded, TOL  # noqa: F401

pytestmark = pytest.mark.gpu


def _seq_dft(port, xr, xi, B, S, D, backward_g4=None):
    """oracle transform along the sequence axis of [B*S, D] planes"""
    def cols(a):
        return np.ascontiguousarray(a.reshape(B, S, D).transpose(0, 2, 1).reshape(B * D, S))

    def rows(a):
        return np.ascontiguousarray(a.reshape(B, D, S).transpose(0, 2, 1).reshape(B * S, D))

    if backward_g4 is None:
        yr, yi = port.dft_fwd(cols(xr), cols(xi))
        return rows(yr), rows(yi)
    d = port.dft_bwd([cols(p) for p in backward_g4])
    return [rows(p) for p in d]


def test_strided_batched_gemm_with_conj_a(gpu, port):
    B, M, N, K = 5, 40, 24, 36
    A = seeded(port, 1, (M, K)) + 1j * seeded(port, 2, (M, K))
    X = seeded(port, 3, (B, K, N)) + 1j * seeded(port, 4, (B, K, N))
    a = ops.CMat.from_host(np.ascontiguousarray(A.real), np.ascontiguousarray(A.imag))
    x = ops.CMat.from_host(X.real.reshape(B * K, N), X.imag.reshape(B * K, N))
    for cj in (0, 1):
        c = ops.CMat.empty(B * M, N)
        ops.cgemm_batched(a, 0, x, K * N, c, M * N, M, N, K, B, b_kmajor=1, conj_a=cj)
        cr, ci = c.host()
        want = np.einsum("mk,bkn->bmn", A.conj() if cj else A, X).reshape(B * M, N)
        assert np.linalg.norm(cr + 1j * ci - want) / np.linalg.norm(want) < 1e-5


@pytest.mark.parametrize("conjugate_pairs", [False, True])
def test_token_model_reduced(gpu, port, conjugate_pairs):
    """conjugate_pairs: the Linear backward passes write the dz* halves as conjugates of the dz products, and of the
    sequence-axis transform only the dz* product is formed (the embedding table gathers dz* alone)."""
    B, S, D, H, V = 3, 32, 64, 128, 512
    R = B * S
    P = {"table": seeded(port, 1, (2, V, D)), "gate": seeded(port, 2, (2, D), 0.5),
         "w1": seeded(port, 3, (2, H, D), D ** -0.5), "w2": seeded(port, 4, (2, D, H), H ** -0.5),
         "w3": seeded(port, 5, (2, V, D), D ** -0.5)}
    ids = port.randint(6, (B, S), V)
    ids[1, 5] = ids[1, 9] = ids[0, 3]      # repeated tokens
    model = TokenModel(B, S, D, H, V, P, conjugate_pairs=conjugate_pairs).set_tokens(ids)
    model.forward()
    model.backward()

    # ---- oracle, layer by layer
    xr, xi = port.embedding_fwd(P["table"][0], P["table"][1], ids)
    xr, xi = xr.reshape(R, D), xi.reshape(R, D)
    mr, mi = _seq_dft(port, xr, xi, B, S, D)
    hr, hi = port.hadamard_fwd(mr, mi, P["gate"][0], P["gate"][1])
    ur, ui = port.linear_fwd(hr, hi, P["w1"][0], P["w1"][1])
    ar, ai = port.gelu_fwd(ur, ui)
    o_r, o_i = port.linear_fwd(ar, ai, P["w2"][0], P["w2"][1])
    lr_, li_ = port.linear_fwd(o_r, o_i, P["w3"][0], P["w3"][1])
    labels = np.roll(ids, -1, axis=1).reshape(-1).astype(np.int32)
    _, _, S_o, loss_o, pred_o = port.crossent_fwd(lr_, li_, labels)
    assert rel_c(model.logits.host(), (lr_, li_)) < TOL
    assert np.allclose(model.loss.download(), loss_o, rtol=2e-4, atol=2e-5)
    assert np.array_equal(model.argmax.download(), pred_o)

    g = port.crossent_bwd(lr_, li_, labels)
    d_o, d_w3 = port.linear_bwd(o_r, o_i, P["w3"][0], P["w3"][1], g)
    d_a, d_w2 = port.linear_bwd(ar, ai, P["w2"][0], P["w2"][1], d_o)
    d_u = port.gelu_bwd(ur, ui, d_a)
    d_h, d_w1 = port.linear_bwd(hr, hi, P["w1"][0], P["w1"][1], d_u)
    d_m, d_gate = port.hadamard_bwd(mr, mi, P["gate"][0], P["gate"][1], d_h)
    d_x = _seq_dft(port, None, None, B, S, D, backward_g4=d_m)
    dt_r, dt_i = port.embedding_bwd(V, D, ids, d_x[2].reshape(B, S * D), d_x[3].reshape(B, S * D))

    def chk(got, want, what, halves=(0, 2)):
        h = got.host()
        for k in halves:
            e = rel_c(h[k:k + 2], [w.reshape(h[k].shape) for w in want[k:k + 2]])
            assert e < TOL, (what, k, e)

    chk(model.d_logits, g, "d logits", halves=(0,) if conjugate_pairs else (0, 2))   # one gradient per value: dz only
    chk(model.d_w3, d_w3, "dW3")
    chk(model.d_w2, d_w2, "dW2")
    chk(model.d_w1, d_w1, "dW1")
    chk(model.d_gate, d_gate, "d gate")
    chk(model.d_m, d_m, "d seq-DFT output")
    chk(model.d_x, d_x, "d embedding rows", halves=(2,) if conjugate_pairs else (0, 2))
    assert rel_c((model.d_table_re.host(), model.d_table_im.host()), (dt_r, dt_i)) < TOL


@pytest.mark.parametrize("conjugate_pairs", [False, True])
def test_token_model_full_size_properties(gpu, port, conjugate_pairs):
    """The fifth configuration at its full size (16 x 512 tokens, vocab 32768, dim 1024, hidden 4096), checked through
    what does not need the CPU path on all of it: the oracle on a subsample of logit rows, bit-identical repetition,
    rows of a weight gradient against complex128 sums over the whole batch, and a directional finite difference of the
    total loss along the gradient of the shared gate weights.  Once with both halves of every gradient pair computed (as
    upstream does) and once with the one-gradient entry points, whose elementwise kernels stream at this size."""
    B, S, D, H, V = 16, 512, 1024, 4096, 32768
    rs = np.random.RandomState(5)

    def nrm(shape, sig):
        return (rs.standard_normal(shape) * sig).astype(np.float32)

    P = {"table": nrm((2, V, D), 1.0), "gate": nrm((2, D), 0.05), "w1": nrm((2, H, D), D ** -0.5),
         "w2": nrm((2, D, H), H ** -0.5), "w3": nrm((2, V, D), D ** -0.5)}
    ids = rs.randint(0, V, (B, S)).astype(np.int32)
    model = TokenModel(B, S, D, H, V, P, conjugate_pairs=conjugate_pairs).set_tokens(ids)
    model.forward()
    model.backward()
    loss0 = model.loss.download().copy()
    gate_grad = [p.copy() for p in model.d_gate.host()]
    assert np.all(np.isfinite(loss0)) and abs(loss0.mean() - np.log(V)) < 1.5

    # rows of the logits layer and of the loss against the oracle
    rows = [0, 511, 4097, 8191]
    o = model.o.host()
    labels = np.roll(ids, -1, axis=1).reshape(-1)[rows].astype(np.int32)
    lr_, li_ = port.linear_fwd(np.ascontiguousarray(o[0][rows]), np.ascontiguousarray(o[1][rows]), P["w3"][0], P["w3"][1])
    _, _, _, loss_o, pred_o = port.crossent_fwd(lr_, li_, labels)
    lg = model.logits.host()
    assert rel_c((lg[0][rows], lg[1][rows]), (lr_, li_)) < TOL / 5
    assert np.allclose(loss0[rows], loss_o, rtol=2e-4, atol=2e-5)
    assert np.array_equal(model.argmax.download()[rows], pred_o)
    del lg, o

    # rows of the first layer's weight gradient over the whole batch: dW[j] = sum_b G[b, j] x[b], dW*[j] = sum_b G*[b, j] conj(x[b])
    # (impl/linear.h:76-107 upstream); with one gradient per value the dz* planes of G are not written and G* = conj(G)
    picked = [0, 1, 2047, 4095]
    du, hh = model.d_u.host(), model.h.host()
    xh = hh[0].astype(np.float64) + 1j * hh[1]
    gz = du[0][:, picked].astype(np.float64) + 1j * du[1][:, picked]
    gs = np.conj(gz) if conjugate_pairs else du[2][:, picked].astype(np.float64) + 1j * du[3][:, picked]
    dw = model.d_w1.host()
    assert rel_c((dw[0][picked], dw[1][picked]), ((gz.T @ xh).real, (gz.T @ xh).imag)) < TOL / 10
    assert rel_c((dw[2][picked], dw[3][picked]), ((gs.T @ np.conj(xh)).real, (gs.T @ np.conj(xh)).imag)) < TOL / 10
    del du, hh, xh, dw

    # same bits on repetition
    model.forward()
    model.backward()
    assert np.array_equal(model.loss.download(), loss0)
    for a, b in zip(model.d_gate.host(), gate_grad):
        assert np.array_equal(a, b)

    # d(total loss) along the normalised dz* of the gate: 2 |dz*| (d/dRe = 2 Re dz*, d/dIm = 2 Im dz*)
    gs = gate_grad[2].astype(np.float64) + 1j * gate_grad[3].astype(np.float64)
    norm = np.linalg.norm(gs)
    direction = gs / norm
    eps = 5e-4  # the loss is strongly curved along this direction: 2e-3 already loses 6 %, 2e-2 loses 40 %
    totals = []
    for sign in (+1, -1):
        w = (P["gate"][0] + 1j * P["gate"][1]) + sign * eps * direction.reshape(-1)
        model.gate = ops.CMat.from_host(np.ascontiguousarray(w.real, np.float32), np.ascontiguousarray(w.imag, np.float32))
        model.forward()
        totals.append(model.loss.download().astype(np.float64).sum())
    numeric = (totals[0] - totals[1]) / (2 * eps)
    assert abs(numeric - 2 * norm) / (2 * norm) < 4e-2, (numeric, 2 * norm)
