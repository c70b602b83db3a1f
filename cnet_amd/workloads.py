"""Multi-layer workloads of the benchmark configurations, expressed as sequences of C-ABI calls (orchestration only).

TokenModel is the complex token model of the fifth configuration: embedding -> DFT along the sequence axis -> Hadamard gate
with shared complex weights -> Linear, CGelu, Linear -> Linear to vocabulary logits -> CrossEntropy on the next token.
Upstream has no transform along an inner axis; its oracle is FourierTrans(seq) applied to every (sequence, channel) column.
Next-token labels: position t of a sequence is labelled with token t+1; the last position wraps to the first token.
"""
import ctypes as C

import numpy as np

from . import capi, ops


class TokenModel:
    def __init__(self, batch, seq, dim, hidden, vocab, params, conjugate_pairs=False):
        """params: dict of host arrays: table (2,V,D), gate (2,D), w1 (2,H,D), w2 (2,D,H), w3 (2,V,D).
        conjugate_pairs: the loss is real, so every dz* gradient is the conjugate of the dz gradient; the Linear backward
        passes then compute the dz products only and write the dz* halves as their conjugates, and of the sequence-axis
        transform only the dz* product is formed (its one consumer, the embedding table, gathers dz* alone)."""
        self.conjugate_pairs = conjugate_pairs
        self.B, self.S, self.D, self.H, self.V = batch, seq, dim, hidden, vocab
        self.rows = batch * seq
        p = {k: ops.CMat.from_host(v[0], v[1]) for k, v in params.items()}
        self.table, self.gate, self.w1, self.w2, self.w3 = p["table"], p["gate"], p["w1"], p["w2"], p["w3"]
        capi.call("cnet_cdft_plan", seq)
        fr, fi = C.c_void_p(), C.c_void_p()
        capi.call("cnet_cdft_twiddle", seq, C.byref(fr), C.byref(fi))
        ld = (seq + 3) // 4 * 4
        self.F = ops.CMat(ops.Plane(fr.value, seq, seq, ld), ops.Plane(fi.value, seq, seq, ld))
        R, D, H, V = self.rows, dim, hidden, vocab
        E = ops.CMat.empty
        G = ops.Grad.empty
        self.x, self.m, self.h = E(R, D), E(R, D), E(R, D)
        self.u, self.a, self.o, self.logits = E(R, H), E(R, H), E(R, D), E(R, V)
        self.s, self.loss, self.argmax = capi.empty(R), capi.empty(R), capi.empty(R, np.int32)
        self.d_logits, self.d_o, self.d_a, self.d_u = G(R, V), G(R, D), G(R, H), G(R, H)
        self.d_h, self.d_m, self.d_x = G(R, D), G(R, D), G(R, D)
        self.d_w1, self.d_w2, self.d_w3, self.d_gate = G(H, D), G(D, H), G(V, D), G(1, D)
        self.d_table_re, self.d_table_im = ops.Plane.empty(V, D), ops.Plane.empty(V, D)
        self.tokens = self.labels = None

    def set_tokens(self, ids):
        ids = np.ascontiguousarray(ids, np.int32).reshape(self.B, self.S)
        self.tokens = ops.ints(ids)
        self.labels = ops.ints(np.roll(ids, -1, axis=1).reshape(-1))
        return self

    def forward(self):
        B, S, D = self.B, self.S, self.D
        xb = ops.CMat(ops.Plane(self.x.re.ptr, B, S * D, S * D), ops.Plane(self.x.im.ptr, B, S * D, S * D))
        ops.embedding_fwd(self.table, self.tokens, xb, S)
        # M_b = F X_b for every sequence b: one strided-batched launch, F shared (stride 0)
        ops.cgemm_batched(self.F, 0, self.x, S * D, self.m, S * D, S, D, S, B, a_kmajor=0, b_kmajor=1)
        ops.hadamard_fwd(self.m, self.gate, self.h, shared=True)
        ops.linear_gelu_fwd(self.h, self.w1, self.u, self.a)   # the CGelu applied where the product is stored
        ops.linear_fwd(self.a, self.w2, self.o)
        ops.linear_fwd(self.o, self.w3, self.logits)
        ops.cross_entropy_fwd(self.logits, self.labels, self.s, self.loss, self.argmax, None)

    def backward(self):
        B, S, D = self.B, self.S, self.D
        if self.conjugate_pairs:
            # one gradient per value: every pass reads the dz planes only; the dz* planes are written where something reads
            # them (parameter gradients, and d_m, whose dz* half feeds the sequence transform)
            ops.cross_entropy_bwd_sym(self.logits, self.s, self.labels, self.d_logits, mirror=False)
            ops.linear_bwd_input_sym(self.d_logits, self.w3, self.d_o, mirror=False)
            ops.linear_bwd_weight_sym(self.d_logits, self.o, self.d_w3)
            ops.linear_bwd_input_sym(self.d_o, self.w2, self.d_a, mirror=False)
            ops.linear_bwd_weight_sym(self.d_o, self.a, self.d_w2)
            ops.gelu_bwd_sym(self.u, self.d_a, self.d_u, mirror=False)
            ops.linear_bwd_input_sym(self.d_u, self.w1, self.d_h, mirror=False)
            ops.linear_bwd_weight_sym(self.d_u, self.h, self.d_w1)
            ops.hadamard_bwd_sym(self.m, self.gate, self.d_h, self.d_m, self.d_gate, shared=True)
        else:
            ops.cross_entropy_bwd(self.logits, self.s, self.labels, self.d_logits)
            ops.linear_bwd_input(self.d_logits, self.w3, self.d_o)
            ops.linear_bwd_weight(self.d_logits, self.o, self.d_w3)
            ops.linear_bwd_input(self.d_o, self.w2, self.d_a)
            ops.linear_bwd_weight(self.d_o, self.a, self.d_w2)
            ops.gelu_bwd(self.u, self.d_a, self.d_u)
            ops.linear_bwd_input(self.d_u, self.w1, self.d_h)
            ops.linear_bwd_weight(self.d_u, self.h, self.d_w1)
            ops.hadamard_bwd(self.m, self.gate, self.d_h, self.d_m, self.d_gate, shared=True)
        # dz_b = F dM_b.dz ; dz*_b = conj(F) dM_b.dz*   (F symmetric)
        gdz = ops.CMat(self.d_m.planes[0], self.d_m.planes[1])
        gds = ops.CMat(self.d_m.planes[2], self.d_m.planes[3])
        xdz = ops.CMat(self.d_x.planes[0], self.d_x.planes[1])
        xds = ops.CMat(self.d_x.planes[2], self.d_x.planes[3])
        if not self.conjugate_pairs:
            ops.cgemm_batched(self.F, 0, gdz, S * D, xdz, S * D, S, D, S, B, b_kmajor=1)
        ops.cgemm_batched(self.F, 0, gds, S * D, xds, S * D, S, D, S, B, b_kmajor=1, conj_a=1)
        gs_re = ops.Plane(self.d_x.planes[2].ptr, B, S * D, S * D)
        gs_im = ops.Plane(self.d_x.planes[3].ptr, B, S * D, S * D)
        ops.embedding_bwd(self.tokens, gs_re, gs_im, self.d_table_re, self.d_table_im, D, self.V, B, S)

    def gemm_flops(self):
        R, S, D, H, V, B = self.rows, self.S, self.D, self.H, self.V, self.B
        lin = 8.0 * R * (D * H + H * D + D * V)
        dft = 8.0 * B * S * S * D
        return 3 * lin + 2 * dft if self.conjugate_pairs else 5 * lin + 3 * dft  # the products that are executed
