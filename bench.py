#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: isolated complex Linear, forward + Wirtinger backward.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = y = x W^T, then (dx, dx*) = (g W, g* conj W), then (dW, dW*) = (g^T x, g*^T conj x): 3 launches, 5 complex
GEMMs, 40*B*N*K real flops (8 per complex multiply-add, the 4-real-GEMM count).  Inputs are synthetic, seeded, and
resident in HBM before the timed region.  Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X published dense fp32 matrix peak
# Bytes the eight L2s exchanged with the fabric per launch (FETCH_SIZE + WRITE_SIZE of `rocprofv3 --pmc`, each scaled by
# what the same counter reads for a 256 MiB copy kernel); an upper bound on HBM traffic, since hits in the memory-side
# cache are included.  Counters cannot be read inside this run: the figures come from the committed summary of a counter
# run of this same command (`--counter-pass`), which names the commit it was measured at.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "cgemm_linear_b4096_1024x1024_traffic.txt")


def measured_traffic():
    """{launch: bytes} and the commit the counters were collected at, from profiles/ (None, None when absent)."""
    if not os.path.exists(TRAFFIC_FILE):
        return None, None
    table, at = {}, None
    for line in open(TRAFFIC_FILE):
        f = line.split()
        if len(f) >= 2 and f[0] == "measured_at":
            at = f[1]
        elif len(f) >= 2 and not line.startswith("#") and f[1].isdigit():
            table[f[0]] = int(f[1])
    return table, at


B, K, N = 4096, 1024, 1024      # the configuration the metric is quoted on: batched complex Linear, 4096 samples, 1024 -> 1024


class HipEvents:
    """hipEvent timing on the stream the library launches on."""

    def __init__(self, stream):
        self.hip = C.CDLL("libamdhip64.so")
        self.stream = C.c_void_p(stream)

    def event(self):
        e = C.c_void_p()
        rc = self.hip.hipEventCreate(C.byref(e))
        assert rc == 0, rc
        return e

    def record(self, e):
        rc = self.hip.hipEventRecord(e, self.stream)
        assert rc == 0, rc

    def elapsed_ms(self, a, b):
        rc = self.hip.hipEventSynchronize(b)
        assert rc == 0, rc
        ms = C.c_float()
        rc = self.hip.hipEventElapsedTime(C.byref(ms), a, b)
        assert rc == 0, rc
        return float(ms.value)


def cpu_baseline(budget_s=15.0):
    """Upstream CPU path (oracle/_ref, "reference") or the restatement ("port") timed on this host: per-sample
    forward + backward of the same Linear on a bounded number of batch rows (per-sample cost is constant: the CPU path
    processes one sample at a time), reported in the metric's unit."""
    from oracle import binding as ob
    lib = ob.load_ref() or ob.load_port()
    port = ob.load_port()
    net = lib.net()
    x = net.add(ob.INPUT, K)
    w = net.add(ob.INPUT, N * K)
    lin = net.add(ob.LINEAR, K, N * K, inputs=[x, w])
    sink = net.add(ob.L2OUT, N, inputs=[lin])
    net.plane(w, ob.RE)[:] = port.normal(3, N * K, 0, K ** -0.5)
    net.plane(w, ob.IM)[:] = port.normal(4, N * K, 0, K ** -0.5)
    rows_max = 256
    xs = port.normal(1, (2, rows_max, K))
    gs = port.normal(5, (4, rows_max, N))

    def one(r):
        net.plane(x, ob.RE)[:] = xs[0, r % rows_max]
        net.plane(x, ob.IM)[:] = xs[1, r % rows_max]
        net.forward()                    # zero non-input gradients, x and W into the layer, y = x W^T
        for p in range(4):
            net.plane(sink, ob.DZ_RE + p)[:] = gs[p, r % rows_max]
        net.node_backward(lin)           # dx, dx*, dW, dW* of this sample
        net.node_backward(w)             # parameter node gathers dW* across samples
        net.node_backward(x)

    for r in range(4):   # warm-up: page in the weight planes, start the thread pool
        one(r)
    rows, t0 = 0, time.perf_counter()
    while rows < B and (rows < 16 or time.perf_counter() - t0 < budget_s):   # a bounded sample of the batch, by time
        one(rows)
        rows += 1
    dt = time.perf_counter() - t0
    return {"value": round(40.0 * rows * N * K / dt / 1e12, 5), "unit": "TFLOP/s", "cores": lib.threads,
            "kind": lib.backend,
            "sample": "%d of %d batch rows, per-sample forward+backward as the upstream CPU loop, %.1f s, "
                      "%.2f ms/row (%.1f samples/s)" % (rows, B, dt, 1e3 * dt / rows, rows / dt)}


def kernel_suite(steps, rows=8192, parts=("mfma", "hbm", "ce")):
    """Per-kernel lines for the other rows of the hot path: the DFT-as-GEMM at config-3 shape (MFMA bound) and the
    elementwise / reduction kernels at config-4/5 shapes (HBM bound).  Bytes are the algorithmic (compulsory) traffic
    per complex element: every operand read once, every result written once, parameters amortised over the batch."""
    from cnet_amd import capi, ops
    capi.init(0)
    ev = HipEvents(capi.load().cnet_stream())
    rs = np.random.RandomState(0)
    rng = np.random.default_rng(0)

    def cmat(r, c):
        return ops.CMat.from_host(rng.standard_normal((r, c), dtype=np.float32), rng.standard_normal((r, c), dtype=np.float32))

    def grad(r, c):
        return ops.Grad.from_host([rng.standard_normal((r, c), dtype=np.float32) for _ in range(4)])

    def timed(fn, warm=3):
        # warm-up: groups of `warm` calls until two groups in a row agree to 2 % (at most 0.2 s): the device may have
        # gone idle while the host prepared the operands of this line, and comes back to its clocks over some 30 ms
        last, t0 = None, time.perf_counter()
        while time.perf_counter() - t0 < 0.2:
            a, b = ev.event(), ev.event()
            ev.record(a)
            for _ in range(warm):
                fn()
            ev.record(b)
            cur = ev.elapsed_ms(a, b)
            if last is not None and abs(cur - last) <= 0.02 * last:
                break
            last = cur
        capi.sync()
        a, b = ev.event(), ev.event()
        ev.record(a)
        for _ in range(steps):
            fn()
        ev.record(b)
        return ev.elapsed_ms(a, b) / steps

    lines = []

    def hbm(kid, name, shape, bytes_per_elem, elems, fn, extra_bytes=0):
        ms = timed(fn)
        gbs = (bytes_per_elem * elems + extra_bytes) / ms / 1e6
        lines.append({"id": kid, "kernel": name, "shape": shape, "ms": round(ms, 4), "roofline": {
            "bound": "hbm", "achieved": round(gbs, 1), "peak": 8000.0, "unit": "GB/s", "frac": round(gbs / 8000.0, 4),
            "bytes_per_complex_element": bytes_per_elem}})

    def mfma(kid, name, shape, flops, fn):
        ms = timed(fn, warm=20)  # millisecond launches: the clocks settle within a few of them
        tf = flops / ms / 1e9
        lines.append({"id": kid, "kernel": name, "shape": shape, "ms": round(ms, 4), "roofline": {
            "bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tf / PEAK_FP32_MFMA_TFLOPS, 4)}})

    if "mfma" in parts:
        dft_lines(mfma, cmat, grad, rs)
    if "hbm" in parts:
        hbm_lines(hbm, cmat, grad, rows)
    if "ce" in parts:
        ce_lines(hbm, cmat, rs)
    return lines


def dft_lines(mfma, cmat, grad, rs):
    from cnet_amd import ops
    # config 3: FourierTrans n = 4096, batch 1024 (3 complex GEMMs against the twiddle matrix)
    Bf, nf = 1024, 4096
    x, y, g, dx = cmat(Bf, nf), ops.CMat.empty(Bf, nf), grad(Bf, nf), ops.Grad.empty(Bf, nf)
    mfma("cdft_fwd", "cdft_fwd", [Bf, nf], 8.0 * Bf * nf * nf, lambda: ops.dft_fwd(x, y))
    mfma("cdft_bwd", "cdft_bwd", [Bf, nf], 16.0 * Bf * nf * nf, lambda: ops.dft_bwd(g, dx))
    xr = ops.CMat.from_host(rs.randn(Bf, nf).astype(np.float32), np.zeros((Bf, nf), np.float32))
    # an eighth of the full transform's flops: columns 0..n/2 only, two real products per complex one (the imaginary plane of
    # the samples is neither read nor multiplied), and the samples folded about n/2 first (cos is even, sin odd), which
    # halves the length of every sum: n/2 + 1 terms, rounded up to whole chunks of 16; the pass that folds forms column n/2
    # itself (n/2 is a multiple of 64 here), so the product has n/2 columns
    kp = (nf // 2 + 1 + 15) // 16 * 16
    mfma("cdft_fwd_real", "cdft_fwd of real samples (columns 0..n/2 by the product, the rest as conjugates; the samples folded about n/2, two real products over half the terms; flops executed, the pass that folds included in the time)",
         [Bf, nf], 4.0 * Bf * kp * (nf // 2), lambda: ops.dft_fwd_real_input(xr, y))
    del xr
    # TriangFourier: only the pairs in <= out contribute, n (n + 1) / 2 complex multiply-adds per row
    tri = nf * (nf + 1) / 2.0
    mfma("ctriang_fwd", "ctriang_dft_fwd (useful flops: upper triangle only)", [Bf, nf], 8.0 * Bf * tri, lambda: ops.triang_dft_fwd(x, y))
    mfma("ctriang_bwd", "ctriang_dft_bwd (useful flops: upper triangle only)", [Bf, nf], 16.0 * Bf * tri, lambda: ops.triang_dft_bwd(g, dx))
    del x, y, g, dx



def hbm_lines(hbm, cmat, grad, rows):
    from cnet_amd import capi, ops
    # config 5 activation shape [8192 x 4096]: 128 MiB per plane (config 4's [2048 x 2048] planes would sit in the 256 MB
    # memory-side cache and overstate the rate).  Even so a kernel that reads two planes of this size still finds part of them
    # in that cache from one call to the next; with rows = 32768 (512 MiB per plane) nothing is served by it.
    R, Cc = rows, 4096
    n = R * Cc
    u, v, w1 = cmat(R, Cc), cmat(R, Cc), cmat(1, Cc)
    yy, g, du, dv, dw1 = ops.CMat.empty(R, Cc), grad(R, Cc), ops.Grad.empty(R, Cc), ops.Grad.empty(R, Cc), ops.Grad.empty(1, Cc)
    hbm("copy", "plain copy of one plane (practical HBM ceiling)", [R, Cc], 8, n, lambda: ops.copy2d(u.re, yy.re))
    hbm("cgelu_fwd", "cgelu_fwd", [R, Cc], 16, n, lambda: ops.gelu_fwd(u, yy))
    hbm("cgelu_bwd", "cgelu_bwd", [R, Cc], 40, n, lambda: ops.gelu_bwd(u, g, du))
    # the same pass for a conjugate gradient pair (real loss): g.dz read, dx.dz written, the dz* halves neither read nor written
    hbm("cgelu_bwd_sym", "cgelu_bwd, conjugate pair (dz only)", [R, Cc], 24, n, lambda: ops.gelu_bwd_sym(u, g, du, mirror=False))
    hbm("crelu_fwd", "crelu_fwd", [R, Cc], 16, n, lambda: ops.crelu_fwd(u, yy))
    hbm("crelu_bwd", "crelu_bwd", [R, Cc], 40, n, lambda: ops.crelu_bwd(u, g, du))
    hbm("residual_fwd", "residual_fwd", [R, Cc], 24, n, lambda: ops.residual_fwd(u, v, yy))
    hbm("residual_bwd", "residual_bwd", [R, Cc], 48, n, lambda: ops.residual_bwd(g, du, dv))
    hbm("residual_bwd_sym", "residual_bwd, conjugate pair (dz only)", [R, Cc], 24, n, lambda: ops.residual_bwd_sym(g, du, dv, mirror=False))
    hbm("hadamard_fwd", "hadamard_fwd (shared weights)", [R, Cc], 16, n, lambda: ops.hadamard_fwd(u, w1, yy, True))
    hbm("hadamard_bwd", "hadamard_bwd (shared weights, batch-summed dW)", [R, Cc], 40, n, lambda: ops.hadamard_bwd(u, w1, g, du, dw1, True),
        extra_bytes=16 * Cc)
    hbm("hadamard_bwd_sym", "hadamard_bwd, conjugate pair (shared weights, dz only)", [R, Cc], 24, n,
        lambda: ops.hadamard_bwd_sym(u, w1, g, du, dw1, True, mirror=False), extra_bytes=8 * Cc)
    # fused pairs of layers: one pass where two were, the intermediate values written but not read back
    hbm("hadamard_cgelu_fwd", "hadamard + cgelu fwd, one pass (shared weights; h and gelu(h) written)", [R, Cc], 24, n,
        lambda: ops.hadamard_gelu_fwd(u, w1, yy, v, True), extra_bytes=8 * Cc)
    hbm("hadamard_cgelu_bwd_sym", "cgelu_bwd + hadamard_bwd, one pass, conjugate pair (shared weights, dz only, dh not kept)", [R, Cc], 24, n,
        lambda: ops.hadamard_gelu_bwd_sym(u, w1, g, None, du, dw1, True, mirror=False), extra_bytes=8 * Cc)
    hbm("residual_cgelu_bwd_sym", "residual_bwd (two consumers) + cgelu_bwd, one pass, conjugate pair (dz only)", [R, Cc], 40, n,
        lambda: ops.residual_gelu_bwd_sym(g, dv, u, du, None, ops.Grad([yy.re, yy.im, yy.re, yy.im]), mirror=False))
    loss = capi.empty(R)
    hbm("l2out_fwd", "l2out_fwd", [R, Cc], 8, n, lambda: ops.l2out_fwd(u, loss))
    hbm("l2out_bwd", "l2out_bwd", [R, Cc], 24, n, lambda: ops.l2out_bwd(u, du))
    hbm("l2out_bwd_sym", "l2out_bwd, conjugate pair (dz only)", [R, Cc], 16, n, lambda: ops.l2out_bwd_sym(u, du, mirror=False))
    s_ = capi.empty(R)
    hbm("l2norm_fwd", "l2norm_fwd (SoftMax)", [R, Cc], 16, n, lambda: ops.l2norm_fwd(u, yy, s_))
    hbm("l2norm_bwd", "l2norm_bwd (SoftMax)", [R, Cc], 40, n, lambda: ops.l2norm_bwd(u, s_, g, du))
    hbm("l2norm_bwd_sym", "l2norm_bwd (SoftMax), conjugate pair (dz only)", [R, Cc], 24, n, lambda: ops.l2norm_bwd_sym(u, s_, g, du, mirror=False))
    hbm("sgd_update", "sgd_update", [n], 32, n, lambda: ops.sgd_update(u, du.planes[2], du.planes[3], 1e-9))
    hbm("adam_update", "adam_update", [n], 48, n, lambda: ops.adam_update(u, du.planes[0], du.planes[1], du.planes[2], du.planes[3], 1e-9, 0.9, 3))
    hbm("zero4", "zero 4 gradient planes", [R, Cc], 16, n, lambda: [p.owner.zero() for p in du.planes])
    out1 = ops.Plane.empty(1, Cc)
    hbm("batch_sum", "batch_sum (one plane)", [R, Cc], 4, n, lambda: ops.batch_sum(u.re, out1))
    del u, v, yy, g, du, dv



def ce_lines(hbm, cmat, rs):
    from cnet_amd import capi, ops
    # config 5: CrossEntropy over 32768 logits (rows reduced from 8192 to 2048 to keep the suite short)
    R, Cc = 2048, 32768
    n = R * Cc
    z = cmat(R, Cc)
    labels = ops.ints(rs.randint(0, Cc, R))
    s_, l_, am = capi.empty(R), capi.empty(R), capi.empty(R, np.int32)
    dz = ops.Grad.empty(R, Cc)
    hbm("ce_fwd", "cross_entropy_fwd (loss, argmax; no normalised output)", [R, Cc], 8, n,
        lambda: ops.cross_entropy_fwd(z, labels, s_, l_, am, None), extra_bytes=4 * R)
    hbm("ce_bwd", "cross_entropy_bwd", [R, Cc], 24, n, lambda: ops.cross_entropy_bwd(z, s_, labels, dz))
    hbm("ce_bwd_sym", "cross_entropy_bwd, conjugate pair (dz only)", [R, Cc], 16, n, lambda: ops.cross_entropy_bwd_sym(z, s_, labels, dz, mirror=False))


def token_model_suite(steps, products=4):
    """Fifth configuration at full size: batch 16 x seq 512, vocab 32768, dim 1024, hidden 4096; forward + backward.
    products = 3: the block kernels form a complex product from three real ones (cnet_cgemm_set_products), conjugate
    gradient pairs only."""
    from cnet_amd import capi
    from cnet_amd.workloads import TokenModel
    capi.init(0)
    capi.call("cnet_cgemm_set_products", products)
    rng = np.random.default_rng(0)
    Bq, S, D, H, V = 16, 512, 1024, 4096, 32768

    def normal(shape, sig=1.0):
        return (sig * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)

    P = {"table": normal((2, V, D)), "gate": normal((2, D), 0.05), "w1": normal((2, H, D), D ** -0.5),
         "w2": normal((2, D, H), H ** -0.5), "w3": normal((2, V, D), D ** -0.5)}
    ids = rng.integers(0, V, (Bq, S)).astype(np.int32)
    ev = HipEvents(capi.load().cnet_stream())
    out = []
    # first with every product computed (what upstream's backward pass does), then with the dz* halves of the gradient
    # pairs written as conjugates of the dz products (the loss is real); one model at a time on the device
    for conjugate_pairs in ((False, True) if products == 4 else (True,)):
        model = TokenModel(Bq, S, D, H, V, P, conjugate_pairs=conjugate_pairs).set_tokens(ids)
        for _ in range(2):
            model.forward(); model.backward()
        capi.sync()
        a, b = ev.event(), ev.event()
        ev.record(a)
        for _ in range(steps):
            model.forward(); model.backward()
        ev.record(b)
        ms = ev.elapsed_ms(a, b) / steps
        loss = float(model.loss.download().mean())
        out.append({"workload": "configs[4]: complex token model fwd+bwd, batch 16 x seq 512, vocab 32768, dim 1024, hidden 4096",
                    "gradient_pairs": "dz* written as conj(dz)" if conjugate_pairs else "both halves computed",
                    "ms_per_step": round(ms, 3), "tokens_per_sec": round(Bq * S / ms * 1e3, 1),
                    "real_products_per_complex_product": products,
                    # complex products executed, each counted as 8 M N K
                    "gemm_tflops_executed": round(model.gemm_flops() / ms / 1e9, 2), "mean_loss": round(loss, 4),
                    "loss_of_uniform_guess": round(float(np.log(V)), 4)})
        del model
    capi.call("cnet_cgemm_set_products", 4)
    return out


TRAIN_BENCH = os.path.join(ROOT, "cnet_amd", "bin", "train_bench")
TOKEN_LR = 0.05


def _train_bench(*args, env=None):
    """One run of the C++ timing driver (cnet_amd/host/train_bench.cpp) in a process of its own; its JSON line or None."""
    import subprocess
    if not os.path.exists(TRAIN_BENCH):
        return None
    r = subprocess.run([TRAIN_BENCH] + [str(a) for a in args], capture_output=True, text=True, timeout=600,
                       env=dict(os.environ, **env) if env else None)
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    if r.returncode != 0 or not lines:
        sys.stderr.write("bench.py: train_bench %s failed:\n" % " ".join(map(str, args)) + r.stdout[-2000:] + r.stderr[-2000:])
        return None
    return json.loads(lines[-1])


def train_lines(steps):
    """Training steps (upload of the batch, forward, loss read-back, backward, SGD) of the FourierTrans -> Hadamard ->
    CGelu -> Linear -> CrossEntropy net on 784-long samples through the C++ facade; one dict per batch size with the
    time per step of each input mode.  None when the driver is not built or fails."""
    out = []
    for batch in (64, 1024, 4096):
        # the same number of samples at every batch size (a loop of 300 steps at batch 64 lasts 17 ms: too short to time)
        n = min(3000, steps * (4096 // batch))
        # "frozen_input" adds the mode in which the data input is marked not trainable (no step on it, no backward pass
        # into it; off by default in the facade, as upstream steps every input function)
        # "on_device" adds the loop whose reader keeps its samples in device memory (BatchedDataReader::storeOnDevice)
        line = _train_bench("readme", batch, n, "frozen_input", "on_device")
        if line is None:
            return None
        # two runs, both reported (`ms_per_step_runs`), the faster one kept as the figure: the loop at batch 4096 is bound by
        # the host's link, which other devices of the host share (one run in a dozen reads twice the time of the others)
        again = _train_bench("readme", batch, n, "frozen_input", "on_device")
        key = "ms_per_step_prefetch_loss_read_one_step_late"
        both_runs = [line[key]] + ([again[key]] if again is not None else [])
        if again is not None and again[key] < line[key]:
            line = again
        line["ms_per_step_runs"] = both_runs
        # configs[0] states real samples (imaginary parts 0), whose imaginary plane is cleared on the device instead of
        # sent; beside it the same loop on samples with uniform imaginary parts, both planes travelling
        both = _train_bench("readme", batch, n, "complex_samples")
        if both is not None:
            line["samples_per_sec_complex_samples"] = both["samples_per_sec_prefetch_loss_read_one_step_late"]
            line["upload_bytes_per_step_complex_samples"] = both["upload_bytes_per_step"]
        out.append(line)
    return out


STACK_LR = 3e-6   # configs[3] names 0.01, at which fp32 overflows in the first update on the CPU path as well; 1e-5 still diverges


def stack_lines(steps=10, products=4):
    """configs[3]: 8 x (Linear 2048 -> 2048, CGelu, Residual), L2Out, batch 2048, `steps` SGD steps through the C++ facade,
    both data inputs uploaded and the loss read back every step; first with the dz* halves of the gradient pairs written
    as conjugates (the facade's default), then with both halves computed as upstream does.  products = 3: the first of the
    two only, with the block kernels forming a complex product from three real ones (CNET_CGEMM_3M=1)."""
    out = []
    for mode in ((), ("both_halves",)) if products == 4 else ((),):
        line = _train_bench("stack", 2048, 8, 2048, steps, STACK_LR, *mode, env={"CNET_CGEMM_3M": "1" if products == 3 else "0"})
        if line is None:
            return None
        line["real_products_per_complex_product"] = products
        out.append(line)
    return out


def token_facade_lines(steps=5):
    """configs[4] through the C++ facade (one token per sample, SeqFourierTrans along the sequence): training steps, i.e.
    upload of tokens and labels, forward, backward, SGD on the table and every weight, mean loss read back; with one
    gradient per value (the facade's default) and with both halves of every pair."""
    out = []
    for mode in ((), ("both_halves",)):
        line = _train_bench("token", 16, 512, 1024, 4096, 32768, steps, TOKEN_LR, *mode)
        if line is None:
            return None
        out.append(line)
    return out


def train_suite(steps):
    lines = train_lines(steps)
    if lines is None:
        sys.exit("bench.py: cnet_amd/bin/train_bench is missing or failed; run __graft_entry__.build() first")
    for l in lines + (stack_lines() or []) + (token_facade_lines() or []):
        print(json.dumps(l))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--counter-pass", action="store_true",
                    help="short run for `rocprofv3 --pmc`: 3 launches of each GEMM kernel plus a plain copy kernel of "
                         "known size (256 MiB read, 256 MiB written) that calibrates FETCH_SIZE / WRITE_SIZE")
    ap.add_argument("--counter-launches", type=int, default=24,
                    help="with --counter-pass: launches in a row of each GEMM kernel after the three calibration rounds")
    ap.add_argument("--rows", type=int, default=8192,
                    help="with --suite kernels: rows of the [rows x 4096] planes the HBM-bound kernels run on (8192: 128 MiB per plane)")
    ap.add_argument("--products", type=int, choices=[3, 4], default=4,
                    help="real matrix products per complex one in the block kernels (cnet_cgemm_set_products) for the "
                         "headline step of this run; 4 is the library's default and what the driver's line is measured with")
    ap.add_argument("--suite", choices=["linear", "kernels", "token_model", "train"], default="linear",
                    help="linear (default): the headline line.  kernels: one line per other kernel of the hot path.  "
                         "token_model: configs[4] fwd+bwd.  train: training steps of the 784 -> 10 net of configs[0] "
                         "through the C++ facade, input pipeline included, at batch 64 and 4096")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (one process, one device, no collectives); --gpus %d is not "
                 "supported. Run with --gpus 1." % args.gpus)

    if args.suite == "kernels":
        for ln in kernel_suite(max(args.steps // 5, 10), rows=args.rows):
            print(json.dumps(ln))
        return
    if args.suite == "token_model":
        for ln in token_model_suite(max(args.steps // 20, 3)):
            print(json.dumps(ln), flush=True)
        return
    if args.suite == "train":
        train_suite(max(args.steps, 30))
        return

    from cnet_amd import capi, ops
    capi.init(0)
    capi.call("cnet_cgemm_set_products", args.products)
    info = capi.device_info()
    ev = HipEvents(capi.load().cnet_stream())
    try:
        import torch
        tsync = torch.cuda.synchronize if torch.cuda.is_available() else (lambda: None)
    except Exception:  # torch is only used for the contract's device-wide synchronize
        tsync = lambda: None

    rng = np.random.default_rng(0)

    def normal(shape, sig=1.0):
        return (sig * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)

    x = ops.CMat.from_host(normal((B, K)), normal((B, K)))
    w = ops.CMat.from_host(normal((N, K), K ** -0.5), normal((N, K), K ** -0.5))
    g = ops.Grad.from_host([normal((B, N)) for _ in range(4)])
    y, dx, dw = ops.CMat.empty(B, N), ops.Grad.empty(B, K), ops.Grad.empty(N, K)

    launches = {
        "linear_fwd": (lambda: ops.linear_fwd(x, w, y), 1),
        "linear_bwd_input": (lambda: ops.linear_bwd_input(g, w, dx), 2),
        "linear_bwd_weight": (lambda: ops.linear_bwd_weight(g, x, dw), 2),
    }

    def step():
        for fn, _ in launches.values():
            fn()

    if args.counter_pass:
        rows, cols = 8192, 8192   # 256 MiB per plane
        src, dst = ops.Plane.empty(rows, cols, zero=True), ops.Plane.empty(rows, cols, zero=True)
        for _ in range(3):
            ops.copy2d(src, dst)
            step()
        # then each launch `--counter-launches` times in a row: the collector reads its counters between dispatches, so a
        # lone dispatch starts on a drained device (cold caches, first wavefronts placed one by one); the median of a run of
        # equal dispatches is the kernel as the timed loop runs it
        for fn, _ in launches.values():
            for _ in range(args.counter_launches):
                fn()
        capi.sync()
        print(json.dumps({"counter_pass": True, "copy_bytes_read": rows * cols * 4, "copy_bytes_written": rows * cols * 4,
                          "launches_in_a_row": args.counter_launches}))
        return

    # no collector pauses inside the timed loops (one of 20 ms was seen to drain the queue in the middle of a loop)
    import gc
    gc.collect()
    gc.disable()
    # Out of idle first: a device that has just been handed over runs its first ~25 steps (30 ms) of this workload up to 25 %
    # slower while its clocks come up (1.45 -> 1.18 ms per step, measured step by step with events).  Groups of 10 steps are
    # run until two in a row agree to 1 % (at most 0.5 s in all); the W warm-up steps and the K timed steps follow.
    def settle(fn):
        done, last = 0, None
        t_pre = time.perf_counter()
        while time.perf_counter() - t_pre < 0.5:
            a, b = ev.event(), ev.event()
            ev.record(a)
            for _ in range(10):
                fn()
            ev.record(b)
            cur = ev.elapsed_ms(a, b)
            done += 10
            if last is not None and abs(cur - last) <= 0.01 * last:
                break
            last = cur
        return done

    preroll = settle(step)
    for _ in range(args.warmup):
        step()
    capi.sync(); tsync()
    e0, e1 = ev.event(), ev.event()
    t0 = time.perf_counter()
    ev.record(e0)
    for _ in range(args.steps):
        step()
    ev.record(e1)
    capi.sync(); tsync()
    wall = time.perf_counter() - t0
    gpu_ms = ev.elapsed_ms(e0, e1)
    ms_per_step = 1e3 * wall / args.steps
    flops_step = 40.0 * B * N * K
    tflops = flops_step / (wall / args.steps) / 1e12

    # per-launch durations (HIP events around back-to-back launches of one kernel on the library's stream)
    kern = {}
    for name, (fn, ngemm) in launches.items():
        fn(); capi.sync()
        groups = []   # five groups of K launches, the median group: one disturbed group does not decide the figure
        for _ in range(5):
            a, b = ev.event(), ev.event()
            ev.record(a)
            for _ in range(args.steps):
                fn()
            ev.record(b)
            groups.append(ev.elapsed_ms(a, b) / args.steps)
        ms = sorted(groups)[2]
        fl = 8.0 * B * N * K * ngemm
        kern[name] = {"ms": round(ms, 4), "flops": fl, "tflops": round(fl / ms / 1e9, 2)}
    gc.enable()
    dom = max(kern, key=lambda k: kern[k]["ms"])
    traffic_table, traffic_at = measured_traffic()
    traffic = traffic_table.get(dom) if traffic_table else None
    # achieved = the flops the kernel executes: 8 M N K per complex product with four real products (the metric's count),
    # three quarters of that with --products 3
    executed = args.products / 4.0
    roofline = {"bound": "mfma", "kernel": "cgemm_fast_kernel (%s)" % dom, "achieved": round(kern[dom]["tflops"] * executed, 2),
                "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": round(kern[dom]["tflops"] * executed / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": traffic if args.products == 4 else None,
                "traffic_measured_at": traffic_at,
                "flops_per_launch": kern[dom]["flops"], "avg_launch_ms": kern[dom]["ms"],
                "all_launches": kern, "device_clock_khz": info.clock_khz, "compute_units": info.compute_units}

    def conjugate_pair_step():
        # Beside the headline (all five products computed, whatever the gradient planes hold): the same layer step through the
        # entry points for a conjugate gradient pair (dz* = conj(dz), as under every real loss), which compute three products
        # and write the other two as conjugates.  Its rate counts the three products that are executed.
        gr, gi = normal((B, N)), normal((B, N))
        gc = ops.Grad.from_host([gr, gi, gr, -gi])

        def step_sym():
            ops.linear_fwd(x, w, y)
            ops.linear_bwd_input_sym(gc, w, dx)
            ops.linear_bwd_weight_sym(gc, x, dw)

        settle(step_sym)   # the host has just spent a while generating the pair: the device has gone idle
        for _ in range(args.warmup):
            step_sym()
        capi.sync()
        a, b = ev.event(), ev.event()
        ev.record(a)
        for _ in range(args.steps):
            step_sym()
        ev.record(b)
        sym_ms = ev.elapsed_ms(a, b) / args.steps
        conjugate_pair = {"ms_per_step": round(sym_ms, 4), "complex_products_executed": 3,
                          "tflops_executed": round(24.0 * B * N * K / sym_ms / 1e9, 2),
                          "samples_per_sec": round(B / sym_ms * 1e3, 1)}

        return conjugate_pair

    def three_products_step():
        # Beside the headline (four real matrix products per complex one, as the metric's 8 M N K counts them): the same five
        # products with the block kernels forming each from three real ones (cnet_cgemm_set_products(3): 6 M N K executed).
        capi.call("cnet_cgemm_set_products", 3)
        settle(step)
        for _ in range(args.warmup):
            step()
        capi.sync()
        a, b = ev.event(), ev.event()
        ev.record(a)
        for _ in range(args.steps):
            step()
        ev.record(b)
        ms3 = ev.elapsed_ms(a, b) / args.steps
        per = {}
        for name, (fn, ngemm) in launches.items():
            groups = []
            for _ in range(3):
                a, b = ev.event(), ev.event()
                ev.record(a)
                for _ in range(args.steps):
                    fn()
                ev.record(b)
                groups.append(ev.elapsed_ms(a, b) / args.steps)
            ms = sorted(groups)[1]
            per[name] = {"ms": round(ms, 4), "tflops_counted_as_8mnk": round(8.0 * B * N * K * ngemm / ms / 1e9, 2),
                         "tflops_executed": round(6.0 * B * N * K * ngemm / ms / 1e9, 2)}
        res = {"option": "cnet_cgemm_set_products(3) / CNET_CGEMM_3M=1; not the default",
               "ms_per_step": round(ms3, 4), "tflops_counted_as_8mnk": round(flops_step / ms3 / 1e9, 2),
               "tflops_executed": round(0.75 * flops_step / ms3 / 1e9, 2),
               "frac_of_fp32_mfma_peak_executed": round(0.75 * flops_step / ms3 / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
               "samples_per_sec": round(B / ms3 * 1e3, 1), "all_launches": per,
               "conjugate_gradient_pair": conjugate_pair_step()}
        capi.call("cnet_cgemm_set_products", 4)
        return res

    def sig(v, digits=3):
        """three significant digits: the line has to fit the 8 kB of output the driver's record keeps"""
        return float("%.*g" % (digits, v)) if isinstance(v, float) else v

    short = {"linear_fwd": "fwd", "linear_bwd_input": "bwd_input", "linear_bwd_weight": "bwd_weight"}
    roofline["launches"] = {short[k]: {"ms": v["ms"], "tflops": v["tflops"]} for k, v in roofline.pop("all_launches").items()}
    out = {
        "metric": "complex-Linear fwd+bwd TFLOP/s (% fp32 MFMA peak); train samples/sec",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "preroll_steps": preroll, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: isolated complex Linear fwd + Wirtinger bwd (dx, dx*, dW, dW*), "
                               "complex64 split-plane", "batch": B, "in": K, "out": N,
                   "flops_per_step": flops_step, "launches_per_step": 3, "real_products_per_complex_product": args.products},
        # of the flops executed (with --products 3: three quarters of the 8 M N K that `value` counts)
        "pct_fp32_mfma_peak": round(100 * tflops * executed / PEAK_FP32_MFMA_TFLOPS, 2),
        "samples_per_sec": round(B / (wall / args.steps), 1),
        "gpu_ms_per_step_events": round(gpu_ms / args.steps, 4),
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:   # the flag leaves the headline alone (profiled runs)
        # Everything below is rounded to three significant digits and keyed tersely; `python bench.py --suite kernels |
        # token_model | train` print the same measurements one verbose line each.
        pair = conjugate_pair_step()
        three = three_products_step()
        capi.call("cnet_cgemm_set_products", args.products)
        out["cpu_baseline"] = cpu_baseline()
        # the step through the entry points for a conjugate gradient pair: 3 complex products executed instead of 5
        out["conjugate_gradient_pair"] = {"ms": sig(pair["ms_per_step"]), "products": 3, "tflops_executed": sig(pair["tflops_executed"])}
        train = train_lines(300)
        if train:
            # The other half of the metric: training steps of the configs[0] net (FourierTrans 784, Hadamard, CGelu, Linear
            # 784 -> 10, CrossEntropy; SGD) through the C++ facade, upload of every batch and read-back of every loss included.
            # ms / sps: real samples fed from the host, the next batch travelling under the current step, each loss read one
            # step late; ms_runs: that figure in each of the two runs (the faster is reported); sps_wait: the host waits for
            # each loss before the next step; sps_sync: copy inside gpuForward; sps_dev: the reader's samples stored on the
            # device (a batch travels as indices); sps_cplx: complex samples (both planes travel); up_B: bytes sent per step
            out["train"] = [{"batch": t["batch"], "ms": sig(t["ms_per_step_prefetch_loss_read_one_step_late"]),
                             "ms_runs": [sig(v) for v in t["ms_per_step_runs"]],
                             "sps": sig(t["samples_per_sec_prefetch_loss_read_one_step_late"]),
                             "sps_wait": sig(t["samples_per_sec_prefetch"]),
                             "sps_sync": sig(t["samples_per_sec_copy_in_forward"]),
                             "sps_dev": sig(t.get("samples_per_sec_samples_stored_on_device")),
                             "sps_cplx": sig(t.get("samples_per_sec_complex_samples")),
                             "up_B": t.get("upload_bytes_per_step")} for t in train]
        # the other configurations and kernels of the hot path, each bounded to a few seconds
        del x, w, g, y, dx, dw

        def stack_brief(t):
            # configs[3] through the C++ facade: 10 SGD steps, data and targets uploaded and the loss read back every step
            return {"products_per_linear": t["complex_products_per_linear"], "ms": sig(t["ms_per_step"]),
                    "ms_after_first": sig(t["ms_per_step_after_the_first"]), "sps": sig(t["samples_per_sec"]),
                    "tflops_executed": sig(t["gemm_tflops_executed"]),
                    "loss_first_last": [sig(t["mean_loss_per_step"][0], 5), sig(t["mean_loss_per_step"][-1], 5)]}

        def token_brief(t):
            return {"pairs": "conj" if t["gradient_pairs"].startswith("dz*") else "both", "ms": sig(t["ms_per_step"]),
                    "tok_s": sig(t["tokens_per_sec"]), "tflops_executed": sig(t["gemm_tflops_executed"]), "loss": sig(t["mean_loss"], 5)}

        stack = stack_lines(10)
        if stack:
            out["configs3_residual_stack"] = {"batch": 2048, "lr": STACK_LR, "runs": [stack_brief(t) for t in stack]}
        # id: see kernel_suite; frac: of 157.3 TFLOP/s (cdft_*, ctriang_*: flops executed) or of 8 TB/s (algorithmic bytes)
        # frac4x: the same HBM-bound kernel on planes four times as large ([32768 x 4096], 512 MiB each): at [8192 x 4096] (the
        # activation shape of configs[4]) a kernel that reads two planes still finds part of them in the 256 MB memory-side cache
        # from one call to the next; at four times the size every byte comes from and goes to HBM
        big = {k["id"]: k["roofline"]["frac"] for k in kernel_suite(10, rows=32768, parts=("hbm",))}
        out["kernels"] = [dict({"id": k["id"], "ms": sig(k["ms"]), "frac": sig(k["roofline"]["frac"])},
                               **({"frac4x": sig(big[k["id"]])} if k["id"] in big else {})) for k in kernel_suite(20)]
        # api "c": forward + backward as a sequence of C-ABI calls; api "facade": training steps (SGD included) through the
        # C++ facade with one token per sample
        out["configs4_token_model"] = [dict(token_brief(t), api="c") for t in token_model_suite(3)]
        for t in token_facade_lines() or []:
            out["configs4_token_model"].append({"api": "facade", "pairs": "conj" if t["gradient_pairs"].startswith("dz*") else "both",
                                                "ms": sig(t["ms_per_step"]), "tok_s": sig(t["tokens_per_sec"]),
                                                "tflops_executed": sig(t["gemm_tflops_executed"]),
                                                "loss_first_last": [sig(t["mean_loss_per_step"][0], 5), sig(t["mean_loss_per_step"][-1], 5)]})
        # option, not the default: cnet_cgemm_set_products(3), three real products per complex one (6 M N K executed)
        three_brief = {"ms": sig(three["ms_per_step"]), "tflops_as_8mnk": sig(three["tflops_counted_as_8mnk"]),
                       "tflops_executed": sig(three["tflops_executed"]),
                       "launch_ms": {short[k]: sig(v["ms"]) for k, v in three["all_launches"].items()},
                       "conjugate_gradient_pair_ms": sig(three["conjugate_gradient_pair"]["ms_per_step"])}
        stack3 = stack_lines(10, products=3)
        if stack3:
            three_brief["configs3_residual_stack"] = stack_brief(stack3[0])
        three_brief["configs4_token_model"] = token_brief(token_model_suite(3, products=3)[0])
        out["three_real_products"] = three_brief
    line = json.dumps(out, separators=(",", ":"))
    if len(line) > 7000:
        sys.stderr.write("bench.py: the line is %d bytes long; the driver's record keeps 8 kB\n" % len(line))
    print(line)


if __name__ == "__main__":
    main()
