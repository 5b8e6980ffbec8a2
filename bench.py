#!/usr/bin/env python
"""Benchmark of the quantization hot path on one MI355X.

One "step" is one BinaryWeightAffine forward at the headline shape (x [4096, 4096], W [4096, 11008]):
sign/alpha/pack of W, the int8 digit operand of x and the 1-bit-weight int8 MFMA product, launched through the C-ABI on
torch's current HIP stream with all inputs already resident in HBM.  The JSON line also carries the quantizer
kernels' HBM figures (`quantizers`) and the small-M sweep (`sweep`).

  value      whole-step fp32-equivalent TFLOP/s  (2*M*K*N / step time), K steps between two synchronisations
  roofline   the dominant kernel (the MFMA product), timed with HIP events around its launches in a repeat of the
             K steps (the event records are queue work of their own and stay out of the timed steps).  Its arithmetic
             is three int8 digit planes per fp32 activation, so `achieved` counts the int8 operations it issues
             (3 x 2MKN) against the int8 MFMA peak; the fp32-equivalent rate (2MKN) is given beside it
  cpu_baseline  the CPU oracle (a port of nnabla's CPU arithmetic, 1 core) on a bounded row sample
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # MI355X dense fp32 matrix
PEAK_INT8_MFMA_TOPS = 5000.0    # MI355X dense int8 matrix
PEAK_HBM_GBS = 8000.0           # MI355X HBM3E
HEADLINE_PROFILE = os.path.join(ROOT, "profiles", "binary_weight_affine_4096x4096x11008.md")
KERNEL_SOURCES = ("gemm_bits.hip", "gemm_layout.hpp")


def kernel_source_sha():
    """sha256 over the sources of the dominant kernel: what a committed profile is stamped with."""
    import hashlib
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "nnabla_amd", "csrc", "kernels", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def profiled_traffic():
    """HBM-side bytes of one launch of the dominant kernel, read from the committed rocprofv3 summary (its line
    `traffic: fetch_bytes=... write_bytes=... source_sha=...`, FETCH_SIZE / WRITE_SIZE scaled by what a streaming kernel
    of known size reads on those counters).  Only reported while the kernel's sources are the ones that were profiled."""
    import re
    try:
        text = open(HEADLINE_PROFILE).read()
    except OSError:
        return None, "no committed profile"
    m = re.search(r"traffic: fetch_bytes=([0-9.e+]+) write_bytes=([0-9.e+]+) source_sha=([0-9a-f]+)", text)
    if not m:
        return None, "the committed profile carries no traffic line"
    if m.group(3) != kernel_source_sha():
        return None, "kernel sources changed since the committed profile (%s): traffic not carried over" % m.group(3)
    return float(m.group(1)) + float(m.group(2)), ("bytes per launch between L2 and the memory side: %.1f MB fetched + "
                                                   "%.1f MB written, rocprofv3 counters of the profile under profiles/ "
                                                   "taken on these kernel sources (%s); algorithmic: 56.2 MB read + "
                                                   "180.4 MB written" % (float(m.group(1)) / 1e6,
                                                                         float(m.group(2)) / 1e6, m.group(3)))


def bench_mfma_rates(dev):
    """What the matrix pipes sustain on kernels of nothing but independent matrix instructions with non-zero operands
    (two blocks of four wavefronts per CU, about a millisecond per launch so that the clocks settle under the power
    limit): the int8 instruction of the products, and the fp6 x fp4 / fp8 x fp8 forms of the scaled instruction.  An
    exact fp32-faithful product on fp6 digits would need five balanced base-32 digits where int8 needs three base-256
    ones, so fp6 x fp4 has to issue more than 5/3 as many operations per second as int8 to pay."""
    import torch
    from nnabla_amd import kernels as k
    sink = torch.zeros(64, device=dev)
    out = {}
    for kind, rounds in (("i8", 4000), ("fp6 x fp4", 4000), ("fp8 x fp8", 4000), ("i8, operands change", 4000),
                         ("i8, digits x bit bytes, operands change", 4000)):
        n, ops = k.mfma_rate_probe(kind, rounds, sink)
        ms = time_kernel(lambda: k.mfma_rate_probe(kind, rounds, sink), 10)
        out[kind] = {"ms": ms, "instructions": n, "ops_per_instruction": ops, "POPs": n * ops / ms / 1e12}
    out["fp6 x fp4 over i8"] = out["fp6 x fp4"]["POPs"] / out["i8"]["POPs"]
    out["needed for five fp6 digits against three int8 digits"] = 5.0 / 3.0
    return out


def _events(n):
    import torch
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def bench_binary_weight_affine(M, K, N, steps, warmup, dev, time_product=True):
    import torch
    from nnabla_amd import kernels as k
    # drawn on the device: host-side generation of 60 M values would leave the GPU idle for seconds right before the
    # timed steps, and the first launches after idle run on ramping clocks
    g = torch.Generator(device=dev).manual_seed(313)
    x = torch.randn(M, K, generator=g, device=dev)
    W = torch.randn(K, N, generator=g, device=dev) * 0.02
    Wb = torch.empty_like(W)
    alpha = torch.empty(N, device=dev)
    y = torch.empty(M, N, device=dev)
    L = k.lib()
    bits = torch.empty(L.nbla_hip_packed_bits_bytes(k._i64(K), k._i64(N)), dtype=torch.uint8, device=dev)
    xs = torch.empty(L.nbla_hip_digit_operand_bytes(k._i64(M), k._i64(K)), dtype=torch.uint8, device=dev)
    pws = torch.empty(max(256, L.nbla_hip_binarize_workspace_bytes(k._i64(K), k._i64(N))), dtype=torch.uint8,
                      device=dev)
    st = k._stream(None)
    gws = torch.empty(max(256, L.nbla_hip_gemm_bits_workspace_bytes(k._i64(M), k._i64(K), k._i64(N))), dtype=torch.uint8,
                      device=dev)
    import ctypes

    def step(ev=None):
        if ev:
            ev[0].record()
        k.check(L.nbla_hip_binarize_weights_f32(k._p(W), k._p(Wb), k._p(alpha), k._p(bits), k._i64(K), k._i64(N), 0,
                                                ctypes.c_float(1.0), None, k._p(pws), ctypes.c_size_t(pws.numel()),
                                                st))
        if ev:
            ev[1].record()
        k.check(L.nbla_hip_split_digits_f32(k._p(x), k._i64(K), k._p(xs), k._i64(M), k._i64(K), st))
        if ev:
            ev[2].record()
        k.check(L.nbla_hip_gemm_bits_f32(k._p(xs), k._p(bits), k._p(alpha), None, k._p(y), k._i64(M), k._i64(K),
                                         k._i64(N), k._i64(1), k._i64(N), k._i64(1), k._p(gws),
                                         ctypes.c_size_t(gws.numel()), st))
        if ev:
            ev[3].record()

    for _ in range(warmup):
        step()
    # The timed region: exactly `steps` steps between two synchronisations, nothing else in the queue.
    # The product's launches of the region carry the runtime's own begin / end stamps (no extra queue entries).
    if time_product:
        k.gemm_bits_timer_arm(steps)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    product = k.gemm_bits_timer_read() if time_product else None
    # The same steps once more with an event between the launches, for the per-kernel durations (the four event
    # records per step are work of their own for the queue, which is why they stay out of the region above).
    evs = [_events(4) for _ in range(steps)]
    t1 = time.perf_counter()
    for i in range(steps):
        step(evs[i])
    torch.cuda.synchronize()
    wall_ev = time.perf_counter() - t1
    prep = sum(e[0].elapsed_time(e[1]) for e in evs) / steps
    split = sum(e[1].elapsed_time(e[2]) for e in evs) / steps
    gemm = sum(e[2].elapsed_time(e[3]) for e in evs) / steps
    return {"ms_per_step": wall * 1e3 / steps, "ms_per_step_with_events": wall_ev * 1e3 / steps, "prepare_ms": prep,
            "split_ms": split, "gemm_ms": gemm, "flop": 2.0 * M * K * N, "product": product}


def bench_whole_forward(M, K, N, steps, warmup, dev, connect=False):
    """BinaryWeightAffine (BinaryConnectAffine with `connect`) forward through the whole-function entry point (what
    the Function class calls)."""
    import torch
    from nnabla_amd import kernels as k
    g = torch.Generator(device=dev).manual_seed(313)
    x = torch.randn(M, K, generator=g, device=dev)
    W = torch.randn(K, N, generator=g, device=dev) * 0.02
    ws = k.binary_affine_workspace(M, K, N, x)
    y, Wb, alpha = torch.empty(M, N, device=dev), torch.empty_like(W), torch.empty(N, device=dev)
    if connect:
        fn = lambda: k.binary_connect_affine(x, W, None, 1.0, workspace=ws, out=y, Wb=Wb)
    else:
        fn = lambda: k.binary_weight_affine(x, W, None, 1.0, workspace=ws, out=y, Wb=Wb, alpha=alpha)
    ms = time_kernel(fn, steps, warmup)
    nbytes = 8.0 * K * N + 4.0 * M * K + 4.0 * M * N + (0.0 if connect else 4.0 * N)   # read W, write Wb; x, y, alpha
    return {"ms_per_step": ms, "forward_bytes_model": nbytes, "forward_GBs": nbytes / ms / 1e6,
            "forward_frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}


def time_kernel(fn, iters, warmup=3):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = _events(2)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def bench_quantizers(dev, iters):
    import torch
    from nnabla_amd import kernels as k
    out = {}
    g = torch.Generator(device="cpu").manual_seed(313)
    x = (torch.randn(256, 65536, generator=g) * 2).to(dev)
    y = torch.empty_like(x)
    ms = time_kernel(lambda: k.fixed_point_quantize(x, True, 8, 2.0 ** -4, out=y), iters)
    nbytes = 8.0 * x.numel()
    out["fixed_point_quantize[256,65536]"] = {"ms": ms, "bytes": nbytes, "GBs": nbytes / ms / 1e6,
                                              "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    ms = time_kernel(lambda: k.pow2_quantize(x, True, True, 4, 1, out=y), iters)
    out["pow2_quantize[256,65536]"] = {"ms": ms, "bytes": nbytes, "GBs": nbytes / ms / 1e6,
                                       "frac_hbm": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    w = (torch.randn(512, 512, 3, 3, generator=g) * 0.05).to(dev)
    wq = torch.empty_like(w)
    ms = time_kernel(lambda: k.pow2_quantize(w, True, True, 4, 1, out=wq), iters)
    nb = 8.0 * w.numel()
    out["pow2_quantize[512,512,3,3]"] = {"ms": ms, "bytes": nb, "GBs": nb / ms / 1e6,
                                         "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    del x, y
    a = torch.randn(64, 256, 56, 56, generator=g).abs_().to(dev)
    ya = torch.empty_like(a)
    q = lambda v: torch.full((1, 1, 1, 1), v, device=dev)
    qmn, qmx, lmn, lmx = q(-6.0), q(6.0), q(0.0), q(255.0)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    for name, xmm, bpe in (("min_max_quantize[64,256,56,56] x_min_max", True, 12.0),
                           ("min_max_quantize[64,256,56,56] fixed range", False, 8.0)):
        ms = time_kernel(lambda: k.min_max_quantize(a, qmn, qmx, lmn, lmx, 0.999, xmm, True, 0.01, out=ya,
                                                    workspace=ws), iters)
        nb = bpe * a.numel()
        out[name] = {"ms": ms, "bytes": nb, "GBs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    # a range per (channel, column): kept axes separated by reduced ones, which the strided kernels serve
    qs = lambda v: torch.full((1, 256, 1, 56), v, device=dev)
    qmn, qmx, lmn, lmx = qs(-6.0), qs(6.0), qs(0.0), qs(255.0)
    ws2 = torch.empty(max(256, k.lib().nbla_hip_min_max_quantize_workspace_bytes(k._shape(a.shape), a.dim(),
                                                                                 k._shape(qmn.shape))),
                      dtype=torch.uint8, device=dev)
    ms = time_kernel(lambda: k.min_max_quantize(a, qmn, qmx, lmn, lmx, 0.999, True, True, 0.01, out=ya, workspace=ws2),
                     iters)
    nb = 12.0 * a.numel()
    out["min_max_quantize[64,256,56,56] x_min_max, ranges [1,256,1,56]"] = {
        "ms": ms, "bytes": nb, "GBs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    # ranges per channel, per column (every kept axis behind the reduced ones) and per (channel, row) (the innermost
    # axis reduced in short runs), and the backward pass with learnt ranges: dx and both range gradients from one pass
    # over dy and x (12 B/elem)
    dy = torch.randn(a.shape, generator=g).to(dev)
    for qshape in ((1, 1, 1, 1), (1, 256, 1, 1), (1, 1, 1, 56), (1, 256, 56, 1)):
        qs = lambda v: torch.full(qshape, v, device=dev)
        qmn, qmx, lmn, lmx = qs(-6.0), qs(6.0), qs(0.0), qs(255.0)
        tag = "ranges [%s]" % ",".join(str(v) for v in qshape)
        if qshape != (1, 1, 1, 1):
            ws3 = torch.empty(max(256, k.lib().nbla_hip_min_max_quantize_workspace_bytes(
                k._shape(a.shape), a.dim(), k._shape(qshape))), dtype=torch.uint8, device=dev)
            ms = time_kernel(lambda: k.min_max_quantize(a, qmn, qmx, lmn, lmx, 0.999, True, True, 0.01, out=ya,
                                                        workspace=ws3), iters)
            nb = 12.0 * a.numel()
            out["min_max_quantize[64,256,56,56] x_min_max, " + tag] = {
                "ms": ms, "bytes": nb, "GBs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
        _, scale = k.min_max_quantize(a, qmn, qmx, lmn, lmx, 0.999, False, False, 0.01, out=ya)
        ms = time_kernel(lambda: k.min_max_quantize_backward(dy, a, qmn, qmx, lmn, lmx, scale, True, False, False),
                         iters)
        nb = 12.0 * a.numel()
        out["min_max_quantize_backward[64,256,56,56] dx + range gradients, " + tag] = {
            "ms": ms, "bytes": nb, "GBs": nb / ms / 1e6, "frac_hbm": nb / ms / 1e6 / PEAK_HBM_GBS}
    return out


def bench_shapes(dev, iters):
    """Shapes away from the benchmark configurations (opt-in, `--section shapes`): extents that are no multiples of
    four, views that are not 16-byte aligned, grouped and depthwise convolutions, operands that broadcast -- the
    places where a kernel written for the aligned case falls to another path.  Times per call in ms."""
    import torch
    from nnabla_amd import kernels as k
    out = {}
    g = torch.Generator(device="cpu").manual_seed(7)
    for (M, K, N) in ((4096, 4096, 11008), (4096, 4095, 11008), (4096, 4096, 11007), (4097, 4097, 11009),
                      (512, 4096, 11008), (512, 4095, 11007), (64, 4096, 11007)):
        x = torch.randn(M, K, generator=g).to(dev)
        W = (torch.randn(K, N, generator=g) * 0.02).to(dev)
        dy = torch.randn(M, N, generator=g).to(dev)
        _, Wb, alpha = k.binary_weight_affine(x, W)
        out["affine %dx%dx%d" % (M, K, N)] = {
            "binary_weight_forward": time_kernel(lambda: k.binary_weight_affine(x, W), iters),
            "binary_weight_backward": time_kernel(lambda: k.binary_affine_backward(dy, x, W, Wb, alpha), iters),
            "affine_forward": time_kernel(lambda: k.affine_digits(x, W), iters),
            "affine_backward": time_kernel(lambda: k.affine_backward(dy, x, W), iters)}
        del x, W, dy, Wb, alpha
    for xs, ws, pad, stride, group in (((32, 256, 14, 14), (256, 256, 3, 3), (1, 1), (1, 1), 1),
                                       ((32, 256, 14, 14), (256, 1, 3, 3), (1, 1), (1, 1), 256),
                                       ((32, 256, 14, 14), (256, 8, 3, 3), (1, 1), (1, 1), 32),
                                       ((32, 256, 28, 28), (512, 256, 3, 3), (1, 1), (2, 2), 1),
                                       ((32, 64, 56, 56), (64, 64, 3, 3), (1, 1), (1, 1), 1),
                                       ((32, 64, 56, 56), (64, 1, 3, 3), (1, 1), (1, 1), 64),
                                       ((32, 256, 56, 56), (256, 8, 3, 3), (1, 1), (1, 1), 32),
                                       ((32, 512, 28, 28), (512, 16, 3, 3), (1, 1), (2, 2), 32),
                                       ((128, 3, 32, 32), (32, 3, 3, 3), (1, 1), (1, 1), 1)):
        x = torch.randn(xs, generator=g).to(dev)
        W = (torch.randn(ws, generator=g) * 0.05).to(dev)
        y, Wb, alpha = k.binary_weight_convolution(x, W, None, pad, stride, None, group)
        dy = torch.randn(y.shape, generator=g).to(dev)
        I = torch.zeros(ws, dtype=torch.int32, device=dev)
        out["convolution %s x %s stride %d group %d" % (list(xs), list(ws), stride[0], group)] = {
            "binary_weight_forward": time_kernel(lambda: k.binary_weight_convolution(x, W, None, pad, stride, None, group),
                                                 iters),
            "binary_weight_backward": time_kernel(lambda: k.binary_convolution_backward(dy, x, W, Wb, alpha, pad, stride,
                                                                                        None, group), iters),
            "convolution_forward": time_kernel(lambda: k.inq_convolution(x, W, I, W, I, None, pad, stride, None, group, 4,
                                                                         k.INQ_PRODUCT_ONLY), iters),
            "convolution_backward": time_kernel(lambda: k.convolution_backward(dy, x, W, pad, stride, None, group), iters)}
    xs = (64, 256, 56, 56)
    n = 64 * 256 * 56 * 56
    buf, buf2 = torch.randn(n + 8, generator=g).to(dev), torch.randn(n + 8, generator=g).to(dev)
    res = torch.empty(n + 8, device=dev)
    for off in (0, 1):
        x, dy, y = buf[off:off + n].view(xs), buf2[off:off + n].view(xs), res[off:off + n].view(xs)
        r = {}
        for qshape in ((1, 1, 1, 1), (1, 256, 1, 1)):
            q = lambda v: torch.full(qshape, v, device=dev)
            qmn, qmx, lmn, lmx = q(-6.0), q(6.0), q(0.0), q(255.0)
            r["min_max_quantize ranges %s" % (list(qshape),)] = time_kernel(
                lambda: k.min_max_quantize(x, qmn, qmx, lmn, lmx, 0.999, True, True, 0.01, out=y), iters)
        m, Mx = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
        r["fixed_point_quantize"] = time_kernel(lambda: k.fixed_point_quantize(x.view(-1), True, 8, 2.0 ** -4,
                                                                               out=y.view(-1)), iters)
        r["prune"] = time_kernel(lambda: k.prune(x.view(-1), 0.9), iters)
        r["min_max_mva_recorder"] = time_kernel(lambda: k.range_recorder(x.view(-1), m, Mx, "MinMaxMvaRecorder",
                                                                         y=y.view(-1)), iters)
        out["[64,256,56,56] %s" % ("16-byte aligned" if off == 0 else "view shifted by one float")] = r
    x, dy = buf[:n].view(xs), buf2[:n].view(xs)
    for bshape in ((64, 256, 56, 56), (1, 256, 1, 1), (1, 1, 1, 56), (1, 1, 1, 1)):
        b = (torch.rand(bshape, generator=g) + 0.5).to(dev)
        out["mul2 [64,256,56,56] x %s" % (list(bshape),)] = {
            "forward": time_kernel(lambda: k.broadcast2("mul2", x, b), iters),
            "gradient_of_the_second_operand": time_kernel(lambda: k.broadcast2_backward("mul2", 1, dy, x, b), iters)}
    return out


def bench_other_configs(dev, iters):
    """Whole-op timings (workspace allocation outside the loop is not possible through the convenience wrappers, so
    the caching allocator's hit is inside): binary convolutions of the ResNet-18 stage and the INQAffine layer."""
    import torch
    from nnabla_amd import kernels as k
    out = {}
    g = torch.Generator(device="cpu").manual_seed(7)
    x = torch.randn(32, 256, 14, 14, generator=g).to(dev)
    W = (torch.randn(256, 256, 3, 3, generator=g) * (2.0 / 2304) ** 0.5).to(dev)
    flop = 2.0 * 32 * 14 * 14 * 256 * 2304
    ms = time_kernel(lambda: k.binary_weight_convolution(x, W, None, (1, 1), (1, 1), (1, 1), 1), iters)
    out["binary_weight_convolution[32,256,14,14]x[256,256,3,3]"] = {"ms": ms, "TFLOPs": flop / ms / 1e9}
    ms = time_kernel(lambda: k.binary_connect_convolution(x, W, None, (1, 1), (1, 1), (1, 1), 1), iters)
    out["binary_connect_convolution[32,256,14,14]x[256,256,3,3]"] = {"ms": ms, "TFLOPs": flop / ms / 1e9}
    # backward of the same stage: dx, dW (db is a column sum) in one call
    dyc = torch.randn(32, 256, 14, 14, generator=g).to(dev)
    gx, gw, gb = torch.zeros_like(x), torch.zeros_like(W), torch.zeros(256, device=dev)
    ms = time_kernel(lambda: k.binary_convolution_backward(dyc, x, W, None, None, (1, 1), (1, 1), (1, 1), 1, 1.0,
                                                           dx=gx, dW=gw, db=gb), iters)
    out["binary_connect_convolution_backward[32,256,14,14]x[256,256,3,3] dx+dW+db"] = {
        "ms": ms, "TFLOPs": 2 * flop / ms / 1e9}
    # the same stage with real-valued weights (plain Convolution / INQConvolution's product)
    Ic = torch.zeros(W.shape, dtype=torch.int32, device=dev)
    Wc, oWc, oIc = W.clone(), W.clone(), Ic.clone()
    ms = time_kernel(lambda: k.inq_convolution(x, Wc, Ic, oWc, oIc, None, (1, 1), (1, 1), (1, 1), 1, 4,
                                               k.INQ_PRODUCT_ONLY), iters)
    out["convolution[32,256,14,14]x[256,256,3,3] real weights"] = {"ms": ms, "TFLOPs": flop / ms / 1e9}
    M, K, N = 1024, 4096, 4096
    xa = torch.randn(M, K, generator=g).to(dev)
    Wq = (torch.randn(K, N, generator=g) * 0.02).to(dev)
    I = torch.zeros(K, N, dtype=torch.int32, device=dev)
    oW, oI = Wq.clone(), I.clone()
    k.inq_affine(xa, Wq, I, oW, oI, None, 4, k.INQ_FIX_ALL)          # every weight becomes a power of two
    ms = time_kernel(lambda: k.inq_affine(xa, Wq, I, oW, oI, None, 4, k.INQ_NO_SELECTION), iters)
    out["inq_affine[1024,4096]x[4096,4096] (restore+quantize+product)"] = {"ms": ms, "TFLOPs": 2.0 * M * K * N / ms / 1e9}
    ms = time_kernel(lambda: k.inq_affine(xa, Wq, I, oW, oI, None, 4, k.INQ_PRODUCT_ONLY), iters)
    out["inq_affine[1024,4096]x[4096,4096] (product only)"] = {"ms": ms, "TFLOPs": 2.0 * M * K * N / ms / 1e9}
    # the 4-layer quantized MLP, batch 1024: FixedPointQuantize -> INQAffine (every weight fixed, steady-state forward:
    # restore + quantize + product) -> 3 x [ReLU -> FixedPointQuantize -> BinaryWeightAffine], all 4096 x 4096
    L = k.lib()
    Wm = [(torch.randn(K, N, generator=g) * 0.02).to(dev) for _ in range(3)]
    act = [torch.empty(M, N, device=dev) for _ in range(2)]
    ws_b = k.binary_affine_workspace(M, K, N, xa)

    def relu_(t):
        k.check(L.nbla_hip_relu_f32(k._p(t), k._p(t), ctypes.c_size_t(t.numel()), k._stream(None)))

    def mlp():
        k.fixed_point_quantize(xa, True, 8, 2.0 ** -4, out=act[0])
        h = k.inq_affine(act[0], Wq, I, oW, oI, None, 4, k.INQ_NO_SELECTION)
        for l in range(3):
            relu_(h)
            k.fixed_point_quantize(h, True, 8, 2.0 ** -4, out=act[0])
            h, _, _ = k.binary_weight_affine(act[0], Wm[l], None, 1.0, workspace=ws_b, out=act[1])
        return h
    ms = time_kernel(mlp, iters)
    out["quantized_mlp[1024 x 4096, 4 layers] forward"] = {"ms": ms, "TFLOPs": 4 * 2.0 * M * K * N / ms / 1e9}
    out["quantized_mlp[1024 x 4096, 4 layers] forward, through the function registry"] = bench_frontend_mlp(
        max(5, iters // 2))
    # backward passes (the next row of the scope table)
    n = 1 << 24
    xq = torch.randn(n, generator=g).to(dev) * 2
    gq = torch.randn(n, generator=g).to(dev)
    dq = torch.empty_like(xq)
    ms = time_kernel(lambda: k.fixed_point_quantize_backward(gq, xq, True, 8, 2.0 ** -4, True, dx=None), iters)
    out["fixed_point_quantize_backward[256,65536] fine-grained"] = {"ms": ms, "GBs": 12.0 * n / ms / 1e6,
                                                                    "frac_hbm": 12.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    # the adjacent elementwise functions: QuantizeLinear / DequantizeLinear (8 B/elem) and Prune (three histogram
    # passes over x plus the masked copy: 20 B/elem)
    x2 = (xq * 20).reshape(256, 65536)
    sc = torch.full((1, 1), 0.3, device=dev)
    zp = torch.zeros((1, 1), device=dev)
    ms = time_kernel(lambda: k.quantize_linear(x2, sc, zp, "HALF_TO_EVEN", False, k.DTYPE_BYTE), iters)
    out["quantize_linear[256,65536] per-tensor"] = {"ms": ms, "GBs": 8.0 * n / ms / 1e6,
                                                    "frac_hbm": 8.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    scc, zpc = torch.rand(1, 65536, device=dev) + 0.1, torch.zeros(1, 65536, device=dev)
    ms = time_kernel(lambda: k.dequantize_linear(x2, scc, zpc), iters)
    out["dequantize_linear[256,65536] per-column"] = {"ms": ms, "GBs": 8.0 * n / ms / 1e6,
                                                      "frac_hbm": 8.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    pws = torch.empty(k.lib().nbla_hip_prune_workspace_bytes(), dtype=torch.uint8, device=dev)
    ms = time_kernel(lambda: k.prune(xq, 0.9, workspace=pws), iters)
    out["prune[256,65536] rate 0.9"] = {"ms": ms, "GBs": 20.0 * n / ms / 1e6,
                                        "frac_hbm": 20.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    # range recorders of quantization-aware training: copy + scan (8 B/elem), or the scan alone when the output
    # aliases the input (4 B/elem)
    rws = torch.empty(k.lib().nbla_hip_range_recorder_workspace_bytes(), dtype=torch.uint8, device=dev)
    rm_, rM_, ry = torch.zeros(1, device=dev), torch.zeros(1, device=dev), torch.empty_like(x2)
    ms = time_kernel(lambda: k.range_recorder(x2, rm_, rM_, "MinMaxMvaRecorder", y=ry, workspace=rws), iters)
    out["min_max_mva_recorder[256,65536]"] = {"ms": ms, "GBs": 8.0 * n / ms / 1e6,
                                              "frac_hbm": 8.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    ms = time_kernel(lambda: k.range_recorder(x2, None, rM_, "AbsMaxRecorder", y=x2, workspace=rws), iters)
    out["abs_max_recorder[256,65536] in place"] = {"ms": ms, "GBs": 4.0 * n / ms / 1e6,
                                                   "frac_hbm": 4.0 * n / ms / 1e6 / PEAK_HBM_GBS}
    M, K, N = 4096, 4096, 11008
    xb = torch.randn(M, K, generator=g).to(dev)
    Wb_ = (torch.randn(K, N, generator=g) * 0.02).to(dev)
    gyb = torch.randn(M, N, generator=g).to(dev)
    alpha = Wb_.abs().mean(0)
    ws = torch.empty(k.lib().nbla_hip_affine_backward_workspace_bytes(k._i64(M), k._i64(K), k._i64(N)),
                     dtype=torch.uint8, device=dev)
    dxb, dwb = torch.empty(M, K, device=dev), torch.empty(K, N, device=dev)
    ms = time_kernel(lambda: k.binary_affine_backward(gyb, xb, Wb_, None, alpha, 1.0, dx=None, want=(True, False, False),
                                                      workspace=ws), max(3, iters // 2))
    out["binary_weight_affine_backward dx [4096,4096,11008]"] = {"ms": ms, "TFLOPs": 2.0 * M * K * N / ms / 1e9}
    ms = time_kernel(lambda: k.binary_affine_backward(gyb, xb, Wb_, None, alpha, 1.0, want=(False, True, False),
                                                      workspace=ws), max(3, iters // 2))
    out["binary_weight_affine_backward dW [4096,4096,11008]"] = {"ms": ms, "TFLOPs": 2.0 * M * K * N / ms / 1e9}
    return out


def bench_frontend_mlp(iters):
    """The same 4-layer quantized MLP built with the Python front-end (F.* on the hip context -> C API -> the
    "hip:float" Function classes -> C-ABI), forward() of the graph timed on the host between device synchronisations."""
    import numpy as np
    import nnabla_amd as nn
    import nnabla_amd.functions as F
    from nnabla_amd import ext_hip
    from nnabla_amd.ext_utils import get_extension_context
    rng = np.random.default_rng(313)
    B, D = 1024, 4096

    def var(a):
        v = nn.Variable(a.shape)
        v.d = a
        return v
    with nn.context_scope(get_extension_context('hip')):
        x = var(rng.standard_normal((B, D), dtype=np.float32))
        Ws = [var(rng.standard_normal((D, D), dtype=np.float32) * np.float32(0.02)) for _ in range(4)]
        h = F.fixed_point_quantize(x, True, 8, 2 ** -4)
        h = F.inq_affine(h, Ws[0], var(np.zeros((D, D), np.float32)), None, 1, 4, (0,), 'largest_abs')
        for l in range(1, 4):
            h = F.relu(h)
            h = F.fixed_point_quantize(h, True, 8, 2 ** -4)
            h = F.binary_weight_affine(h, Ws[l], nn.Variable((D, D)), nn.Variable((D,)))
        for _ in range(5):
            h.forward()
        ext_hip.device_synchronize('0')
        t0 = time.perf_counter()
        for _ in range(iters):
            h.forward()
        ext_hip.device_synchronize('0')
        ms = (time.perf_counter() - t0) / iters * 1e3
    return {"ms": ms, "TFLOPs": 4 * 2.0 * B * D * D / ms / 1e9}


def cpu_baseline(K, N, rows):
    """The CPU oracle (port of the reference's CPU arithmetic, single thread) on `rows` rows of the workload."""
    import numpy as np
    import oracle
    rng = np.random.default_rng(313)
    x = rng.standard_normal((rows, K), dtype=np.float32)
    W = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
    oracle.binary_weight_affine(x[:4], W[:, :64].copy(), None, 1.0)  # load the library
    t0 = time.perf_counter()
    oracle.binary_weight_affine(x, W, None, 1.0)
    dt = time.perf_counter() - t0
    out = {"value": 2.0 * rows * K * N / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
           "sample": "BinaryWeightAffine forward (sign/alpha passes over the full W + fp32 GEMM) on %d of 4096 "
                     "rows of x, K=%d, N=%d, %.1f s" % (rows, K, N, dt)}
    # a second, separately labelled figure: the same fp32 product alone with the host BLAS on all cores
    import torch
    xt, wt = torch.from_numpy(x), torch.from_numpy(W)
    torch.matmul(xt[:64], wt)
    t0 = time.perf_counter()
    torch.matmul(xt, wt)
    dt = time.perf_counter() - t0
    out["host_blas_sgemm"] = {"TFLOPs": 2.0 * rows * K * N / dt / 1e12, "threads": torch.get_num_threads(),
                              "note": "torch.matmul fp32 of the same rows, product only (no sign / alpha passes)"}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps; the first few dozen launches after idle run at ramping clocks")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-rows", type=int, default=2048)
    ap.add_argument("--section", choices=("all", "headline", "sweep", "quantizers", "other", "mfma", "shapes"),
                    default="all",
                    help="headline: only the timed BinaryWeightAffine steps (what the rocprofv3 summaries profile); "
                         "sweep: headline plus the forward at M = 1 .. 1024 and BinaryConnectAffine (`sweep`); "
                         "quantizers: headline plus the quantizer kernels; other: headline plus the convolution, INQ, "
                         "MLP, backward and adjacent-function workloads (`other_configs`); mfma: headline plus the rates "
                         "of kernels of nothing but matrix instructions (`mfma_rates`); shapes (not part of `all`): "
                         "headline plus shapes away from the benchmark configurations (`shapes`)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1).")
    import torch
    from nnabla_amd import kernels
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    kernels.init(0)

    M, K, N = 4096, 4096, 11008
    # The other sections run first: the headline steps are then timed on a device that is already at its working
    # clocks (the first dozens of launches after idle run on ramping clocks).  With --section headline there is
    # nothing before them and the figure is a cold one.
    sweep = {}
    for m in ((1, 8, 16, 32, 64, 128, 256, 512, 1024) if args.section in ("all", "sweep") else ()):
        s = bench_whole_forward(m, K, N, max(10, args.steps), 5, dev)
        if m > 256:   # two walks: the product runs on the matrix cores from packed bits; its share, timed between events
            t = bench_binary_weight_affine(m, K, N, max(5, args.steps // 2), 2, dev, time_product=False)
            packed_bytes = K * N / 8 + 3.0 * m * K + 4.0 * m * N + 4.0 * N
            s.update({"gemm_ms": t["gemm_ms"], "prepare_ms": t["prepare_ms"], "gemm_TFLOPs": t["flop"] / t["gemm_ms"] / 1e9,
                      "gemm_weight_GBs": packed_bytes / t["gemm_ms"] / 1e6,
                      "path": "two walks: sign / alpha / packed bits, then the packed-bit product"})
        elif m > 64:
            s["path"] = ("one walk over W: signs shared through LDS, digit operand of x, int8 matrix instructions "
                         "(K in two slices, added by a second launch)")
        elif m > 16:
            s["path"] = "one pass over W, signs fed to bf16 matrix instructions from the registers (x as three bf16 terms)"
        else:
            s["path"] = "one pass over W on the vector ALUs (no packed bits, no separate product launch)"
        sweep["M=%d" % m] = s
    # BinaryConnectAffine on the same shapes (the same kernels without alpha)
    for m in ((1, 8, 64, 512, 4096) if args.section in ("all", "sweep") else ()):
        sweep["BinaryConnectAffine M=%d" % m] = bench_whole_forward(m, K, N, max(10, args.steps // 2), 5, dev,
                                                                    connect=True)
    quant = bench_quantizers(dev, max(10, args.steps)) if args.section in ("all", "quantizers") else {}
    other = bench_other_configs(dev, max(5, args.steps // 2)) if args.section in ("all", "other") else {}
    mfma = bench_mfma_rates(dev) if args.section in ("all", "mfma") else {}
    shapes = bench_shapes(dev, max(5, args.steps // 5)) if args.section == "shapes" else {}
    r = bench_binary_weight_affine(M, K, N, args.steps, args.warmup, dev)
    tflops = r["flop"] / (r["ms_per_step"] * 1e-3) / 1e12
    # the product's duration: the begin / end stamps of its launches inside the timed region
    kernel_ms = r["product"]["mean_ms"]
    gemm_tflops = r["flop"] / (kernel_ms * 1e-3) / 1e12
    traffic, traffic_note = profiled_traffic()
    line = {
        "metric": "binary-weight affine TFLOP/s + quantizer GB/s, % of MI355X roofline",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 in/out; int8 x 3 digit MFMA operands, exact int32 accumulate", "data": "synthetic",
        "config": {"workload": "BinaryWeightAffine forward, x [4096,4096] ~ N(0,1), W [4096,11008] ~ N(0,0.02^2), "
                               "quantize_zero_to=1, no bias; whole forward = sign/alpha/pack + split + MFMA product",
                   "M": M, "K": K, "N": N},
        "roofline": {"bound": "mfma", "achieved": 3 * gemm_tflops, "peak": PEAK_INT8_MFMA_TOPS, "unit": "TOP/s",
                     "frac": 3 * gemm_tflops / PEAK_INT8_MFMA_TOPS, "traffic": traffic, "traffic_note": traffic_note,
                     "kernel": "gemm_bits_kernel<32,512,1,4,1,false>", "kernel_ms": kernel_ms,
                     "kernel_ms_min_max": [r["product"]["min_ms"], r["product"]["max_ms"]],
                     "kernel_launches_timed": r["product"]["launches"],
                     "note": "int8 operations issued (3 digit planes x 2*M*K*N) against the int8 MFMA peak; kernel_ms "
                             "is the mean over the launches of the timed steps, each stamped by the runtime with its "
                             "own begin and end (events attached to the dispatch)",
                     "fp32_equiv_TFLOPs": gemm_tflops, "fp32_equiv_over_fp32_mfma_peak": gemm_tflops / PEAK_FP32_MFMA_TFLOPS},
        "step_breakdown_ms": {"prepare": r["prepare_ms"], "split": r["split_ms"], "gemm": r["gemm_ms"],
                              "step_with_events": r["ms_per_step_with_events"],
                              "note": "an instrumented repeat of the timed steps, four event records per step: each "
                                      "share includes the queue bubbles around its event records (the product's own "
                                      "duration is roofline.kernel_ms)"},
        "mfma_rates": mfma,
        "sweep": sweep,
        "quantizers": quant,
        "other_configs": other,
    }
    if shapes:
        line["shapes"] = shapes
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(K, N, args.cpu_rows)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
