#!/usr/bin/env python3
"""Headline benchmark: AMConv2D forward + grad-input + grad-filter on the
ResNet-50 stage-1 3x3 layer (input NHWC [32,56,56,64] post-ReLU, filter
[3,3,64,64] He-normal, stride 1 SAME, upstream gradient N(0,1)) with the MBM_7
LUT, on ONE MI355X.  One step = the three passes over one synthetic batch that
is already resident in HBM.

Prints one JSON line: approximate GMAC/s (1 MAC = one approximate product + one
FP32 add; every pass is credited with the forward MAC count), the achieved
fraction of the VALU-issue / LDS-gather roofline of the GEMM kernel's
instruction mix (peaks measured on this device by micro-kernels in the same
run, nominal figures beside them), the other benchmark configurations (dense
layer, LeNet-5 convolutions, the 4096^3 GEMM sweep over ten tables, the
attention block, and every convolution of ResNet-50's bottleneck stages) under "configs", and the CPU oracle timed on a bounded sample
of the headline workload on the host cores.

`--only NAME` runs one workload alone (headline, cfg1, cfg2, cfg3-m11, cfg4, cfg4-m11,
cfg5, resnet50, short-k) without micro-kernels or CPU baseline: the form the profiler runs.
"""
import argparse
import ctypes as C
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "approx GMAC/s + % VALU/LDS roofline, AMConv2D fwd+bwd ResNet-50 3x3, MBM_7"
XS, WS = (32, 56, 56, 64), (3, 3, 64, 64)
MACS_PER_PASS = 32 * 56 * 56 * 64 * 3 * 3 * 64  # 3 699 376 128
# VALU instructions per MAC of the LDS-table kernel.  The design's minimum is 2.0 (per two MACs two
# v_lshl_add_u64 -- the LUT addresses and the product factors of two columns -- and two v_fma: the
# mix the micro-kernel issues); the inner loop as compiled has 142 per 64 MACs (operand decode
# included), and SQ_INSTS_VALU x 64 / MACs of the whole forward kernel in the committed counter
# profile is 2.47 (staging, epilogue, tail).  The roofline is priced with the minimum -- the highest
# roof, so the lowest fraction -- and states the others.
VALU_OPS_PER_MAC_MIN = 2.0
VALU_OPS_PER_MAC_LOOP = 142 / 64
VALU_OPS_PER_MAC_PROFILED = 2.47
MIN_TIMED_SECONDS = 0.3
SPEC_CLOCK_HZ = 2.4e9
WIDE_BYTES_PER_PRODUCT = 1.5   # row-staged engine at 4096 rows per workgroup, 8 columns: table row + lane operand through L2


def make_lut(kind, m):
    """Table from the library's own generator (nothing reference-derived on the measured path)."""
    from approxtrain_amd import ApproxMulLut, lut_gen
    return ApproxMulLut.from_entries(lut_gen.generate_builtin(kind, m, 1 if m <= 7 else 4), m)


def synthetic(device):
    import numpy as np
    import torch
    x = np.maximum(np.random.default_rng(9).standard_normal(XS), 0).astype(np.float32)
    w = (np.random.default_rng(10).standard_normal(WS) * np.sqrt(2.0 / 576)).astype(np.float32)
    dy = np.random.default_rng(11).standard_normal(XS).astype(np.float32)
    return x, w, dy, [torch.from_numpy(a).to(device) for a in (x, w, dy)]


def device_ms(fn, min_reps=3, min_ms=20.0, max_reps=200):
    """Mean device time of fn() in ms: HIP events on the stream the library's kernels run on
    (torch's current stream is the one handed to the library), after one warm-up call."""
    import torch
    fn()
    torch.cuda.synchronize()
    reps = min_reps
    while True:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        total = e0.elapsed_time(e1)
        if total >= min_ms or reps >= max_reps:
            return total / reps
        reps = min(max_reps, max(reps * 2, int(reps * min_ms / max(total, 1e-3)) + 1))


def device_ms_graph(fn, calls=40, replays=5):
    """Device time of fn() in ms for calls shorter than the host takes to enqueue one (about 18 us from
    Python): `calls` of them are captured into one HIP graph on a side stream and the graph's replay is
    timed with HIP events (median of `replays`, the statistic of the headline step time), so the figure
    holds no host time between launches."""
    import torch
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        fn()
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            for _ in range(calls):
                fn()
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / calls)
    return statistics.median(times)


def _microbench(lib, kind, blocks, sink, wide_table=None):
    import torch
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    best = 0.0
    for _ in range(3):
        ms, ops = C.c_double(), C.c_double()
        if wide_table is None:
            rc = lib.amsim_microbench(kind, blocks, 2000, 3, stream, C.c_void_p(sink.data_ptr()), C.byref(ms), C.byref(ops))
        else:
            rc = lib.amsim_microbench_wide(kind, blocks, 400, 3, stream, C.c_void_p(wide_table.data_ptr()),
                                           wide_table.numel() * 4, C.c_void_p(sink.data_ptr()), C.byref(ms), C.byref(ops))
        if rc != 0:
            raise RuntimeError(lib.amsim_last_error().decode())
        best = max(best, ops.value / (ms.value * 1e-3))
    return best


def measure_peaks(lib, cus):
    """Machine rates the kernels are priced against, measured on this device: VALU issue for the
    LDS-table kernel's instruction mix, byte gathers inside one 128-byte LDS row (the better of a
    64 KB / drained and a GEMM-footprint / pipelined micro-kernel), and for tables too wide for the
    LDS the rates of the row-staged design (scattered 16-bit LDS gathers, row pulls into LDS, and
    one global gather per product as the design it replaces).  Also the shader clock under the
    VALU mix: the ratio of the shader-clock and 100 MHz counters over one workgroup's loop."""
    import torch
    sink = torch.zeros(1024, device="cuda")
    out, clocks = {}, {}
    for name, kind, blocks in (("valu_mix_lane_ops_per_s", 17, cus * 8), ("valu_mix_5_per_2_macs_lane_ops_per_s", 15, cus * 8),
                               ("valu_fma_lane_ops_per_s", 10, cus * 8),
                               ("wide_valu_pair_lane_ops_per_s", 16, cus * 8),
                               ("lds_u8_row_gathers_per_s_64k_drained", 1, cus * 8),
                               ("lds_u8_row_gathers_per_s_gemm_footprint", 21, cus * 12),
                               ("lds_u8_scattered_gathers_per_s", 22, cus * 12)):
        out[name] = _microbench(lib, kind, blocks, sink)
        if kind >= 10 and kind <= 17:
            torch.cuda.synchronize()
            t = sink[512:516].cpu().view(torch.int64)
            if int(t[1]) > 0:
                clocks[name.replace("_lane_ops_per_s", "")] = float(t[0]) / float(t[1]) * 1e8
    table = torch.randint(0, 2 ** 31 - 1, (2 * 1024 * 1024 + 1024,), dtype=torch.int32, device="cuda")  # 8 MB + 4 KB
    out["wide_lds_u16_scattered_gathers_per_s"] = _microbench(lib, 2, cus, sink, table)
    out["wide_row_pull_bytes_per_s"] = _microbench(lib, 1, cus, sink, table)
    out["wide_global_gathers_per_s"] = _microbench(lib, 0, cus * 8, sink, table)
    out["wide_pull_and_gather_products_per_s"] = _microbench(lib, 3, cus, sink, table)
    out["wide_lds_b128_scattered_products_per_s"] = _microbench(lib, 4, cus, sink, table)
    out["wide_row_pull_to_registers_bytes_per_s"] = _microbench(lib, 5, cus, sink, table)
    return out, clocks


def profiled_traffic():
    """HBM bytes per launch of the forward kernel from the committed rocprofv3 counter summary
    (FETCH_SIZE / WRITE_SIZE runs scaled by the calibration copy; see the file for the commands).
    The counters cannot be read from inside this process: the figure is the last profiled one."""
    path = os.path.join(ROOT, "profiles", "lutgemm_conv3x3_resnet50_mbm7.txt")
    try:
        lines = open(path).read().split("\n")
        start = next(i for i, l in enumerate(lines) if l.startswith("== HBM traffic counters"))
        for l in lines[start:]:
            if l.startswith("lutgemm_kernel<16, 1, 1,"):
                read_mib, written_mib = (float(v) for v in l.split()[-2:])
                return {"bytes": int((read_mib + written_mib) * 2 ** 20), "read_bytes": int(read_mib * 2 ** 20),
                        "written_bytes": int(written_mib * 2 ** 20), "measured_in_run": False,
                        "source": "profiles/lutgemm_conv3x3_resnet50_mbm7.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)"}
    except (OSError, StopIteration, ValueError):
        pass
    return None


def cpu_baseline(x, w, dy):
    """The CPU oracle (a port of the reference's loop nests with the LUT
    product) on a bounded sample: the first images of the batch, all three
    passes; single thread (as the reference's CPU kernels are) and OpenMP."""
    import numpy as np
    from approxtrain_amd import lut_gen
    from oracle import cpu
    lut32 = cpu.expand_u8(np.asarray(lut_gen.generate_builtin("MBM", 7, 1), dtype=np.uint8), 7)
    nimg = 12
    xs = (nimg,) + XS[1:]
    x1, dy1 = x[:nimg].copy(), dy[:nimg].copy()
    macs = 3 * MACS_PER_PASS // XS[0] * nimg

    def run(threads):
        t0 = time.perf_counter()
        cpu.conv2d_fwd(lut32, 7, x1, w, (1, 1), "SAME", threads=threads)
        cpu.conv2d_grad_input(lut32, 7, xs, w, dy1, (1, 1), "SAME", threads=threads)
        cpu.conv2d_grad_filter(lut32, 7, x1, WS, dy1, (1, 1), "SAME", threads=threads)
        return macs / (time.perf_counter() - t0) / 1e9

    single = run(1)
    cores = min(cpu.max_threads(), len(os.sched_getaffinity(0)))
    multi = run(cores) if cores > 1 else single
    return {"value": round(multi, 4), "unit": "GMAC/s", "cores": cores, "kind": "port",
            "single_thread_value": round(single, 4),
            "sample": "first %d images of the batch ([%d,56,56,64]), fwd + grad-input + grad-filter = %.3f GMAC, "
                      "timed once single-threaded and once with OpenMP (about 12 s of CPU work); a rate, so not scaled"
                      % (nimg, nimg, macs / 1e9)}


# ---- the other benchmark configurations ---------------------------------------------------------

def _entry(macs, ms, roof_gmacs, lds_roof_gmacs=None, min_bytes_per_product=None, pull_bytes_per_s=None):
    """lds_roof_gmacs / min_bytes_per_product (width-11 entries): the rate also as a fraction of the
    roof of tables that fit the LDS, and against what the problem itself allows -- the table-row bytes
    a tile of the problem's own row count must pull from L2 per product (a 4 KB row per column and
    reduction step serves at most min(rows, 4096) products) plus 0.5 byte of lane operand -- at the
    measured pull rate: a bound set by the problem, not by this engine's choice of tile."""
    g = macs / (ms * 1e-3) / 1e9
    e = {"macs": int(macs), "device_ms": round(ms, 4), "gmacs": round(g, 1),
         "roof_frac": round(g / roof_gmacs, 4) if roof_gmacs else None}
    if lds_roof_gmacs:
        e["frac_of_lds_table_roof"] = round(g / lds_roof_gmacs, 4)
    if min_bytes_per_product and pull_bytes_per_s:
        e["min_l2_bytes_per_product"] = round(min_bytes_per_product, 3)
        e["frac_of_l2_pull_bound_at_min_bytes"] = round(g * 1e9 * min_bytes_per_product / pull_bytes_per_s, 4)
    return e


def wide_min_bytes_per_product(rows):
    """Bytes a width-11 problem with `rows` rows over the lanes must pull from L2 per product."""
    return 4096.0 / min(max(rows, 1), 4096) + 0.5


def glorot(rng, shape, fan_in, fan_out):
    import numpy as np
    lim = math.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-lim, lim, shape).astype(np.float32)


def run_cfg1(roof):
    """denseam forward, LeNet-300-100 first layer: X[128,784] U[0,1), W[784,300] Glorot-uniform, MBM_7."""
    import numpy as np
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MBM", 7)
    x = torch.from_numpy(np.random.default_rng(1).random((128, 784), dtype=np.float32)).cuda()
    w = torch.from_numpy(glorot(np.random.default_rng(2), (784, 300), 784, 300)).cuda()
    return {"denseam_fwd_128x784x300": _entry(128 * 784 * 300, device_ms_graph(lambda: functors.denseam(lut, x, w)), roof)}


def run_cfg2(roof):
    """LeNet-5 convolutions, MIT_7: conv1 5x5 1->6 SAME on [256,28,28,1], conv2 5x5 6->16 VALID on
    [256,14,14,6]; forward, grad-input, grad-filter, each credited with the forward MAC count."""
    import numpy as np
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MIT", 7)
    out = {}
    for name, xs, ws, padding, seeds in (("conv1", (256, 28, 28, 1), (5, 5, 1, 6), "SAME", (3, 4, 7)),
                                         ("conv2", (256, 14, 14, 6), (5, 5, 6, 16), "VALID", (5, 6, 8))):
        r = np.random.default_rng(seeds[0])
        x = r.random(xs, dtype=np.float32) if xs[3] == 1 else np.abs(r.standard_normal(xs)).astype(np.float32)
        w = glorot(np.random.default_rng(seeds[1]), ws, ws[0] * ws[1] * ws[2], ws[0] * ws[1] * ws[3])
        xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
        y = functors.convam(lut, xd, wd, (1, 1), padding)
        dy = torch.from_numpy((np.random.default_rng(seeds[2]).standard_normal(tuple(y.shape)) * 0.1).astype(np.float32)).cuda()
        macs = y.numel() * ws[0] * ws[1] * ws[2]
        out[name + "_fwd"] = _entry(macs, device_ms_graph(lambda: functors.convam(lut, xd, wd, (1, 1), padding)), roof)
        out[name + "_grad_input"] = _entry(macs, device_ms_graph(lambda: functors.convam_input_grad(lut, xs, wd, dy, (1, 1), padding)), roof)
        out[name + "_grad_filter"] = _entry(macs, device_ms_graph(lambda: functors.convam_filter_grad(lut, xd, ws, dy, (1, 1), padding)), roof)
    return out


def run_cfg3_wide(roof, wide_roof, pull):
    """The headline layer (cfg3) with the width-11 table MBM_11: forward, grad-input, grad-filter on the
    row-staged engine (the forward / grad-input patches from an im2col in the workspace, the filter
    gradient's 576 filter elements over the lanes)."""
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MBM", 11)
    _, _, _, (xd, wd, dyd) = synthetic("cuda")
    passes = (("fwd", 32 * 56 * 56, lambda: functors.convam(lut, xd, wd, (1, 1), "SAME")),
              ("grad_input", 32 * 56 * 56, lambda: functors.convam_input_grad(lut, XS, wd, dyd, (1, 1), "SAME")),
              ("grad_filter", 3 * 3 * 64, lambda: functors.convam_filter_grad(lut, xd, WS, dyd, (1, 1), "SAME")))
    out = {name: _entry(MACS_PER_PASS, device_ms(fn), wide_roof, roof, wide_min_bytes_per_product(rows), pull)
           for name, rows, fn in passes}
    lut.close()
    return out


def run_cfg4(roof, wide_roof, tables=None, pull=None):
    """MatMulAM 4096^3 sweep: C = A.B, dA = dC.B^T, dB = A^T.dC with N(0,1) operands, for MBM and
    MIT at mantissa widths 1, 3, 5, 7 (table in LDS) and 11 (16-bit table in device memory, rows
    staged through LDS).  The width-11 tables come from the generator's closed-form rules: no
    reference file or model exists above width 7, so their parity is unpinned beyond that rule."""
    import torch
    from approxtrain_amd import functors
    n = 4096
    g = torch.Generator(device="cuda")
    A, B, dC = (torch.randn((n, n), device="cuda", generator=g.manual_seed(s)) for s in (12, 13, 14))
    out = {}
    for kind in ("MBM", "MIT"):
        for m in (1, 3, 5, 7, 11):
            if tables is not None and (kind, m) not in tables:
                continue
            lut = make_lut(kind, m)
            r = wide_roof if m > 7 else roof
            extra = (roof, wide_min_bytes_per_product(n), pull) if m > 7 else ()
            e = {"C=A.B": _entry(n ** 3, device_ms(lambda: functors.gemm(lut, A, B)), r, *extra),
                 "dA=dC.Bt": _entry(n ** 3, device_ms(lambda: functors.gemm(lut, dC, B, trans_b=True)), r, *extra),
                 "dB=At.dC": _entry(n ** 3, device_ms(lambda: functors.gemm(lut, A, dC, trans_a=True)), r, *extra)}
            out["%s_%d" % (kind, m)] = e
            lut.close()
    return out


def run_cfg5(roof):
    """AMMHA encoder block: batch 32, seq 256, d_model 512, 8 heads of 64, MBM_7.  Projections as
    [8192,512].[512,512] dense layers (forward, and both gradients), the attention core
    (QK^T, scale + softmax, PV) over 256 (batch x head) items through the attention entry points,
    QK^T and PV alone as strided-batch GEMMs, and the whole block forward + backward."""
    import numpy as np
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MBM", 7)
    b, s, d, h = 32, 256, 512, 8
    dk = d // h
    x = torch.from_numpy(np.random.default_rng(15).standard_normal((b * s, d)).astype(np.float32)).cuda()
    ws = [torch.from_numpy(glorot(np.random.default_rng(sd), (d, d), d, d)).cuda() for sd in (16, 17, 18, 19)]
    dy = torch.randn((b * s, d), device="cuda")

    def heads(t):
        return t.reshape(b, s, h, dk).permute(0, 2, 1, 3).reshape(b * h, s, dk).contiguous()

    q, k, v = (heads(functors.denseam(lut, x, w)) for w in ws[:3])
    div = math.sqrt(dk)
    o, wts = functors.attention(lut, q, k, v, div)
    go = torch.randn_like(o)
    pm = b * s * d * d
    am = b * h * s * s * dk
    out = {
        "projection_fwd_8192x512x512": _entry(pm, device_ms(lambda: functors.denseam(lut, x, ws[0])), roof),
        "projection_dX_and_dW": _entry(2 * pm, device_ms(lambda: functors.denseam_grad(lut, dy, x, ws[0])), roof),
        "QKt_256x(256x64x256)": _entry(am, device_ms(lambda: functors.gemm(lut, q, k, trans_b=True)), roof),
        "PV_256x(256x256x64)": _entry(am, device_ms(lambda: functors.gemm(lut, wts, v)), roof),
        "attention_core_fwd (QKt, softmax, PV)": _entry(2 * am, device_ms(lambda: functors.attention(lut, q, k, v, div)), roof),
        "attention_core_bwd (4 products, softmax grad)": _entry(4 * am, device_ms(lambda: functors.attention_grad(lut, q, k, v, wts, go, div)), roof),
    }

    def block():
        for w in ws:
            functors.denseam(lut, x, w)
        functors.attention(lut, q, k, v, div)
        functors.attention_grad(lut, q, k, v, wts, go, div)
        for w in ws:
            functors.denseam_grad(lut, dy, x, w)

    out["block_fwd_bwd (4 projections + core)"] = _entry(12 * pm + 6 * am, device_ms(block), roof)
    return out


def run_short_reductions(roof):
    """Where short reductions lose their time.  Dense products [M, K] . [K, 256] with K = 64, 128, 256 at
    M = 50 176, 100 352, 200 704 (3136 to 12 544 tiles of 64 x 64 outputs on 1536 workgroup slots), each
    timed as a whole call (pre-pass + main kernel) from a captured graph: a straight line through the
    three times gives the cost of one more tile -- the marginal rate -- and what a call costs before its
    first product (pre-pass launch, ramp-up of the first round of workgroups, drain of the last)."""
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MBM", 7)
    out = {}
    for K in (64, 128, 256):
        B = torch.randn((K, 256), device="cuda")
        pts = []
        for mult in (4, 8, 16):
            M = 12544 * mult
            A = torch.randn((M, K), device="cuda")
            us = device_ms_graph(lambda: functors.gemm(lut, A, B), calls=10, replays=5) * 1e3
            pts.append((M * 256 * K, us))
            del A
        n = len(pts)
        sx, sy = sum(p[0] for p in pts), sum(p[1] for p in pts)
        sxx, sxy = sum(p[0] * p[0] for p in pts), sum(p[0] * p[1] for p in pts)
        slope = (n * sxy - sx * sy) / (n * sxx - sx * sx)  # us per MAC
        fixed = (sy - slope * sx) / n
        e = {"call_us_at_3136_6272_12544_tiles": [round(p[1], 1) for p in pts],
             "fixed_us_per_call": round(fixed, 1), "marginal_gmacs": round(1e-3 / slope, 1)}
        if roof:
            e["marginal_roof_frac"] = round(1e-3 / slope / roof, 4)
        out["K=%d" % K] = e
    return out


RESNET50_SIZES = (("feature_maps_56_to_7", 56, 64), ("feature_maps_32_to_4_cifar", 32, 3))


def resnet50_layers(hw0, cin0):
    """The distinct convolutions of ResNet-50's bottleneck stages 2-5 for an hw0 x hw0 x cin0 input to
    stage 2: (name, H = W, Cin, Cout, filter size, stride, how many the model holds)."""
    layers = []
    hw, cin = hw0, cin0
    for stage, (f1, f3, nblocks, stride) in enumerate(((64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2), (512, 2048, 3, 2)), start=2):
        ohw = (hw - 1) // stride + 1
        layers += [("s%da_1x1/%d_%d_%d" % (stage, stride, cin, f1), hw, cin, f1, 1, stride, 1),
                   ("s%da_shortcut_1x1/%d_%d_%d" % (stage, stride, cin, f3), hw, cin, f3, 1, stride, 1),
                   ("s%d_3x3_%d_%d" % (stage, f1, f1), ohw, f1, f1, 3, 1, nblocks),
                   ("s%d_1x1_%d_%d" % (stage, f1, f3), ohw, f1, f3, 1, 1, nblocks),
                   ("s%d_1x1_%d_%d" % (stage, f3, f1), ohw, f3, f1, 1, 1, nblocks - 1)]
        hw, cin = ohw, f3
    return layers


def run_resnet50(roof, only_layer=None):
    """Every convolution of ResNet-50's bottleneck stages 2-5 (the layout profile/resnet50.py:295-313
    builds: per stage one block with a strided 1x1 and a 1x1 shortcut, then identity blocks of
    1x1 -> 3x3 -> 1x1) at batch 32, MBM_7: forward, grad-input and grad-filter of each distinct layer
    shape timed once and weighted by how often the model holds it.  Two sizes: feature maps 56 / 28 /
    14 / 7 (an ImageNet-sized input behind the stem and pooling; its stage-2 3x3 layer is the headline
    workload) and 32 / 16 / 8 / 4 on a 3-channel image (the reference's CIFAR-10 profile model)."""
    import torch
    from approxtrain_amd import functors
    lut = make_lut("MBM", 7)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(20)
    out = {}
    for label, hw0, cin0 in RESNET50_SIZES:
        layers = [l for l in resnet50_layers(hw0, cin0) if only_layer is None or l[0] == only_layer]
        if not layers:
            continue
        total_ms = total_macs = 0.0
        per_layer = {}
        for name, hw, cin, cout, k, stride, count in layers:
            xs, ws, pad = (32, hw, hw, cin), (k, k, cin, cout), ("SAME" if k == 3 else "VALID")
            x = torch.relu(torch.randn(*xs, device="cuda", generator=gen))
            w = torch.randn(*ws, device="cuda", generator=gen) * math.sqrt(2.0 / (k * k * cin))
            y = functors.convam(lut, x, w, (stride, stride), pad)
            dy = torch.randn(*y.shape, device="cuda", generator=gen)
            macs = y.numel() * k * k * cin
            ms = [device_ms_graph(lambda: functors.convam(lut, x, w, (stride, stride), pad), calls=10, replays=3),
                  device_ms_graph(lambda: functors.convam_input_grad(lut, xs, w, dy, (stride, stride), pad), calls=10, replays=3),
                  device_ms_graph(lambda: functors.convam_filter_grad(lut, x, ws, dy, (stride, stride), pad), calls=10, replays=3)]
            total_ms += sum(ms) * count
            total_macs += 3.0 * macs * count
            per_layer[name] = {"count": count, "mmacs_per_pass": round(macs / 1e6, 1),
                               "fwd_gi_gf_gmacs": [round(macs / (t * 1e-3) / 1e9, 1) for t in ms]}
        e = _entry(total_macs, total_ms, roof)
        e["layers"] = per_layer
        out[label] = e
    return out


def calibration_copy(lib):
    """One plain copy of known size (64 MiB read + 64 MiB written), outside every timed region:
    the kernel that FETCH_SIZE / WRITE_SIZE counter readings are scaled against."""
    import torch
    cal_src = torch.ones(16 * 1024 * 1024, device="cuda")
    cal_dst = torch.empty_like(cal_src)
    lib.amsim_calibration_copy(C.c_void_p(cal_src.data_ptr()), C.c_void_p(cal_dst.data_ptr()), cal_src.numel(),
                               C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="headline workload only")
    ap.add_argument("--layer", default=None, help="with --only resnet50: one layer by name, e.g. s3a_1x1/2_256_128 (both sizes)")
    ap.add_argument("--only", default=None, help="run one workload alone: headline, cfg1, cfg2, cfg3-m11, cfg4, cfg4-m11, cfg5, resnet50, short-k")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import approxtrain_amd
    from approxtrain_amd import functors
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    lib = approxtrain_amd.load_library()
    torch.cuda.set_device(0)
    arch = C.create_string_buffer(64)
    cus = C.c_int()
    lib.amsim_device_info(arch, 64, C.byref(cus))

    if args.only and args.only != "headline":
        runners = {"cfg1": lambda: run_cfg1(None), "cfg2": lambda: run_cfg2(None), "cfg4": lambda: run_cfg4(None, None),
                   "cfg3-m11": lambda: run_cfg3_wide(None, None, None), "short-k": lambda: run_short_reductions(None),
                   "cfg4-m11": lambda: run_cfg4(None, None, tables={("MBM", 11), ("MIT", 11)}), "cfg5": lambda: run_cfg5(None),
                   "resnet50": lambda: run_resnet50(None, args.layer)}
        if args.only not in runners:
            sys.exit("unknown workload " + args.only)
        calibration_copy(lib)
        print(json.dumps({"workload": args.only, "results": runners[args.only]()}))
        return

    x, w, dy, (xd, wd, dyd) = synthetic("cuda")
    lut = make_lut("MBM", 7)

    passes = {
        "fwd": lambda: functors.convam(lut, xd, wd, (1, 1), "SAME"),
        "grad_input": lambda: functors.convam_input_grad(lut, XS, wd, dyd, (1, 1), "SAME"),
        "grad_filter": lambda: functors.convam_filter_grad(lut, xd, WS, dyd, (1, 1), "SAME"),
    }

    def step():
        for fn in passes.values():
            fn()

    def timed_block():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    for _ in range(args.warmup):
        step()
    # Blocks of exactly --steps steps, each bracketed by a device synchronisation, until at least
    # MIN_TIMED_SECONDS have been timed; the reported step time is the median block's.
    blocks = [timed_block()]
    while sum(blocks) < MIN_TIMED_SECONDS and len(blocks) < 1000:
        blocks.append(timed_block())
    ms_per_step = statistics.median(blocks) * 1e3 / args.steps

    # per-pass device time with HIP events on the stream the kernels run on
    pass_ms = {name: device_ms(fn, min_reps=args.steps, min_ms=100.0) for name, fn in passes.items()}
    if args.only == "headline":
        print(json.dumps({"workload": "headline", "ms_per_step": round(ms_per_step, 4), "pass_ms": pass_ms}))
        return

    calibration_copy(lib)

    peaks, clocks = measure_peaks(lib, cus.value)
    ops_per_mac = VALU_OPS_PER_MAC_MIN
    valu_bound = peaks["valu_mix_lane_ops_per_s"] / ops_per_mac / 1e9
    lds_rate = max(peaks["lds_u8_row_gathers_per_s_64k_drained"], peaks["lds_u8_row_gathers_per_s_gemm_footprint"])
    lds_bound = lds_rate / 1e9
    peak = min(valu_bound, lds_bound)
    # Row-staged engine (tables too wide for the LDS) at 4096^3, width 11: per product 1 byte of table row
    # (a 4 KB row serves a workgroup's 4096 rows) + 0.5 byte of lane operand (4 bytes serve 8 columns) come
    # in from L2; one 16-bit multiply-add + one FMA; one eighth of a 16-byte LDS read.
    wide_bounds = {
        "l2_pull_at_1.5_bytes_per_product": max(peaks["wide_row_pull_bytes_per_s"], peaks["wide_row_pull_to_registers_bytes_per_s"]) / WIDE_BYTES_PER_PRODUCT / 1e9,
        "valu_pair_at_2_ops_per_product": peaks["wide_valu_pair_lane_ops_per_s"] / 2.0 / 1e9,
        "lds_16_byte_scattered_reads": peaks["wide_lds_b128_scattered_products_per_s"] / 1e9,
    }
    wide_peak = min(wide_bounds.values())
    wide_pull = max(peaks["wide_row_pull_bytes_per_s"], peaks["wide_row_pull_to_registers_bytes_per_s"])
    clock = clocks.get("valu_mix", SPEC_CLOCK_HZ)
    # dominant kernel: the patch-gather LUT GEMM of the forward pass (grad-input runs the same kernel)
    achieved = MACS_PER_PASS / (pass_ms["fwd"] * 1e-3) / 1e9
    value = 3 * MACS_PER_PASS / (ms_per_step * 1e-3) / 1e9
    alg_bytes = 4 * (2 * 32 * 56 * 56 * 64 + 3 * 3 * 64 * 64)  # un-lowered input + output + filter
    result = {
        "metric": METRIC, "value": round(value, 2), "unit": "GMAC/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "AMConv2D fwd + grad-input + grad-filter, input NHWC [32,56,56,64] max(0,N(0,1)), "
                               "filter [3,3,64,64] He-normal, stride 1 SAME, dY N(0,1), LUT MBM_7 (m=7) in LDS",
                   "macs_per_step": 3 * MACS_PER_PASS, "device": arch.value.decode(), "compute_units": cus.value},
        "timing": {"blocks_of_steps_timed": len(blocks), "seconds_timed": round(sum(blocks), 4),
                   "ms_per_step_min_block": round(min(blocks) * 1e3 / args.steps, 4),
                   "ms_per_step_max_block": round(max(blocks) * 1e3 / args.steps, 4),
                   "rule": "median over blocks of exactly --steps steps, blocks repeated until %.1f s are timed" % MIN_TIMED_SECONDS},
        "pass_ms": {k: round(v, 4) for k, v in pass_ms.items()},
        "pass_gmacs": {k: round(MACS_PER_PASS / (v * 1e-3) / 1e9, 1) for k, v in pass_ms.items()},
        "roofline": {
            "bound": "valu" if valu_bound <= lds_bound else "lds",
            "kernel": "lutgemm_kernel<16,1,P_PATCH> (forward pass)",
            "achieved": round(achieved, 1), "peak": round(peak, 1), "unit": "GMAC/s",
            "frac": round(achieved / peak, 4),
            "frac_whole_step": round(value / peak, 4),
            "valu_ops_per_mac": {"design_minimum": VALU_OPS_PER_MAC_MIN, "inner_loop_isa": round(VALU_OPS_PER_MAC_LOOP, 3),
                                 "profiled_SQ_INSTS_VALU_x64_per_mac": VALU_OPS_PER_MAC_PROFILED, "used": ops_per_mac},
            "valu_bound_gmacs": round(valu_bound, 1), "lds_bound_gmacs": round(lds_bound, 1),
            "valu_bound_gmacs_at_loop_count": round(peaks["valu_mix_lane_ops_per_s"] / VALU_OPS_PER_MAC_LOOP / 1e9, 1),
            "valu_bound_gmacs_at_profiled_count": round(peaks["valu_mix_lane_ops_per_s"] / VALU_OPS_PER_MAC_PROFILED / 1e9, 1),
            "measured_peaks": {k: round(v / 1e12, 3) for k, v in peaks.items()}, "measured_peaks_unit": "T/s",
            "shader_clock_ghz_measured": {k: round(v / 1e9, 3) for k, v in clocks.items()},
            "nominal": {
                "note": "compute units x 4 SIMDs x 16 lanes x clock for VALU instructions that read a scalar register "
                        "(instructions on vector registers only issue a wavefront in 2 cycles: 32 lanes per clock); "
                        "compute units x 32 lanes per clock for LDS gathers of 4 bytes or less",
                "valu_lane_ops_per_s_at_measured_clock_T": round(cus.value * 64 * clock / 1e12, 2),
                "valu_lane_ops_per_s_at_2.4GHz_T": round(cus.value * 64 * SPEC_CLOCK_HZ / 1e12, 2),
                "lds_gathers_per_s_at_measured_clock_T": round(cus.value * 32 * clock / 1e12, 2),
                "lds_gathers_per_s_at_2.4GHz_T": round(cus.value * 32 * SPEC_CLOCK_HZ / 1e12, 2),
                "frac_of_nominal_lds_at_2.4GHz": round(achieved * 1e9 / (cus.value * 32 * SPEC_CLOCK_HZ), 4),
            },
            "wide_table_peak_gmacs": round(wide_peak, 1),
            "wide_table_bounds_gmacs": {k: round(v, 1) for k, v in wide_bounds.items()},
            "hbm": {"algorithmic_bytes": alg_bytes, "achieved_GBps": round(alg_bytes / (pass_ms["fwd"] * 1e-3) / 1e9, 1),
                    "peak_GBps": 8000.0},
            "traffic": profiled_traffic(),
        },
    }
    if not args.no_configs:
        result["configs"] = {
            "note": "device time per call from HIP events (ms; cfg1 and cfg2, whose calls are shorter than the host's "
                    "enqueue time, from the replay of a captured graph of 40 calls), MACs as counted for the headline, roof_frac against "
                    "roofline.peak (tables in LDS) or roofline.wide_table_peak_gmacs (width 11: the lowest of "
                    "roofline.wide_table_bounds_gmacs -- bytes pulled in from L2 at 1.5 per product, the factor + FMA "
                    "instruction pair, scattered 16-byte LDS reads); width-11 entries also carry their fraction of the LDS-table "
                    "roof and of the L2 pull bound at the bytes per product the problem's own row count requires",
            "cfg1": run_cfg1(peak), "cfg2": run_cfg2(peak), "cfg3_MBM_11": run_cfg3_wide(peak, wide_peak, wide_pull),
            "cfg4": run_cfg4(peak, wide_peak, pull=wide_pull), "cfg5": run_cfg5(peak),
            "resnet50_convolutions_batch32": run_resnet50(peak),
            "short_reductions_fixed_cost_and_marginal_rate": run_short_reductions(peak),
        }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x, w, dy)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
