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
run), and the CPU oracle timed on a bounded sample of the same workload on the
host cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "approx GMAC/s + % VALU/LDS roofline, AMConv2D fwd+bwd ResNet-50 3x3, MBM_7"
LUT_FILE = os.path.join(ROOT, "tests", "golden", "lut", "MBM_7.bin")
XS, WS = (32, 56, 56, 64), (3, 3, 64, 64)
MACS_PER_PASS = 32 * 56 * 56 * 64 * 3 * 3 * 64  # 3 699 376 128
VALU_OPS_PER_MAC = 2.5    # per two MACs: one v_lshl_add_u64 (two LUT addresses), two v_lshl_add_u32 (byte -> product factor), two v_fma
NOMINAL_OPS_PER_MAC = 5   # the figure the roofline definition quotes as nominal


def synthetic(device):
    import numpy as np
    import torch
    x = np.maximum(np.random.default_rng(9).standard_normal(XS), 0).astype(np.float32)
    w = (np.random.default_rng(10).standard_normal(WS) * np.sqrt(2.0 / 576)).astype(np.float32)
    dy = np.random.default_rng(11).standard_normal(XS).astype(np.float32)
    return x, w, dy, [torch.from_numpy(a).to(device) for a in (x, w, dy)]


def measure_peaks(lib, cus):
    """VALU issue rate for the kernel's per-MAC instruction mix and the LDS
    gather rate for its access shape (byte reads inside one 128-byte row),
    measured on this device."""
    import torch
    sink = torch.zeros(1024, device="cuda")
    out = {}
    for name, kind in (("valu_mix_lane_ops_per_s", 15), ("valu_fma_lane_ops_per_s", 10),
                       ("lds_u8_row_gathers_per_s", 1), ("lds_u8_scattered_gathers_per_s", 2)):
        best = 0.0
        for _ in range(3):
            ms, ops = C.c_double(), C.c_double()
            rc = lib.amsim_microbench(kind, cus * 8, 2000, 3, C.c_void_p(torch.cuda.current_stream().cuda_stream),
                                      C.c_void_p(sink.data_ptr()), C.byref(ms), C.byref(ops))
            if rc != 0:
                raise RuntimeError(lib.amsim_last_error().decode())
            best = max(best, ops.value / (ms.value * 1e-3))
        out[name] = best
    return out


def profiled_traffic():
    """HBM bytes per launch of the forward kernel from the committed rocprofv3 counter summary
    (FETCH_SIZE / WRITE_SIZE runs scaled by the calibration copy; see the file for the commands).
    The counters cannot be read from inside this process, so the figure is the last profiled one."""
    path = os.path.join(ROOT, "profiles", "lutgemm_conv3x3_resnet50_mbm7.txt")
    try:
        lines = open(path).read().split("\n")
        start = next(i for i, l in enumerate(lines) if l.startswith("== HBM traffic counters"))
        for l in lines[start:]:
            if l.startswith("lutgemm_kernel<16, 1, 1,"):
                read_mib, written_mib = (float(v) for v in l.split()[-2:])
                return {"bytes": int((read_mib + written_mib) * 2 ** 20), "read_bytes": int(read_mib * 2 ** 20),
                        "written_bytes": int(written_mib * 2 ** 20),
                        "source": "profiles/lutgemm_conv3x3_resnet50_mbm7.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)"}
    except (OSError, StopIteration, ValueError):
        pass
    return None


def cpu_baseline(x, w, dy):
    """The CPU oracle (a port of the reference's loop nests with the LUT
    product) on a bounded sample: the first images of the batch, all three
    passes; single thread (as the reference's CPU kernels are) and OpenMP."""
    import numpy as np
    from oracle import cpu
    lut32 = cpu.expand_u8(np.fromfile(LUT_FILE, dtype=np.uint8), 7)
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import approxtrain_amd
    from approxtrain_amd import ApproxMulLut, functors
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    lib = approxtrain_amd.load_library()
    torch.cuda.set_device(0)
    arch = C.create_string_buffer(64)
    cus = C.c_int()
    lib.amsim_device_info(arch, 64, C.byref(cus))

    x, w, dy, (xd, wd, dyd) = synthetic("cuda")
    lut = ApproxMulLut(LUT_FILE)

    passes = {
        "fwd": lambda: functors.convam(lut, xd, wd, (1, 1), "SAME"),
        "grad_input": lambda: functors.convam_input_grad(lut, XS, wd, dyd, (1, 1), "SAME"),
        "grad_filter": lambda: functors.convam_filter_grad(lut, xd, WS, dyd, (1, 1), "SAME"),
    }

    def step():
        for fn in passes.values():
            fn()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # per-pass device time with HIP events on the stream the kernels run on
    # (torch's current stream is the one handed to the library)
    pass_ms = {}
    for name, fn in passes.items():
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        pass_ms[name] = e0.elapsed_time(e1) / args.steps

    # one plain copy of known size (64 MiB read + 64 MiB written), outside every timed
    # region: the kernel that FETCH_SIZE / WRITE_SIZE counter readings are scaled against
    cal_src = torch.ones(16 * 1024 * 1024, device="cuda")
    cal_dst = torch.empty_like(cal_src)
    lib.amsim_calibration_copy(C.c_void_p(cal_src.data_ptr()), C.c_void_p(cal_dst.data_ptr()), cal_src.numel(),
                               C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()

    peaks = measure_peaks(lib, cus.value)
    valu_bound = peaks["valu_mix_lane_ops_per_s"] / VALU_OPS_PER_MAC / 1e9
    lds_bound = peaks["lds_u8_row_gathers_per_s"] / 1e9
    peak = min(valu_bound, lds_bound)
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
        "pass_ms": {k: round(v, 4) for k, v in pass_ms.items()},
        "pass_gmacs": {k: round(MACS_PER_PASS / (v * 1e-3) / 1e9, 1) for k, v in pass_ms.items()},
        "roofline": {
            "bound": "valu" if valu_bound <= lds_bound else "lds",
            "kernel": "lutgemm_kernel<16,1,P_PATCH> (forward pass)",
            "achieved": round(achieved, 1), "peak": round(peak, 1), "unit": "GMAC/s",
            "frac": round(achieved / peak, 4),
            "frac_whole_step": round(value / peak, 4),
            "valu_ops_per_mac": VALU_OPS_PER_MAC,
            "valu_bound_gmacs": round(valu_bound, 1), "lds_bound_gmacs": round(lds_bound, 1),
            "nominal_5op_valu_bound_gmacs": round(peaks["valu_mix_lane_ops_per_s"] / NOMINAL_OPS_PER_MAC / 1e9, 1),
            "measured_peaks": {k: round(v / 1e12, 3) for k, v in peaks.items()}, "measured_peaks_unit": "T/s",
            "hbm": {"algorithmic_bytes": alg_bytes, "achieved_GBps": round(alg_bytes / (pass_ms["fwd"] * 1e-3) / 1e9, 1),
                    "peak_GBps": 8000.0},
            "traffic": profiled_traffic(),
        },
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(x, w, dy)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
