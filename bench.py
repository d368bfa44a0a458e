#!/usr/bin/env python3
"""Benchmark of the conv-as-GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2|cfg1|cfg3|cfg4|cfg5]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident in
HBM.  The default workload is the VGG16-style 3x3 layer (N=64, 256 -> 256 channels, 56x56, fp32,
NCHW): forward + filter gradient + bias gradient + input gradient through the implicit-GEMM
kernels.  One JSON line is printed: whole-step GFLOP/s as ``value``, the forward kernel's measured
fraction of the fp32 MFMA peak under ``roofline`` (HIP events around that kernel inside the timed
region), and the CPU restatement of the reference's path (Cython-style im2col in C/OpenMP + NumPy
``@``), timed on the host cores on a bounded sample, under ``cpu_baseline``.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "conv GFLOP/s & % fp32 MFMA peak (3x3 VGG layer); VGG16 train img/s, 1 GPU"
FP32_MFMA_PEAK_TFLOPS = 157.3   # 256 CU x 2.4 GHz x 256 FLOP/clk/CU
HBM_PEAK_GBS = 8000.0

# HBM-side bytes per launch of the forward kernel, from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), each
# scaled by what the same counter reads for a 256 MiB copy (factors 2.000 and 1.000):
# main launch (166365.0 * 2.0 + 262144.0) KiB plus the fixup launch of its cut tiles (32825.7 * 2.0 + 4096.0) KiB.
# The figure belongs to one launch form of one build: `launch` is what pydtnn_hip_debug_last_launch reported for
# the forward call in the profiled runs and `commit` the source revision they were built from.  A run whose
# forward call launches anything else reports traffic null instead of this constant.
TRAFFIC_PROFILE = {
    "file": "profiles/cfg2_conv3x3_pmc_counters.md",
    "commit": "c763f5b",
    "launch": {"kind": "balanced", "tile": [256, 128], "workgroups": 512, "cut_tiles": 32, "splits": 1},
    "bytes": int((166365.0 * 2.0 + 262144.0 + 32825.7 * 2.0 + 4096.0) * 1024),
}


def traffic_of_forward(launch):
    """(traffic, traffic_source) of the roofline object: the profiled constant when this run's forward call took
    the profiled launch form, else null with the reason."""
    if launch == TRAFFIC_PROFILE["launch"]:
        return TRAFFIC_PROFILE["bytes"], (
            f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of commit {TRAFFIC_PROFILE['commit']} summarised in "
            f"{TRAFFIC_PROFILE['file']} (a constant read off that profile, not measured by this run; this run's "
            f"forward call took the profiled launch form {launch})")
    return None, (f"none: this run's forward call launched {launch}, the counters in {TRAFFIC_PROFILE['file']} were "
                  f"collected for {TRAFFIC_PROFILE['launch']}")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "resnet50"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vgg16", action="store_true", help="skip the VGG16 training-step extra of the default run")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip cfg1, cfg3 and cfg4 (GPU and CPU legs) in the default run's extra")
    ap.add_argument("--settle", type=float, default=SETTLE_SECONDS,
                    help="least duration in seconds of the untimed part before each timed region (counter passes of "
                         "a profiler, whose figures do not depend on the clocks, use 0)")
    ap.add_argument("--one-stream", action="store_true",
                    help="cfg5: build the headline model with enable_backward_overlap=False (kernel traces then show "
                         "each kernel alone on the chip)")
    ap.add_argument("--no-folding-extra", action="store_true",
                    help="skip the extra VGG16 runs (enable_relu_folding=False; NHWC) that are reported beside the headline one")
    ap.add_argument("--conv-layers", action="store_true",
                    help="with --workload cfg5: also time forward / dW / dX of each distinct VGG16 convolution alone")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a plain 256 MiB device copy (chan_eltwise_vec4_kernel with no epilogue) three "
                         "times, so that rocprofv3 FETCH_SIZE / WRITE_SIZE readings can be scaled to bytes")
    return ap.parse_args()


# --------------------------------------------------------------------------- synthetic inputs (seed 0)

def he_normal(rng, shape, fan_in):
    import numpy as np
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def make_cfg2(n=64):
    import numpy as np
    rng = np.random.default_rng(0)
    x = rng.standard_normal((n, 256, 56, 56), dtype=np.float32)
    w = he_normal(rng, (256, 256, 3, 3), 2304)
    b = np.zeros(256, np.float32)
    dy = rng.standard_normal((n, 256, 56, 56), dtype=np.float32)
    return x, w, b, dy


class Timer:
    """HIP events on torch's current stream, which is the stream every kernel here is launched on."""

    def __init__(self, torch):
        self.torch = torch
        self.pairs = []

    def __call__(self, fn, *a, **kw):
        s, e = self.torch.cuda.Event(enable_timing=True), self.torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn(*a, **kw)
        e.record()
        self.pairs.append((s, e))
        return out

    def mean_ms(self):
        return sum(s.elapsed_time(e) for s, e in self.pairs) / max(1, len(self.pairs))

    def median_ms(self):
        """For single short launches: an interval that caught a host hiccup (the queue ran dry between the two
        events) does not count."""
        times = sorted(s.elapsed_time(e) for s, e in self.pairs)
        return times[len(times) // 2]


SETTLE_SECONDS = 0.1


def timed_steps(torch, step, steps, warmup):
    """`warmup` untimed steps, then exactly `steps` timed ones between two synchronizations.  The untimed part
    lasts at least SETTLE_SECONDS: after an idle spell the GPU runs below its sustained clocks for some 20 ms
    (the ResNet block measures 0.33 ms for its first 50 steps and 0.295 ms from then on), which the warm-up
    steps of a sub-millisecond workload would not cover."""
    t_start = time.perf_counter()
    for _ in range(warmup):
        step(None)
    torch.cuda.synchronize()
    while time.perf_counter() - t_start < SETTLE_SECONDS:
        for _ in range(10):
            step(None)
        torch.cuda.synchronize()
    timers = {}
    t0 = time.perf_counter()
    for _ in range(steps):
        step(timers)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps, timers


# --------------------------------------------------------------------------- workloads

def run_cfg2(torch, pd, args):
    import numpy as np
    x, w, b, dy = make_cfg2()
    n = x.shape[0]
    model = pd.Model(tensor_format="NCHW", batch_size=n)
    model.mode = pd.TRAIN_MODE
    conv = pd.Conv2D(nfilters=256, filter_shape=(3, 3), padding=1)
    conv.set_model(model)
    conv.initialize(prev_shape=(256, 56, 56))
    conv.weights, conv.biases = torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda()
    xd, dyd = torch.from_numpy(x).cuda(), torch.from_numpy(dy).cuda()
    from pydtnn_amd import ops

    def step(timers):
        if timers is None:
            conv.forward(xd)
            conv.backward(dyd)
            return
        for name in ("fwd", "dw", "db", "dx"):
            timers.setdefault(name, Timer(torch))
        kw = conv._cg_kwargs()
        conv.cg_x = xd
        timers["fwd"](conv.cg.conv_gemm_nchw, conv.weights, xd, biases=None, biases_vector=conv.biases, **kw)
        dw = torch.empty_like(conv.weights)
        timers["dw"](conv.cg.conv_gemm_nchw, dyd, xd, biases=dw, trans=True, **kw)
        timers["db"](ops.bias_grad, dyd, 256, 56 * 56)
        dx = torch.empty_like(xd)
        timers["dx"](conv.cg.deconv_gemm_nchw, conv.weights, dyd, dx, **kw)

    ms, timers = timed_steps(torch, step, args.steps, args.warmup)
    from pydtnn_amd import native
    conv.cg.conv_gemm_nchw(conv.weights, xd, biases=None, biases_vector=conv.biases, **conv._cg_kwargs())
    fwd_launch = native.last_launch()
    gemm_flop = 2.0 * 256 * 2304 * n * 56 * 56
    step_flop = 3 * gemm_flop
    fwd_ms = timers["fwd"].mean_ms()
    achieved = gemm_flop / (fwd_ms * 1e-3) / 1e12
    kernels = {k: round(t.mean_ms(), 4) for k, t in timers.items()}
    extra = {
        "kernel_ms": kernels,
        "fwd_tflops": round(achieved, 2),
        "dw_tflops": round(gemm_flop / (kernels["dw"] * 1e-3) / 1e12, 2),
        "dx_tflops": round(gemm_flop / (kernels["dx"] * 1e-3) / 1e12, 2),
        "fwd_pct_fp32_mfma_peak": round(100 * achieved / FP32_MFMA_PEAK_TFLOPS, 2),
        "step_gflop": round(step_flop / 1e9, 2),
    }
    # explicit-path streams: bytes(x) + bytes(cols) and bytes(cols) + bytes(dx).  The C ABI is called on buffers
    # allocated once, so that no allocation falls between a pair of timing events.
    from pydtnn_amd.native import check, f32, lib, stream_ptr
    geom = (3, 3, 1, 1, 1, 1, 1, 1)
    mat = torch.empty(256 * 9 * n * 56 * 56, device="cuda")   # x_cols (K x P) or x_rows (P x K)
    back = torch.empty_like(xd)
    stream_bytes = x.nbytes + mat.numel() * 4
    calls = {
        "im2col": lambda: check(lib().pydtnn_hip_im2col_nchw(f32(xd), f32(mat), n, 256, 56, 56, *geom, stream_ptr()),
                                "im2col_nchw"),
        "col2im": lambda: check(lib().pydtnn_hip_col2im_nchw(f32(mat), f32(back), n, 256, 56, 56, *geom, stream_ptr()),
                                "col2im_nchw"),
        # the NHWC pair on the same layer (x viewed as N,56,56,256; the values do not matter for a stream)
        "im2row": lambda: check(lib().pydtnn_hip_im2row_nhwc(f32(xd), f32(mat), n, 56, 56, 256, *geom, stream_ptr()),
                                "im2row_nhwc"),
        "row2im": lambda: check(lib().pydtnn_hip_row2im_nhwc(f32(mat), f32(back), n, 56, 56, 256, *geom, stream_ptr()),
                                "row2im_nhwc"),
    }
    # each gather alone: one untimed launch, then the median of ten launches in a row; the adjoints also right
    # after the kernel that wrote their matrix (its dirty lines are still being written back while they read)
    for first, second in (("im2col", "col2im"), ("im2row", "row2im")):
        for name in (first, second):
            t = Timer(torch)
            for i in range(11):
                calls[name]() if i == 0 else t(calls[name])
            torch.cuda.synchronize()
            extra[name + "_gbs"] = round(stream_bytes / (t.median_ms() * 1e-3) / 1e9, 1)
        t2 = Timer(torch)
        for i in range(6):
            calls[first]()
            calls[second]() if i == 0 else t2(calls[second])
        torch.cuda.synchronize()
        extra[f"{second}_after_{first}_gbs"] = round(stream_bytes / (t2.median_ms() * 1e-3) / 1e9, 1)
    extra["im2col_pct_hbm_peak"] = round(100 * extra["im2col_gbs"] / HBM_PEAK_GBS, 1)
    extra["col2im_pct_hbm_peak"] = round(100 * extra["col2im_gbs"] / HBM_PEAK_GBS, 1)
    # the explicit route on the same layer (Conv2D with enable_conv_gemm=False): the three GEMMs over the
    # materialised column matrix, (co,K)@(K,P) forward, (co,P)@(P,K) for dw and (K,co)@(co,P) + col2im for dx,
    # each 236.76 GFLOP, with the buffers of the gather timings above
    # the (K x P) product of the explicit dx and, behind it, the scratch of the balanced launch
    kxp_bytes = lib().pydtnn_hip_conv_workspace_bytes(native.OP_DX_I2C, 0, n, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1)
    kxp = torch.empty(kxp_bytes // 4, device="cuda")
    g13 = (n, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1)
    calls["im2col"]()
    y_i2c, dw_i2c = torch.empty_like(xd), torch.empty_like(conv.weights)
    dw_ws, dw_ws_bytes = native.conv_workspace(native.OP_DW, False, g13)
    i2c = {
        "i2c_fwd": lambda: check(lib().pydtnn_hip_conv_i2c_forward(0, *g13, f32(conv.weights), f32(mat), f32(y_i2c),
                                                                   f32(conv.biases), dw_ws, dw_ws_bytes, stream_ptr()),
                                 "i2c forward"),
        "i2c_dw": lambda: check(lib().pydtnn_hip_conv_i2c_dw(0, *g13, f32(dyd), f32(mat), f32(dw_i2c), dw_ws,
                                                             dw_ws_bytes, stream_ptr()), "i2c dw"),
        "i2c_dx": lambda: check(lib().pydtnn_hip_conv_i2c_dx(0, *g13, f32(conv.weights), f32(dyd), f32(back), f32(kxp),
                                                             kxp.numel() * 4, stream_ptr()), "i2c dx"),
    }
    for name, fn in i2c.items():
        t = Timer(torch)
        for i in range(5):
            fn() if i == 0 else t(fn)
        torch.cuda.synchronize()
        extra[name + "_ms"] = round(t.median_ms(), 4)
        extra[name + "_tflops"] = round(gemm_flop / (t.median_ms() * 1e-3) / 1e12, 2)
    extra["i2c_note"] = ("explicit route at cfg2: GEMMs over the materialised (K x P) matrix; i2c_fwd excludes the "
                         "im2col pass (im2col_gbs), i2c_dx includes the col2im pass")
    del kxp, y_i2c
    # the bias -> BN(inference) -> ReLU epilogue as a stand-alone pass over y (2 * bytes(y)); fused into the
    # GEMM's store it costs no traffic at all
    ch = [torch.rand(256, device="cuda") + 0.5 for _ in range(5)]
    t3 = Timer(torch)
    for i in range(6):
        fn = lambda: ops.chan_eltwise(xd, channels=256, inner=56 * 56, bias=ch[0], bn=(ch[1], ch[2], ch[3], ch[4]),
                                      relu=True, out=back)
        fn() if i == 0 else t3(fn)
    torch.cuda.synchronize()
    extra["epilogue_gbs"] = round(2 * x.nbytes / (t3.median_ms() * 1e-3) / 1e9, 1)
    extra["epilogue_pct_hbm_peak"] = round(100 * extra["epilogue_gbs"] / HBM_PEAK_GBS, 1)
    del mat, back
    extra.update(compat_route(x, w, b, gemm_flop))
    del xd, dyd
    extra.update(f64_route(torch, gemm_flop))
    traffic, traffic_source = traffic_of_forward(fwd_launch)
    profiled = fwd_launch == TRAFFIC_PROFILE["launch"]
    roofline = {"bound": "mfma",
                "kernel": ("gemm_streamk_kernel_big_tile<256x128, PlainK4, Im2colNchwMN, EpiNchw> + streamk_fixup_kernel "
                           "(forward)") if profiled else f"the forward call's launch: {fwd_launch}",
                "achieved": round(achieved, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": traffic,
                "traffic_source": traffic_source, "launch": fwd_launch}
    workload = ("cfg2: VGG16-style 3x3 conv layer fwd+dW+db+dX, fp32 NCHW, N=64, 256->256, 56x56, stride 1, pad 1, "
                "implicit GEMM")
    return ms, step_flop / (ms * 1e-3) / 1e9, workload, roofline, extra


FP64_MFMA_PEAK_TFLOPS = 78.6


def f64_route(torch, gemm_flop, n=64):
    """The explicit route's three GEMMs of cfg2 in float64 (the reference's float64 path is im2col + a @ b),
    on the v_mfma_f64_16x16x4_f64 engine, against the 78.6 TFLOP/s float64 matrix peak."""
    from pydtnn_amd import ops
    gen = torch.Generator(device="cuda").manual_seed(0)
    p = n * 56 * 56
    w2d = torch.randn((256, 2304), device="cuda", dtype=torch.float64, generator=gen)
    cols = torch.randn((2304, p), device="cuda", dtype=torch.float64, generator=gen)
    dy_cols = torch.randn((256, p), device="cuda", dtype=torch.float64, generator=gen)
    y = torch.empty((256, p), device="cuda", dtype=torch.float64)
    dw = torch.empty((256, 2304), device="cuda", dtype=torch.float64)
    calls = {"f64_i2c_fwd": lambda: ops.matmul(w2d, cols, c=y),            # (co,K) @ (K,P)
             "f64_i2c_dw": lambda: ops.matmul(dy_cols, cols.t(), c=dw),    # (co,P) @ (P,K)
             "f64_i2c_dx_gemm": lambda: ops.matmul(w2d.t(), dy_cols, c=cols)}  # (K,co) @ (co,P)
    out = {}
    for name, fn in calls.items():
        t = Timer(torch)
        for i in range(4):
            fn() if i == 0 else t(fn)
        torch.cuda.synchronize()
        ms = t.median_ms()
        out[name + "_ms"] = round(ms, 3)
        out[name + "_tflops"] = round(gemm_flop / (ms * 1e-3) / 1e12, 2)
        out[name + "_pct_fp64_mfma_peak"] = round(100 * gemm_flop / (ms * 1e-3) / 1e12 / FP64_MFMA_PEAK_TFLOPS, 1)
    return out


def compat_route(x, w, b, gemm_flop, reps=3):
    """cfg2's forward through libconvGemm.so with host pointers, exactly as the reference's shim calls it
    (pydtnn/backends/cpu/libs/conv_gemm.py:191-205): 205 MB in and 205 MB out over PCIe per call, so the rate
    is that of the copies.  Reported beside the device-resident numbers, never as `value`."""
    import ctypes
    import numpy as np
    from pydtnn_amd import native
    lib = ctypes.CDLL(native.COMPAT_LIB_PATH)
    ac, bc = ctypes.POINTER(ctypes.c_float)(), ctypes.POINTER(ctypes.c_float)()
    lib.alloc_pack_buffs.restype = ctypes.c_int
    if lib.alloc_pack_buffs(ctypes.byref(ac), ctypes.byref(bc)) != 0:
        return {}
    n, c, h, wd = x.shape
    y = np.empty((n, 256, h, wd), np.float32)
    u, vp, none = ctypes.c_uint, (lambda a: ctypes.c_void_p(a.ctypes.data)), ctypes.c_void_p(None)

    def call():
        lib.sconvGemmNCHW(ctypes.c_char(b'N'), u(n), u(c), u(h), u(wd), u(256), u(3), u(3), u(1), u(1), u(1), u(1),
                          u(1), u(1), vp(w), vp(x), vp(y), vp(b), none, none, none, none, ctypes.c_bool(False), ac, bc)

    call()  # allocates the library's device buffers
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        call()
        times.append(time.perf_counter() - t0)
    libc = ctypes.CDLL("libc.so.6")
    libc.free(ac)
    libc.free(bc)
    best = min(times)
    return {"compat_hostptr_fwd_ms": round(best * 1e3, 2), "compat_hostptr_fwd_tflops": round(gemm_flop / best / 1e12, 2),
            "compat_hostptr_pcie_gbs": round((x.nbytes + y.nbytes) / best / 1e9, 1)}


def cpu_baseline_cfg2(sample_images=64, reps=30):
    """The reference's CPU route (im2col -> NumPy @ -> bias add -> 1023 transpose; backward likewise) restated
    by the oracle and timed on this host.  BLAS and OpenMP are both held to `cores` threads."""
    import numpy as np
    from threadpoolctl import threadpool_limits
    from oracle import cpu_ref
    from bench_configs import _cpu_cores, host_cpus
    cores = _cpu_cores()
    x, w, b, dy = make_cfg2(sample_images)
    p = cpu_ref.ConvParams(3, 3, 1, 1)
    times = []
    budget = time.perf_counter() + 25.0  # about 10 s of CPU work on the GPU box; never more than this
    with threadpool_limits(limits=cores):
        for it in range(reps + 1):
            t0 = time.perf_counter()
            y, x_cols = cpu_ref.conv2d_forward_nchw_i2c(x, w, b, p)
            cpu_ref.conv2d_backward_nchw_i2c(dy, x_cols, w, x.shape, p)
            if it > 0:
                times.append(time.perf_counter() - t0)
            del y, x_cols
            if time.perf_counter() > budget and times:
                break
    best = min(times)
    flop = 3 * 2.0 * 256 * 2304 * sample_images * 56 * 56
    return {"value": round(flop / best / 1e9, 1), "unit": "GFLOP/s", "cores": cores, "host_logical_cpus": host_cpus(),
            "kind": "port",
            "sample": f"{sample_images} of 64 images of cfg2, fwd+dW+db+dX, 1 warm-up then best of {len(times)} "
                      f"({best:.2f} s each, {sum(times):.1f} s in all); C/OpenMP im2col+col2im and NumPy(OpenBLAS) "
                      f"matmul limited to {cores} threads"}


def build_vgg16(pd, n=64, tensor_format="NCHW", **flags):
    """pydtnn/models/vgg16.py without its two Dropout(0.5) layers (the configuration has none)."""
    model = pd.Model(tensor_format=tensor_format, batch_size=n, **flags)
    return pd.models.create_vgg16_imagenet(model, dropout=False)


def run_cfg5(torch, pd, args, steps=None, warmup=None):
    import numpy as np
    np.random.seed(0)
    n = 64
    model = build_vgg16(pd, n, enable_backward_overlap=not args.one_stream)
    # the same network with every Relu layer making its own two passes (Model(enable_relu_folding=False); same
    # losses, gradients and weights bit for bit): reported beside the headline number
    np.random.seed(0)
    plain_model = build_vgg16(pd, n, enable_relu_folding=False)
    rng = np.random.default_rng(0)
    x = torch.from_numpy(rng.random((n, 3, 224, 224), dtype=np.float32)).cuda()
    labels = rng.integers(0, 1000, n)
    y_targ = torch.zeros((n, 1000), device="cuda")
    y_targ[torch.arange(n), torch.from_numpy(labels).cuda()] = 1.0
    loss_fn, opt = pd.CategoricalCrossEntropy(), pd.SGD(learning_rate=0.01, momentum=0.9)
    losses = []

    def step(timers):
        losses.append(model.train_batch(x, y_targ, loss_fn, opt))

    ms, _ = timed_steps(torch, step, steps or args.steps, warmup if warmup is not None else args.warmup)
    plain_losses, plain_opt = [], pd.SGD(learning_rate=0.01, momentum=0.9)

    def plain_step(timers):
        plain_losses.append(plain_model.train_batch(x, y_targ, loss_fn, plain_opt))

    plain_ms = None
    if not args.no_folding_extra:
        plain_ms, _ = timed_steps(torch, plain_step, steps or args.steps,
                                   warmup if warmup is not None else args.warmup)
    # ... and with the whole backward pass on one stream (Model(enable_backward_overlap=False); same bits again)
    one_stream_ms = None
    if not args.no_folding_extra:
        del plain_model
        np.random.seed(0)
        one_stream_model = build_vgg16(pd, n, enable_backward_overlap=False)
        one_stream_losses, one_stream_opt = [], pd.SGD(learning_rate=0.01, momentum=0.9)

        def one_stream_step(timers):
            one_stream_losses.append(one_stream_model.train_batch(x, y_targ, loss_fn, one_stream_opt))

        one_stream_ms, _ = timed_steps(torch, one_stream_step, steps or args.steps,
                                        warmup if warmup is not None else args.warmup)
        del one_stream_model
    # the same step in the reference's other tensor format (its default on the CPU), also beside the headline
    nhwc_ms = None
    if not args.no_folding_extra:
        np.random.seed(0)
        nhwc_model = build_vgg16(pd, n, tensor_format="NHWC")
        x_nhwc = x.permute(0, 2, 3, 1).contiguous()
        nhwc_opt = pd.SGD(learning_rate=0.01, momentum=0.9)

        def nhwc_step(timers):
            nhwc_model.train_batch(x_nhwc, y_targ, loss_fn, nhwc_opt)

        nhwc_ms, _ = timed_steps(torch, nhwc_step, steps or args.steps, warmup if warmup is not None else args.warmup)
    flop = 5929.5e9
    extra = {"vgg16_train_img_per_s": round(n / (ms * 1e-3), 1), "vgg16_ms_per_step": round(ms, 2),
             "vgg16_tflops": round(flop / (ms * 1e-3) / 1e12, 2),
             "vgg16_pct_fp32_mfma_peak": round(100 * flop / (ms * 1e-3) / 1e12 / FP32_MFMA_PEAK_TFLOPS, 2),
             "vgg16_first_last_loss": [round(float(losses[0]), 4), round(float(losses[-1]), 4)],
             "vgg16_params": int(model.nparams)}
    if plain_ms is not None:
        extra.update({"vgg16_separate_relu_img_per_s": round(n / (plain_ms * 1e-3), 1),
                      "vgg16_separate_relu_ms_per_step": round(plain_ms, 2),
                      "vgg16_separate_relu_same_losses": [float(a) for a in losses] == [float(b) for b in plain_losses]})
    if one_stream_ms is not None:
        extra.update({"vgg16_one_stream_img_per_s": round(n / (one_stream_ms * 1e-3), 1),
                      "vgg16_one_stream_ms_per_step": round(one_stream_ms, 2),
                      "vgg16_one_stream_same_losses": [float(a) for a in losses] == [float(b) for b in one_stream_losses]})
    if nhwc_ms is not None:
        extra.update({"vgg16_nhwc_train_img_per_s": round(n / (nhwc_ms * 1e-3), 1),
                      "vgg16_nhwc_ms_per_step": round(nhwc_ms, 2)})
    return ms, extra


VGG16_CONVS = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56),
               (256, 512, 28), (512, 512, 28), (512, 512, 14)]


def vgg16_conv_layers(torch, n=64, reps=5):
    """Each distinct 3x3 convolution of VGG16 alone, batch n: [ci, co, hw, GFLOP, fwd ms, dW ms, dX ms]."""
    from pydtnn_amd.conv_gemm import ConvGemm
    cg = ConvGemm()
    rows = []
    for ci, co, hw in VGG16_CONVS:
        x = torch.randn(n, ci, hw, hw, device="cuda")
        w = torch.randn(co, ci, 3, 3, device="cuda") * (2.0 / (9 * ci)) ** 0.5
        dy = torch.randn(n, co, hw, hw, device="cuda")
        dw, dx = torch.empty_like(w), torch.empty_like(x)
        kw = dict(vpadding=1, hpadding=1)
        calls = [lambda: cg.conv_gemm_nchw(w, x, **kw),
                 lambda: cg.conv_gemm_nchw(dy, x, biases=dw, trans=True, **kw),
                 lambda: cg.deconv_gemm_nchw(w, dy, dx, **kw)]
        times = []
        for fn in calls:
            fn()
            t = Timer(torch)
            for _ in range(reps):
                t(fn)
            torch.cuda.synchronize()
            times.append(round(t.mean_ms(), 4))
        rows.append([ci, co, hw, round(2.0 * co * ci * 9 * n * hw * hw / 1e9, 1)] + times)
    return rows


def main():
    global SETTLE_SECONDS
    args = parse_args()
    SETTLE_SECONDS = args.settle
    if args.gpus != 1:
        print(f"bench.py: this build runs on one GPU; --gpus {args.gpus} is not supported "
              f"(no collectives or sharding are part of it).", file=sys.stderr)
        sys.exit(2)
    import torch
    import pydtnn_amd as pd
    from pydtnn_amd import native
    native.lib()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU fallback.", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    if args.workload == "cfg2":
        ms, value, workload, roofline, extra = run_cfg2(torch, pd, args)
        unit = "GFLOP/s"
        if not args.no_vgg16:
            _, vgg = run_cfg5(torch, pd, args, steps=6, warmup=2)
            extra.update(vgg)
        if not args.no_other_configs:
            from bench_configs import other_configs_extra
            extra.update(other_configs_extra(torch, pd, timed_steps, cpu=not args.no_cpu_baseline))
    elif args.workload == "cfg5":
        ms, extra = run_cfg5(torch, pd, args)
        if args.conv_layers:
            extra["vgg16_conv_layers_ci_co_hw_gflop_fwd_dw_dx_ms"] = vgg16_conv_layers(torch)
        value, unit = 5929.5e9 / (ms * 1e-3) / 1e9, "GFLOP/s"
        workload = "cfg5: full VGG16 training step, fp32 NCHW, batch 64, 3x224x224, SGD momentum"
        roofline = {"bound": "mfma", "kernel": "whole step", "achieved": round(value / 1e3, 3),
                    "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(value / 1e3 / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
    elif args.workload == "resnet50":
        # not one of the five configurations: the whole network around cfg4's block, for kernel traces
        from bench_configs import resnet50_inference_extra
        extra = resnet50_inference_extra(torch, pd, timed_steps, steps=args.steps, warmup=args.warmup,
                                         layerwise=not args.no_folding_extra)
        ms = extra["resnet50_nhwc_fused_inference_ms"]
        value, unit = extra["resnet50_nhwc_fused_inference_tflops"] * 1e3, "GFLOP/s"
        workload = ("ResNet-50 inference, fp32 NHWC, batch 64, 3x224x224, every enable_fused_* flag on "
                    "(pydtnn/models/resnet50_imagenet.py)")
        roofline = {"bound": "mfma", "kernel": "whole network", "achieved": round(value / 1e3, 3),
                    "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(value / 1e3 / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
        args.no_cpu_baseline = True
    else:
        from bench_configs import run_other
        ms, value, unit, workload, roofline, extra = run_other(torch, pd, args, Timer, timed_steps)

    if args.copy_calibration:
        from pydtnn_amd import ops
        src = torch.ones(64 * 1024 * 1024, device="cuda")  # 256 MiB read + 256 MiB written per launch
        dst = torch.empty_like(src)
        for _ in range(3):
            ops.chan_eltwise(src, channels=1, inner=1, out=dst)
        torch.cuda.synchronize()
        del src, dst

    cpu = None
    if not args.no_cpu_baseline:
        from bench_configs import cpu_baseline_other, cpu_baseline_vgg16
        if args.workload == "cfg2":
            cpu = cpu_baseline_cfg2()
            if not args.no_vgg16:
                extra["vgg16_cpu_baseline"] = cpu_baseline_vgg16()
        elif args.workload == "cfg5":
            cpu = cpu_baseline_vgg16()
        else:
            cpu = cpu_baseline_other(args.workload)

    print(json.dumps({
        "metric": METRIC, "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": workload, "untimed_seconds_before_each_timed_region": SETTLE_SECONDS},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra}))


if __name__ == "__main__":
    main()
