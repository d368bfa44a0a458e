"""Workloads cfg1, cfg3 and cfg4 of the benchmark (``bench.py --workload ...``); cfg2 and cfg5 live in bench.py.

All inputs come from ``numpy.random.default_rng(0)`` and are resident in HBM before the timed region.
"""
import numpy as np

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0


def he_normal(rng, shape, fan_in):
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def make_cfg1():
    """MNIST-shaped first layer, NHWC: N=64, 28x28x1 -> 32, 3x3, stride 1, pad 1, bias zeros."""
    rng = np.random.default_rng(0)
    x = rng.random((64, 28, 28, 1), dtype=np.float32)
    w = he_normal(rng, (1, 3, 3, 32), 9)
    b = np.zeros(32, np.float32)
    return x, w, b


def make_cfg3(n=64):
    """AlexNet conv1, NCHW: N=64, 3x227x227 uint8 pixels / 255 -> 96, 11x11, stride 4, pad 0; bias + ReLU fused."""
    rng = np.random.default_rng(0)
    x = rng.integers(0, 256, (n, 3, 227, 227), dtype=np.uint8).astype(np.float32) / np.float32(255)
    w = he_normal(rng, (96, 3, 11, 11), 363)
    b = (rng.standard_normal(96) * 0.1).astype(np.float32)  # non-zero so that the epilogue is observable
    return x, w, b


def make_cfg4(n=64):
    """ResNet-50 bottleneck, NHWC, inference: 1x1 256->64, 3x3 64->64 pad 1, 1x1 64->256, BN after each, residual."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((n, 56, 56, 256), dtype=np.float32)
    ws = [he_normal(rng, (256, 1, 1, 64), 256), he_normal(rng, (64, 3, 3, 64), 576), he_normal(rng, (64, 1, 1, 256), 64)]
    bns = []
    for c in (64, 64, 256):
        gamma = rng.uniform(0.5, 1.5, c).astype(np.float32)
        beta = rng.normal(0, 0.1, c).astype(np.float32)
        mean = rng.normal(0, 0.1, c).astype(np.float32)
        var = rng.uniform(0.5, 1.5, c).astype(np.float32)
        bns.append((gamma, beta, mean, var))
    return x, ws, bns


def build_cfg4_model(pd, torch, ws, bns, fused=True):
    flags = dict(enable_fused_conv_bn_relu=True, enable_fused_conv_bn=True) if fused else {}
    model = pd.Model(tensor_format="NHWC", batch_size=64, **flags)
    model.add(pd.Input(shape=(56, 56, 256)))
    model.add(pd.AdditionBlock(
        [pd.Conv2D(nfilters=64, filter_shape=(1, 1)), pd.BatchNormalization(), pd.Relu(),
         pd.Conv2D(nfilters=64, filter_shape=(3, 3), padding=1), pd.BatchNormalization(), pd.Relu(),
         pd.Conv2D(nfilters=256, filter_shape=(1, 1)), pd.BatchNormalization()],
        []))
    model.add(pd.Relu())
    convs = [l for l in model.get_all_layers() if l.canonical_name == "Conv2D"]
    bnl = [l for l in model.get_all_layers() if l.canonical_name == "BatchNormalization"]
    for conv, w in zip(convs, ws):
        conv.weights = torch.from_numpy(w).cuda()
    for layer, (gamma, beta, mean, var) in zip(bnl, bns):
        layer.gamma, layer.beta = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
        layer.running_mean, layer.running_var = torch.from_numpy(mean).cuda(), torch.from_numpy(var).cuda()
        layer.updated_running_var = True
    return model


def run_other(torch, pd, args, Timer, timed_steps):
    from pydtnn_amd.conv_gemm import ConvGemm
    cg = ConvGemm()
    if args.workload == "cfg1":
        x, w, b = make_cfg1()
        xd, wd, bd = (torch.from_numpy(a).cuda() for a in (x, w, b))

        def step(timers):
            cg.conv_gemm_nhwc(wd, xd, biases_vector=bd, vpadding=1, hpadding=1)

        ms, _ = timed_steps(torch, step, args.steps, args.warmup)
        flop = 2.0 * 32 * 9 * 64 * 28 * 28
        nbytes = x.nbytes + w.nbytes + 64 * 28 * 28 * 32 * 4
        gbs = nbytes / (ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": "gemm_kernel<64x64, Im2rowNhwcK, FilterNhwcMN, EpiPlain>",
                    "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                    "traffic": None}
        workload = "cfg1: Conv2D forward, fp32 NHWC, N=64, 28x28x1 -> 32, 3x3, stride 1, pad 1 (launch-latency bound)"
        return ms, flop / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, {"bytes": nbytes, "gbs": round(gbs, 1)}

    if args.workload == "cfg3":
        x, w, b = make_cfg3()
        xd, wd, bd = (torch.from_numpy(a).cuda() for a in (x, w, b))

        def step(timers):
            cg.conv_gemm_nchw(wd, xd, biases_vector=bd, vstride=4, hstride=4, relu=True)

        ms, _ = timed_steps(torch, step, args.steps, args.warmup)
        flop = 2.0 * 96 * 363 * 64 * 55 * 55
        tf = flop / (ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": "gemm_kernel<128x128, PlainK, Im2colNchwMN, EpiNchw>",
                    "achieved": round(tf, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
        workload = ("cfg3: AlexNet conv1 forward + fused bias + ReLU, fp32 NCHW, N=64, 3x227x227 -> 96, 11x11, "
                    "stride 4, pad 0 (M=96 fills 75 % of a 128-row tile, K=363)")
        return ms, flop / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, {}

    x, ws, bns = make_cfg4()
    model = build_cfg4_model(pd, torch, ws, bns, fused=True)
    plain = build_cfg4_model(pd, torch, ws, bns, fused=False)
    xd = torch.from_numpy(x).cuda()
    model.evaluate_dataset_batch(xd)  # applies the fusion pass

    def step(timers):
        model.evaluate_batch(xd)

    ms, _ = timed_steps(torch, step, args.steps, args.warmup)

    def step_plain(timers):
        plain.evaluate_batch(xd)

    ms_plain, _ = timed_steps(torch, step_plain, args.steps, args.warmup)
    flop = 2.0 * 64 * 56 * 56 * (256 * 64 + 576 * 64 + 64 * 256)
    tf = flop / (ms * 1e-3) / 1e12
    nbytes = 4.0 * 64 * 56 * 56 * (256 + 64 + 64 + 64 + 64 + 256 + 256 + 256 + 256 + 256)
    roofline = {"bound": "mfma", "kernel": "3 fused conv+BN(+ReLU) implicit GEMMs + residual add + ReLU",
                "achieved": round(tf, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
    extra = {"unfused_ms": round(ms_plain, 4), "fused_ms": round(ms, 4),
             "block_gbs_vs_8TBs": round(nbytes / (ms * 1e-3) / 1e9, 1),
             "layers": [l.canonical_name for l in model.get_all_layers()]}
    workload = ("cfg4: ResNet-50 bottleneck inference, fp32 NHWC, N=64, 56x56x256: fused Conv+BN+ReLU 1x1 256->64, "
                "3x3 64->64, Conv+BN 1x1 64->256, residual add, ReLU")
    return ms, flop / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, extra
