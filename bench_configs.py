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


# --------------------------------------------------------------------------- CPU baselines
# The reference's CPU route (Cython im2col / im2row with OpenMP, NumPy @, separate bias / BN / ReLU passes)
# as restated by the oracle, timed on this host.  Reported beside the GPU figure, never a target.

def _cpu_cores():
    """Threads of the CPU legs: the process's share of the host (OMP_NUM_THREADS where the launcher sets it,
    otherwise every CPU the process may run on)."""
    import os
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return int(os.environ.get("OMP_NUM_THREADS", usable))


def host_cpus():
    import os
    return os.cpu_count() or 1


def _time_cpu(fn, budget_s, max_reps):
    """One warm-up, then repetitions until `budget_s` of work or `max_reps`; returns (best, reps, total)."""
    import time
    from threadpoolctl import threadpool_limits
    times = []
    with threadpool_limits(limits=_cpu_cores()):
        fn()
        stop = time.perf_counter() + budget_s
        while len(times) < max_reps and (not times or time.perf_counter() < stop):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
    return min(times), len(times), sum(times)


def _cpu_report(value, unit, what, best, reps, total):
    return {"value": round(value, 1), "unit": unit, "cores": _cpu_cores(), "host_logical_cpus": host_cpus(),
            "kind": "port",
            "sample": f"{what}, 1 warm-up then best of {reps} ({best:.3g} s each, {total:.1f} s in all); C/OpenMP "
                      f"gathers and NumPy(OpenBLAS) matmul limited to {_cpu_cores()} threads"}


def cpu_baseline_other(workload, budget_s=12.0):
    from oracle import cpu_ref
    if workload == "cfg1":
        x, w, b = make_cfg1()
        p = cpu_ref.ConvParams(3, 3, 1, 1)
        best, reps, total = _time_cpu(lambda: cpu_ref.conv2d_forward_nhwc_i2c(x, w, b, p), min(budget_s, 10.0), 2000)
        return _cpu_report(2.0 * 32 * 9 * 64 * 28 * 28 / best / 1e9, "GFLOP/s", "all 64 images of cfg1, forward", best,
                           reps, total)
    if workload == "cfg3":
        x, w, b = make_cfg3()
        p = cpu_ref.ConvParams(11, 11, 0, 0, 4, 4)

        def fwd():
            y, _ = cpu_ref.conv2d_forward_nchw_i2c(x, w, b, p)
            cpu_ref.relu(y)

        best, reps, total = _time_cpu(fwd, budget_s, 100)
        return _cpu_report(2.0 * 96 * 363 * 64 * 55 * 55 / best / 1e9, "GFLOP/s",
                           "all 64 images of cfg3, forward + bias + ReLU as separate passes", best, reps, total)
    if workload == "cfg4":
        import numpy as np
        x, ws, bns = make_cfg4()
        geoms = [cpu_ref.ConvParams(1, 1), cpu_ref.ConvParams(3, 3, 1, 1), cpu_ref.ConvParams(1, 1)]
        stats = [(mean, (1.0 / np.sqrt(var + 1e-5)).astype(np.float32), gamma, beta) for gamma, beta, mean, var in bns]

        def block():
            cur = x
            for i, (w, p, bn) in enumerate(zip(ws, geoms, stats)):
                cur, _ = cpu_ref.conv2d_forward_nhwc_i2c(cur, w, None, p)
                cur = cpu_ref.fused_epilogue(cur, "NHWC", bn=bn, relu_flag=i < 2)
            cur = cpu_ref.eltw_sum(cur, x)
            cpu_ref.relu(cur)

        best, reps, total = _time_cpu(block, budget_s, 100)
        flop = 2.0 * 64 * 56 * 56 * (256 * 64 + 576 * 64 + 64 * 256)
        return _cpu_report(flop / best / 1e9, "GFLOP/s",
                           "all 64 images of cfg4, unfused layers (conv, BN, ReLU, add as separate passes)", best, reps,
                           total)
    raise ValueError(workload)


VGG16_PLAN = [(3, 64), (64, 64), "M", (64, 128), (128, 128), "M", (128, 256), (256, 256), (256, 256), "M",
              (256, 512), (512, 512), (512, 512), "M", (512, 512), (512, 512), (512, 512), "M"]


def cpu_baseline_vgg16(sample_images=16, budget_s=14.0):
    """One VGG16 training step (forward, loss, backward, SGD with momentum) of the oracle on `sample_images`
    images.  The FC and optimizer parts do not shrink with the batch, so the rate of a sample is a lower bound
    of the full-batch rate."""
    import numpy as np
    from oracle import cpu_ref
    rng = np.random.default_rng(0)
    n = sample_images
    x0 = rng.random((n, 3, 224, 224), dtype=np.float32)
    y_targ = np.eye(1000, dtype=np.float32)[rng.integers(0, 1000, n)]
    p3 = cpu_ref.ConvParams(3, 3, 1, 1)
    params = []
    for spec in VGG16_PLAN:
        if spec != "M":
            ci, co = spec
            params.append([he_normal(rng, (co, ci, 3, 3), ci * 9), np.zeros(co, np.float32)])
    for fi, fo in [(25088, 4096), (4096, 4096), (4096, 1000)]:
        params.append([he_normal(rng, (fi, fo), fi), np.zeros(fo, np.float32)])
    velocity = [[np.zeros_like(w), np.zeros_like(b)] for w, b in params]

    def step():
        saved, cur, pi = [], x0, 0
        for spec in VGG16_PLAN:
            if spec == "M":
                shape = cur.shape
                cur, idx = cpu_ref.max_pool_2d_fwd_nchw(cur, 2, 2, 0, 0, 2, 2)
                saved.append(("pool", shape, idx))
            else:
                w, b = params[pi]
                shape = cur.shape
                cur, cols = cpu_ref.conv2d_forward_nchw_i2c(cur, w, b, p3)
                cur, mask = cpu_ref.relu(cur)
                saved.append(("conv", pi, shape, cols, mask))
                pi += 1
        flat_shape = cur.shape
        cur = cur.reshape(n, -1)
        fcs = []
        for j in range(3):
            w, b = params[pi + j]
            fcs.append(cur)
            cur = cpu_ref.fc_forward(cur, w, b)
            if j < 2:
                cur, mask = cpu_ref.relu(cur)
                fcs.append(mask)
        y = cpu_ref.softmax_forward(cur)
        _, d = cpu_ref.categorical_cross_entropy(y, y_targ, n)
        d = cpu_ref.softmax_backward(d, y)
        grads = {}
        for j in (2, 1, 0):
            if j < 2:
                d = d * fcs.pop()
            w, _ = params[pi + j]
            dw, db, d = cpu_ref.fc_backward(d, fcs.pop(), w)
            grads[pi + j] = (dw, db)
        d = d.reshape(flat_shape)
        for item in reversed(saved):
            if item[0] == "pool":
                _, shape, idx = item
                d = cpu_ref.max_pool_2d_bwd_nchw(d, idx, *shape, 2, 2, 0, 0, 2, 2)
            else:
                _, k, shape, cols, mask = item
                d = d * mask
                dw, db, d = cpu_ref.conv2d_backward_nchw_i2c(d, cols, params[k][0], shape, p3, need_dx=k > 0)
                grads[k] = (dw, db)
        for k, (dw, db) in grads.items():
            params[k][0], velocity[k][0] = cpu_ref.sgd_update(params[k][0], dw.astype(np.float32), velocity[k][0],
                                                              np.float32(0.01), np.float32(0.9))
            params[k][1], velocity[k][1] = cpu_ref.sgd_update(params[k][1], db.astype(np.float32), velocity[k][1],
                                                              np.float32(0.01), np.float32(0.9))

    best, reps, total = _time_cpu(step, budget_s, 4)
    return _cpu_report(n / best, "img/s", f"{n} of 64 images of cfg5 (one VGG16 training step; the FC and SGD parts "
                                          f"do not shrink with the sample, so this understates the full batch)",
                       best, reps, total)


def run_cfg1(torch, pd, timed_steps, steps, warmup):
    """The Conv2D layer's forward in EVALUATE_MODE: the layer prepares its call once (geometry, filter and bias bound
    in the library's plan) and, with Model(enable_memory_cache=True), keeps its output tensor between steps, as the
    reference's GPU layers do.  Beside it: the same convolution through the ConvGemm shim with every argument passed
    and a fresh output per call, and the kernel alone (HIP events around 200 launches in a row)."""
    import time
    from pydtnn_amd.conv_gemm import ConvGemm
    cg = ConvGemm()
    x, w, b = make_cfg1()
    xd, wd, bd = (torch.from_numpy(a).cuda() for a in (x, w, b))
    model = pd.Model(tensor_format="NHWC", batch_size=64, enable_memory_cache=True)
    model.mode = pd.EVALUATE_MODE
    conv = pd.Conv2D(nfilters=32, filter_shape=(3, 3), padding=1)
    conv.set_model(model)
    conv.initialize(prev_shape=(28, 28, 1))
    conv.weights, conv.biases = wd, bd
    assert conv.forward.__name__ == "_forward_nhwc_cg"
    forward = conv.forward

    def step(timers):
        forward(xd)

    ms, _ = timed_steps(torch, step, steps, warmup)

    def shim_step(timers):
        cg.conv_gemm_nhwc(wd, xd, biases_vector=bd, vpadding=1, hpadding=1)

    shim_ms, _ = timed_steps(torch, shim_step, steps, warmup)
    assert torch.equal(forward(xd), cg.conv_gemm_nhwc(wd, xd, biases_vector=bd, vpadding=1, hpadding=1))
    # the kernel alone: launches back to back between two events, so that the queue never runs dry
    reps = 200
    for _ in range(20):
        forward(xd)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(reps):
        forward(xd)
    host_us = (time.perf_counter() - t0) * 1e6 / reps     # what the launching thread spends per call
    e1.record()
    torch.cuda.synchronize()
    device_us = e0.elapsed_time(e1) * 1e3 / reps
    flop = 2.0 * 32 * 9 * 64 * 28 * 28
    nbytes = x.nbytes + w.nbytes + 64 * 28 * 28 * 32 * 4
    gbs = nbytes / (ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "conv_stream_nchw_kernel<1, 1, 0, 12, true, true>",
                "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                "traffic": None}
    workload = ("cfg1: Conv2D layer forward (EVALUATE_MODE, call prepared at initialisation, output tensor kept: "
                "Model(enable_memory_cache=True)), fp32 NHWC, N=64, 28x28x1 -> 32, 3x3, stride 1, pad 1 "
                "(launch-latency bound)")
    extra = {"bytes": nbytes, "gbs": round(gbs, 1), "shim_ms": round(shim_ms, 4),
             "host_us_per_call": round(host_us, 2), "device_us_per_call_back_to_back": round(device_us, 2)}
    return ms, flop / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, extra


def run_cfg3(torch, pd, timed_steps, steps, warmup):
    from pydtnn_amd.conv_gemm import ConvGemm
    cg = ConvGemm()
    x, w, b = make_cfg3()
    xd, wd, bd = (torch.from_numpy(a).cuda() for a in (x, w, b))

    def step(timers):
        cg.conv_gemm_nchw(wd, xd, biases_vector=bd, vstride=4, hstride=4, relu=True)

    ms, _ = timed_steps(torch, step, steps, warmup)
    flop = 2.0 * 96 * 363 * 64 * 55 * 55
    tf = flop / (ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "conv_stream_nchw_kernel<3, 23> (filter matrix in LDS, bias + ReLU in the store)",
                "achieved": round(tf, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
    workload = ("cfg3: AlexNet conv1 forward + fused bias + ReLU, fp32 NCHW, N=64, 3x227x227 -> 96, 11x11, "
                "stride 4, pad 0 (K=363)")
    return ms, flop / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, {}


CFG4_FLOP = 2.0 * 64 * 56 * 56 * (256 * 64 + 576 * 64 + 64 * 256)
# what the fused block cannot avoid moving: x read by the first convolution and again as the residual, the two
# 64-channel intermediates written and read, the output written
CFG4_MIN_BYTES = 4.0 * 64 * 56 * 56 * (256 + 64 + 64 + 64 + 64 + 256 + 256)


def run_cfg4(torch, pd, timed_steps, steps, warmup):
    x, ws, bns = make_cfg4()
    model = build_cfg4_model(pd, torch, ws, bns, fused=True)
    plain = build_cfg4_model(pd, torch, ws, bns, fused=False)
    xd = torch.from_numpy(x).cuda()
    model.evaluate_dataset_batch(xd)  # applies the fusion pass

    def step(timers):
        model.evaluate_batch(xd)

    ms, _ = timed_steps(torch, step, steps, warmup)

    def step_plain(timers):
        plain.evaluate_batch(xd)

    ms_plain, _ = timed_steps(torch, step_plain, steps, warmup)
    tf = CFG4_FLOP / (ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "the block's fused conv+BN(+ReLU)(+residual) implicit GEMMs",
                "achieved": round(tf, 3), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(tf / FP32_MFMA_PEAK_TFLOPS, 4), "traffic": None}
    extra = {"unfused_ms": round(ms_plain, 4), "fused_ms": round(ms, 4),
             "block_gbs_vs_8TBs": round(CFG4_MIN_BYTES / (ms * 1e-3) / 1e9, 1),
             "layers": [l.canonical_name for l in model.get_all_layers()]}
    workload = ("cfg4: ResNet-50 bottleneck inference, fp32 NHWC, N=64, 56x56x256: fused Conv+BN+ReLU 1x1 256->64, "
                "3x3 64->64, Conv+BN 1x1 64->256, residual add, ReLU")
    return ms, CFG4_FLOP / (ms * 1e-3) / 1e9, "GFLOP/s", workload, roofline, extra


def run_other(torch, pd, args, Timer, timed_steps):
    fn = {"cfg1": run_cfg1, "cfg3": run_cfg3, "cfg4": run_cfg4}[args.workload]
    return fn(torch, pd, timed_steps, args.steps, args.warmup)


def resnet50_inference_extra(torch, pd, timed_steps, n=64, steps=10, warmup=2, layerwise=True):
    """ResNet-50 at 224x224 (pydtnn/models/resnet50_imagenet.py), NHWC, batch n, inference through
    evaluate_dataset_batch: the fusion pass of pydtnn/model.py:294-349 with every enable_fused_* flag on, against
    the same network layer by layer.  FLOPs are those of its convolutions and FC layer (2 per multiply-add)."""
    import numpy as np
    out = {}
    x = torch.from_numpy(np.random.default_rng(0).random((n, 224, 224, 3), dtype=np.float32)).cuda()
    for key, flags in (("fused", dict(enable_fused_bn_relu=True, enable_fused_conv_relu=True, enable_fused_conv_bn=True,
                                      enable_fused_conv_bn_relu=True)), ("layerwise", {}))[:2 if layerwise else 1]:
        np.random.seed(0)
        model = pd.Model(tensor_format="NHWC", batch_size=n, **flags)
        pd.models.create_resnet50_imagenet(model)
        flop = 0.0   # counted before the fusion pass replaces the layers
        for layer in model.get_all_layers():
            if layer.canonical_name == "Conv2D":
                flop += 2.0 * layer.co * layer.ci * layer.kh * layer.kw * layer.ho * layer.wo
            elif layer.canonical_name == "FC":
                flop += 2.0 * layer.weights.shape[0] * layer.weights.shape[1]
        model.evaluate_dataset_batch(x)

        def step(timers, model=model):
            model.evaluate_batch(x)

        ms, _ = timed_steps(torch, step, steps, warmup)
        out[f"resnet50_nhwc_{key}_inference_ms"] = round(ms, 3)
        out[f"resnet50_nhwc_{key}_inference_img_per_s"] = round(n / (ms * 1e-3), 1)
        out["resnet50_gflop_per_image"] = round(flop / 1e9, 2)
        out[f"resnet50_nhwc_{key}_inference_tflops"] = round(n * flop / (ms * 1e-3) / 1e12, 1)
        del model
    return out


def other_configs_extra(torch, pd, timed_steps, cpu=True, steps=50, warmup=5):
    """cfg1, cfg3 and cfg4 for the default run's `extra`: GPU time and rate of each beside its CPU route."""
    out = {}
    configs = (("cfg1", run_cfg1, 2.0), ("cfg3", run_cfg3, 5.0), ("cfg4", run_cfg4, 5.0))
    # every GPU timing before the first CPU baseline: the worker threads of a CPU run keep spinning for a while
    # after it and slow the thread that launches kernels, which a step of one 0.13 ms kernel cannot hide
    for name, fn, _ in configs:
        ms, value, unit, _, roofline, extra = fn(torch, pd, timed_steps, steps, warmup)
        out[f"{name}_ms"] = round(ms, 4)
        out[f"{name}_gflops"] = round(value, 1)
        out[f"{name}_roofline"] = {k: roofline[k] for k in ("bound", "achieved", "peak", "unit", "frac")}
        if name == "cfg1":
            out["cfg1_shim_ms"] = extra["shim_ms"]
            out["cfg1_host_us_per_call"] = extra["host_us_per_call"]
            out["cfg1_device_us_per_call_back_to_back"] = extra["device_us_per_call_back_to_back"]
        if name == "cfg4":
            out["cfg4_unfused_ms"] = extra["unfused_ms"]
            out["cfg4_gbs_of_min_traffic"] = extra["block_gbs_vs_8TBs"]
    out.update(resnet50_inference_extra(torch, pd, timed_steps))
    if cpu:
        for name, _, budget in configs:
            out[f"{name}_cpu_baseline"] = cpu_baseline_other(name, budget)
    return out
