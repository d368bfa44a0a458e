"""GPU parity at the exact shapes the benchmark times (batch 64), for the launches whose tile / split choice
depends on the problem size.

Each of the nine distinct VGG16 convolutions runs forward, filter gradient and input gradient through the
Conv2D layer in both tensor formats; y, dw, db and dx are checked by *sampled direct convolution in float64*
(a few thousand randomly chosen elements recomputed from their defining sums on the host: no column matrix,
independent of any tiling), the pattern of pydtnn/tests/check_conv_gemm_models.py:100-167 at full size.
FC1 (64 x 25088 x 4096, split along k) is checked whole against float64.  Tolerance: the fp32 bar of the
task, max |a - b| / max |b| <= 1e-4.
"""
import numpy as np
import pytest
import torch

from gpu_util import FP32_REL_TOL, announce, assert_close, dev, host

pytestmark = pytest.mark.gpu

VGG16_CONVS = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56),
               (256, 512, 28), (512, 512, 28), (512, 512, 14)]


@pytest.fixture(scope="module")
def pd():
    import pydtnn_amd
    from pydtnn_amd import native
    native.lib()
    return pydtnn_amd


def sampled_conv3x3_check(x, w, b, dy, y, dw, db, dx, samples=2000, dw_samples=10, seed=0, relu_y=False,
                          gate_dx=None):
    """x (n,c,h,w), w (co,c,3,3), dy / y (n,co,h,w), dx like x or None: NCHW host arrays of a 3x3, pad 1, stride 1
    convolution.  Returns the largest errors relative to each result's largest magnitude.  ``relu_y``: y holds
    relu(conv + b); ``gate_dx``: a boolean array like x, dx holds the input gradient where it is True and 0
    elsewhere (the forms a training step produces when a Relu layer's work is done by its neighbours)."""
    n, c, h, wd = x.shape
    co = w.shape[0]
    rng = np.random.default_rng(seed)
    s = samples
    ni, oy, ox = rng.integers(0, n, s), rng.integers(0, h, s), rng.integers(0, wd, s)
    # borders and corners are where padding predicates live: force some samples there
    oy[: s // 8] = rng.choice([0, h - 1], s // 8)
    ox[s // 16: s // 8 + s // 16] = rng.choice([0, wd - 1], s // 8)
    ni[:16] = n - 1
    oc, ic = rng.integers(0, co, s), rng.integers(0, c, s)
    oc[:8], ic[:8] = co - 1, c - 1

    def taps(t, channels, flip):
        out = np.zeros((s, channels, 9))
        for i in range(3):
            for j in range(3):
                yy, xx = (oy + 1 - i, ox + 1 - j) if flip else (oy + i - 1, ox + j - 1)
                ok = (yy >= 0) & (yy < h) & (xx >= 0) & (xx < wd)
                out[ok, :, i * 3 + j] = t[ni[ok], :, yy[ok], xx[ok]]
        return out

    errs = {}
    # y[n,o,oy,ox] = b[o] + sum_{c,i,j} w[o,c,i,j] x[n,c,oy+i-1,ox+j-1]
    ref_y = np.einsum("sck,sck->s", taps(x, c, False), w[oc].reshape(s, c, 9).astype(np.float64)) + b[oc]
    if relu_y:
        ref_y = np.maximum(ref_y, 0.0)
    errs["y"] = float(np.max(np.abs(y[ni, oc, oy, ox] - ref_y)) / np.abs(y).max())
    if dx is not None:
        # dx[n,c,y,x] = sum_{o,i,j} w[o,c,i,j] dy[n,o,y+1-i,x+1-j]
        ref_dx = np.einsum("sok,sok->s", taps(dy, co, True),
                           w[:, ic].transpose(1, 0, 2, 3).reshape(s, co, 9).astype(np.float64))
        if gate_dx is not None:
            ref_dx = ref_dx * gate_dx[ni, ic, oy, ox]
        errs["dx"] = float(np.max(np.abs(dx[ni, ic, oy, ox] - ref_dx)) / np.abs(dx).max())
    # dw[o,c,i,j] = sum_{n,oy,ox} dy[n,o,oy,ox] x[n,c,oy+i-1,ox+j-1]
    worst = 0.0
    picks = [(co - 1, c - 1, 2, 2), (0, 0, 0, 0)] + [
        (rng.integers(0, co), rng.integers(0, c), rng.integers(0, 3), rng.integers(0, 3)) for _ in range(dw_samples)]
    for o, ci, i, j in picks:
        ys, ye = max(0, 1 - i), min(h, h + 1 - i)
        xs, xe = max(0, 1 - j), min(wd, wd + 1 - j)
        ref = np.sum(dy[:, o, ys:ye, xs:xe].astype(np.float64) * x[:, ci, ys + i - 1:ye + i - 1, xs + j - 1:xe + j - 1])
        worst = max(worst, abs(dw[o, ci, i, j] - ref))
    errs["dw"] = float(worst / np.abs(dw).max())
    ref_db = dy.sum(axis=(0, 2, 3), dtype=np.float64)
    errs["db"] = float(np.max(np.abs(db - ref_db)) / np.abs(ref_db).max())
    return errs


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
@pytest.mark.parametrize("ci,co,hw", VGG16_CONVS, ids=[f"{a}to{b}at{c}" for a, b, c in VGG16_CONVS])
def test_vgg16_convolution_at_batch_64(pd, fmt, ci, co, hw):
    announce("vgg16 conv, batch 64", fmt, ci, co, hw)
    n = 64
    gen = torch.Generator(device="cuda").manual_seed(ci * 1000 + hw)
    xd = torch.randn((n, ci, hw, hw), device="cuda", generator=gen)
    dyd = torch.randn((n, co, hw, hw), device="cuda", generator=gen)
    rng = np.random.default_rng(co + hw)
    w = (rng.standard_normal((co, ci, 3, 3)) * np.sqrt(2.0 / (ci * 9))).astype(np.float32)
    b = rng.standard_normal(co).astype(np.float32)
    model = pd.Model(tensor_format=fmt, batch_size=n)
    model.mode = pd.TRAIN_MODE
    conv = pd.Conv2D(nfilters=co, filter_shape=(3, 3), padding=1)
    conv.set_model(model)
    need_dx = ci != 3  # the first layer of the network computes no dx
    if fmt == "NCHW":
        conv.initialize(prev_shape=(ci, hw, hw), need_dx=need_dx)
        conv.weights, conv.biases = dev(w), dev(b)
        y = conv.forward(xd)
        dx = conv.backward(dyd)
        dw = conv.dw
    else:
        conv.initialize(prev_shape=(hw, hw, ci), need_dx=need_dx)
        conv.weights, conv.biases = dev(w.transpose(1, 2, 3, 0)), dev(b)
        y = conv.forward(xd.permute(0, 2, 3, 1).contiguous()).permute(0, 3, 1, 2)
        dx = conv.backward(dyd.permute(0, 2, 3, 1).contiguous())
        dx = dx.permute(0, 3, 1, 2) if dx is not None else None
        dw = conv.dw.permute(3, 0, 1, 2)
    assert conv.forward.__name__ == f"_forward_{fmt.lower()}_cg"
    assert (dx is None) == (not need_dx)
    errs = sampled_conv3x3_check(host(xd), w, b, host(dyd), host(y.contiguous()), host(dw.contiguous()),
                                 host(conv.db), host(dx.contiguous()) if dx is not None else None)
    print("   max errors relative to scale:", {k: f"{v:.2e}" for k, v in errs.items()}, flush=True)
    for k, v in errs.items():
        assert v <= FP32_REL_TOL, f"{fmt} {ci}->{co}@{hw}: {k} error {v:.3e}"


@pytest.mark.parametrize("shape", [(64, 25088, 4096), (64, 4096, 4096), (64, 4096, 1000)], ids=repr)
def test_vgg16_fc_layers_at_batch_64(pd, shape):
    """y = x W + b, dw = x^T dy, dx = dy W^T at the three FC shapes of VGG16 (the first is split along k)."""
    n, fin, fout = shape
    announce("vgg16 fc, batch 64", shape)
    rng = np.random.default_rng(fin + fout)
    x = rng.standard_normal((n, fin), dtype=np.float32)
    w = (rng.standard_normal((fin, fout), dtype=np.float32) * np.float32(np.sqrt(2.0 / fin)))
    b = rng.standard_normal(fout).astype(np.float32)
    dy = rng.standard_normal((n, fout), dtype=np.float32)
    model = pd.Model(tensor_format="NCHW", batch_size=n)
    model.mode = pd.TRAIN_MODE
    fc = pd.FC(shape=(fout,))
    fc.set_model(model)
    fc.initialize(prev_shape=(fin,))
    fc.weights, fc.biases = dev(w), dev(b)
    y = host(fc.forward(dev(x)))
    dx = host(fc.backward(dev(dy)))
    x64, w64, dy64 = x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64)
    assert_close(y, x64 @ w64 + b, what="fc y")
    assert_close(dx, dy64 @ w64.T, what="fc dx")
    assert_close(host(fc.db), dy64.sum(axis=0), tol=1e-5, what="fc db")
    # dw is (fin, fout): whole against float64 where that is cheap, a band of rows for the largest
    rows = slice(0, fin) if fin * fout <= 4096 * 4096 else slice(fin - 3000, fin)
    ref_dw = x64[:, rows].T @ dy64
    got_dw = host(fc.dw)
    assert np.max(np.abs(got_dw[rows] - ref_dw)) / np.abs(ref_dw).max() <= FP32_REL_TOL
    # the rows outside the band: column sums are linear in dw, sum_i dw[i, :] = (sum_i x[:, i])^T dy
    assert_close(got_dw.sum(axis=0, dtype=np.float64), x64.sum(axis=1) @ dy64, what="fc dw column sums")


# --------------------------------------------------------------------------- the training step as the benchmark runs it
def _vgg16_for_step(pd, fmt, **flags):
    np.random.seed(0)
    model = pd.Model(tensor_format=fmt, batch_size=64, **flags)
    return pd.models.create_vgg16_imagenet(model, dropout=False, initializer="he_normal")


def _trainable_state(model):
    """Every tensor a training step changes: (name, tensor) for weights, biases and their velocities."""
    out = []
    for layer in model.get_all_layers():
        for var in layer.grad_vars:
            out.append((f"{layer!r}.{var}", getattr(layer, var)))
            out.append((f"{layer!r}.velocity_{var}", getattr(layer, "velocity_" + var)))
    return out


def _record_convolutions(model, ids):
    """Wraps forward / backward of the named convolutions so that the tensors of the last step stay at hand:
    x (the layer's input), y (what its forward returned), dy (what its backward received), dx (what it returned)."""
    seen = {}
    for layer in model.layers:
        if layer.canonical_name != "Conv2D" or layer.id not in ids:
            continue
        rec = seen[layer.id] = {"layer": layer}

        def wrap(fwd, bwd, rec):
            def forward(x):
                rec["x"] = x
                rec["y"] = fwd(x)
                return rec["y"]

            def backward(dy):
                rec["dy"] = dy
                rec["dx"] = bwd(dy)
                return rec["dx"]
            return forward, backward

        layer.forward, layer.backward = wrap(layer.forward, layer.backward, rec)
    return seen


@pytest.mark.parametrize("fmt", ["NCHW", "NHWC"])
def test_vgg16_training_step_variants_at_batch_64(pd, fmt):
    """Two train_batch steps of VGG16 at batch 64, as bench.py runs them: the default model (a Relu layer's work
    done by the stores of its neighbours, filter gradients on a second stream), the model with every Relu layer
    making its own passes, and the model with the whole backward pass on one stream must leave bit-identical
    weights, biases and velocities in every layer.  For the default model in NCHW the folded tensors of three
    convolutions, taken from inside the second step, are recomputed on the host in float64 at sampled positions:
    y = relu(conv(x) + b), dw and db from the dy the layer received, and dx multiplied by the mask of the Relu
    below.  The pattern of pydtnn/tests/check_conv_gemm_models.py:100-167 (same model, two code paths, layer by
    layer) at the benchmark's size."""
    announce("vgg16 training step, three variants", fmt)
    n = 64
    rng = np.random.default_rng(0)
    x = torch.from_numpy(rng.random((n, 3, 224, 224), dtype=np.float32)).cuda()
    if fmt == "NHWC":
        x = x.permute(0, 2, 3, 1).contiguous()
    y_targ = torch.zeros((n, 1000), device="cuda")
    y_targ[torch.arange(n), torch.from_numpy(rng.integers(0, 1000, n)).cuda()] = 1.0
    loss_fn = pd.CategoricalCrossEntropy()
    variants = {"default": {}, "separate relu": dict(enable_relu_folding=False),
                "one stream": dict(enable_backward_overlap=False)}
    states, losses, recorded = {}, {}, None
    for name, flags in variants.items():
        announce("  variant", name)
        model = _vgg16_for_step(pd, fmt, **flags)
        opt = pd.SGD(learning_rate=0.01, momentum=0.9)
        if name == "default" and fmt == "NCHW":
            # conv1_2 (64 -> 64 at 224), conv3_2 (256 -> 256 at 56), conv5_1 (512 -> 512 at 14)
            convs = [l for l in model.layers if l.canonical_name == "Conv2D"]
            recorded = _record_convolutions(model, {convs[1].id, convs[5].id, convs[10].id})
        losses[name] = [float(model.train_batch(x, y_targ, loss_fn, opt))]
        # the parameters the second step computes with (biases are no longer zero there)
        before = {i: (host(r["layer"].weights), host(r["layer"].biases)) for i, r in (recorded or {}).items()} \
            if name == "default" else {}
        losses[name].append(float(model.train_batch(x, y_targ, loss_fn, opt)))
        torch.cuda.synchronize()
        states[name] = [(k, t.clone()) for k, t in _trainable_state(model)]
        for i, (w_before, b_before) in before.items():
            rec = recorded[i]
            layer = rec["layer"]
            announce("  sampled float64 check of", repr(layer), tuple(rec["x"].shape))
            assert layer.relu_above is not None and rec["y"].min().item() >= 0.0   # the store did the Relu above
            xh = host(rec["x"])
            gate = xh > 0 if layer.relu_below is not None else None   # ... and the dx store the Relu below
            errs = sampled_conv3x3_check(xh, w_before, b_before, host(rec["dy"]), host(rec["y"]), host(layer.dw),
                                         host(layer.db), host(rec["dx"]), relu_y=True, gate_dx=gate)
            print("   max errors relative to scale:", {k: f"{e:.2e}" for k, e in errs.items()}, flush=True)
            for k, e in errs.items():
                assert e <= FP32_REL_TOL, f"{layer!r}: {k} error {e:.3e}"
            rec.clear()
        del model
    assert losses["default"] == losses["separate relu"] == losses["one stream"], losses
    assert np.isfinite(losses["default"]).all() and losses["default"][1] != losses["default"][0]
    for name in ("separate relu", "one stream"):
        for (k, a), (k2, b) in zip(states["default"], states[name]):
            assert k == k2
            assert torch.equal(a, b), f"{fmt}: {k} differs between the default model and '{name}'"
    assert len(states["default"]) == 2 * 2 * 16   # 13 convolutions + 3 FC layers, weights and biases, + velocities
