"""Minimal ``Model``: what the conv-as-GEMM layers need from pydtnn/model.py and nothing else.

Kept from the reference: keyword flags readable as attributes (``tensor_format``, ``dtype``,
``batch_size``, ``enable_conv_gemm``, ``enable_fused_bn_relu`` / ``_conv_relu`` / ``_conv_bn`` /
``_conv_bn_relu``; pydtnn/parser.py:64-79, :131), ``mode``, ``matmul``, a no-op ``tracer``,
``add`` with ``need_dx = layer.id > 1`` (pydtnn/model.py:268-283), the layer-fusion rewrite
(pydtnn/model.py:294-349) and the single-process forward / backward / update loop
(pydtnn/model.py:450-492, :623-644).  Datasets, MPI, checkpoints, schedulers and the CLI are not
part of this build.
"""
import contextlib

import numpy as np
import torch

from . import layers as L
from . import ops
from .best_of import BestOf
from .tracers import (PYDTNN_MDL_BACKWARD, PYDTNN_MDL_EVENT, PYDTNN_MDL_EVENTS, PYDTNN_MDL_FORWARD,
                      PYDTNN_MDL_UPDATE_DW, NullTracer)
from .layers import EVALUATE_MODE, TRAIN_MODE, UNSPECIFIED_MODE
from .utils import PYDTNN_TENSOR_FORMAT_NCHW, PYDTNN_TENSOR_FORMAT_NHWC


# The second stream of enable_backward_overlap, one per device for the whole process: the scratch buffers of the
# library binding are kept per (device, stream), so models that come and go must not each bring a stream of their own.
_SIDE_STREAMS = {}


def _side_stream(device):
    side = _SIDE_STREAMS.get(device.index)
    if side is None:
        side = _SIDE_STREAMS[device.index] = torch.cuda.Stream(device=device)     # default priority
    return side


def _layer_id_generator():
    current_layer_id = 0
    while True:
        yield current_layer_id
        current_layer_id += 1


_DEFAULTS = dict(
    batch_size=64,
    tensor_format="AUTO",
    enable_conv_gemm=True,   # the implicit-GEMM path is always available on this backend
    enable_conv_winograd=False,
    enable_best_of=False,
    enable_memory_cache=False,
    enable_fused_bn_relu=False,
    enable_fused_conv_relu=False,
    enable_fused_conv_bn=False,
    enable_fused_conv_bn_relu=False,
    # Not a reference flag.  Inside train_batch a Relu layer of the top-level sequence is computed by the stores
    # of its neighbours (the convolution before it, the convolution or pooling layer after it) instead of by
    # two passes of its own.  Losses, gradients, masks and updated weights are bit-identical either way; what
    # changes is visible only between the layers of that loop (the convolution hands the Relu layer a tensor it
    # has already rectified, the layer above the Relu a dx already multiplied by the mask), and a layer's
    # forward / backward called outside train_batch never does it.  False restores the separate passes.
    enable_relu_folding=True,
    # Not a reference flag.  Inside train_batch the filter / weight and bias gradients of a Conv2D or FC layer are
    # enqueued on a second stream (default priority) while the layer's input gradient, and the layers below, go on
    # with the caller's stream; the weight updates wait for both.  Same kernels and bit-identical results: only
    # their order on the device changes, so that one kernel's last, partly idle round of workgroups is filled by
    # the other's.  False keeps everything on the caller's stream.
    enable_backward_overlap=True,
)


class Model:

    def __init__(self, dtype=torch.float32, **kwargs):
        unknown = set(kwargs) - set(_DEFAULTS)
        if unknown:
            raise TypeError(f"unknown Model flags: {sorted(unknown)}")
        self.kwargs = dict(_DEFAULTS)
        self.kwargs.update(kwargs)
        if isinstance(dtype, str):
            dtype = {"float32": torch.float32, "float64": torch.float64}[dtype]
        if dtype not in (torch.float32, torch.float64):
            raise ValueError("models compute in float32 or float64")
        self.dtype = dtype
        if dtype == torch.float64:
            # libconvGemm is float32 only (pydtnn/backends/cpu/libs/conv_gemm.py:101-107): a float64 model takes
            # the explicit im2col / im2row + GEMM route, as it does in the reference
            if kwargs.get("enable_conv_gemm"):
                raise ValueError("the implicit ConvGemm route is float32 only; a float64 model uses the explicit one")
            self.kwargs["enable_conv_gemm"] = False
        self.tracer = NullTracer()
        self.layers = []
        self.layer_id = _layer_id_generator()
        self.matmul = ops.matmul
        self.nparams = 0
        self.rank, self.nprocs, self.comm = 0, 1, None
        self.mode = UNSPECIFIED_MODE
        # pydtnn/model.py:207-215: AUTO resolves to NCHW on a GPU backend
        fmt = self.kwargs["tensor_format"]
        self.tensor_format = PYDTNN_TENSOR_FORMAT_NHWC if fmt == "NHWC" else PYDTNN_TENSOR_FORMAT_NCHW
        self.batch_size = self.kwargs["batch_size"]
        self._fused = False
        self.stepping = False  # True while train_batch runs its own forward / backward loops
        self._overlap_min_elements = 1 << 16
        self._side_used = set()  # second streams this step has put work on and not yet waited for
        self._side_launches = 0  # bodies sent to a second stream so far
        # pydtnn/model.py:216-218: without the flag every BestOf just calls its first alternative
        BestOf.use_always_the_first_alternative(not self.kwargs["enable_best_of"])

    def __getattr__(self, item):
        try:
            return self.__dict__["kwargs"][item]
        except KeyError:
            raise AttributeError(f"'Model' object has no attribute '{item}'") from None

    # ------------------------------------------------------------------ construction
    def add(self, layer):
        layer.set_model(self)
        need_dx = layer.id > 1
        prev = self.layers[-1] if self.layers else None
        prev_shape = prev.shape if layer.id > 0 else ()
        layer.initialize(prev_shape, need_dx)
        self.nparams += layer.nparams
        self.layers.append(layer)
        if self.kwargs["enable_relu_folding"]:
            self._link_relu_neighbours(prev, layer)
        if layer.act:
            self.add(layer.act())

    @staticmethod
    def _link_relu_neighbours(prev, layer):
        """Tells a convolution which Relu consumes its output, and a convolution / pooling layer which Relu
        produced its input, so that their cg kernels can do that Relu's work in TRAIN_MODE.  Only layers of
        the top-level sequence are linked: there each output has exactly one consumer."""
        if type(layer) is L.Relu and type(prev) is L.Conv2D:
            prev.relu_above = layer
        elif type(prev) is L.Relu and type(layer) in (L.Conv2D, L.MaxPool2D):
            layer.relu_below = prev

    def get_all_layers(self, from_layers=None):
        if from_layers is None:
            from_layers = self.layers
        out = []
        for layer in from_layers:
            out.append(layer)
            out += self.get_all_layers(layer.children)
        return out

    # ------------------------------------------------------------------ fusion (pydtnn/model.py:294-349)
    def apply_layer_fusion(self, bn_relu=None, conv_relu=None, conv_bn=None, conv_bn_relu=None):
        """Rewrites [Conv2D, BatchNormalization, Relu] runs into fused inference layers.  Flags default to
        the model's ``enable_fused_*`` settings.  As in the reference a convolution is only fused when its
        installed forward is one the fused class implements (the ``cg`` variants, never ``i2c``)."""
        bn_relu = self.enable_fused_bn_relu if bn_relu is None else bn_relu
        conv_relu = self.enable_fused_conv_relu if conv_relu is None else conv_relu
        conv_bn = self.enable_fused_conv_bn if conv_bn is None else conv_bn
        conv_bn_relu = self.enable_fused_conv_bn_relu if conv_bn_relu is None else conv_bn_relu

        def fusable(conv, cls):
            # pydtnn/model.py:313, :330: the convolution's installed forward must be one the fused class has
            name = conv.forward.__name__
            return name.endswith("_cg") and hasattr(cls, name)

        def fuse(layers):
            fused = []
            for i, curr in enumerate(layers):
                if curr.is_block_layer:
                    for j, p in enumerate(curr.paths):
                        curr.paths[j] = fuse(p)
                elif conv_bn_relu and len(fused) > 1 and curr.canonical_name == "Relu" and \
                        fused[-1].canonical_name == "BatchNormalization" and fused[-2].canonical_name == "Conv2D":
                    cls = L.Conv2DBatchNormalizationRelu
                    if fusable(fused[-2], cls):
                        bn_layer = fused.pop()
                        cv_layer = fused.pop()
                        curr = cls(from_parent=cv_layer, from_parent2=bn_layer)
                        curr.initialize(from_parent_dict=cv_layer.__dict__)
                elif (conv_relu or conv_bn) and len(fused) > 0 and \
                        (curr.canonical_name == "Relu" or curr.canonical_name == "BatchNormalization") and \
                        fused[-1].canonical_name == "Conv2D" and \
                        not (conv_bn_relu and i + 1 < len(layers) and layers[i + 1].canonical_name == "Relu"):
                    # as in the reference, either flag enables both the conv+ReLU and the conv+BN rewrite
                    cls = L.Conv2DRelu if curr.canonical_name == "Relu" else L.Conv2DBatchNormalization
                    if fusable(fused[-1], cls):
                        prev = fused.pop()
                        curr = cls(from_parent=prev, from_parent2=curr)
                        curr.initialize(from_parent_dict=prev.__dict__)
                elif bn_relu and len(fused) > 0 and curr.canonical_name == "Relu" and \
                        fused[-1].canonical_name == "BatchNormalization":
                    prev = fused.pop()
                    curr = L.BatchNormalizationRelu(from_parent=prev)
                fused.append(curr)
            return fused

        def link_blocks(layers):
            # an addition block whose sum is made by the last convolution of a path (AdditionBlock.forward)
            # can also do the Relu layer that consumes its output
            for i, layer in enumerate(layers):
                if layer.is_block_layer:
                    nxt = layers[i + 1] if i + 1 < len(layers) else None
                    layer.relu_above = nxt if type(nxt) is L.Relu else None
                    for p in layer.paths:
                        link_blocks(p)

        if bn_relu or conv_relu or conv_bn or conv_bn_relu:
            self.layers = fuse(self.layers)
            self._fused = True
            if conv_relu or conv_bn or conv_bn_relu:
                link_blocks(self.layers)

    # ------------------------------------------------------------------ loops
    def train_batch(self, x, y_targ, loss_func, optimizer, global_batch_size=None):
        """One pass of pydtnn/model.py:450-492 (blocking path, one process): forward, loss, backward, update."""
        if self._fused:
            raise RuntimeError("Fused layers cannot be used in training mode!")
        self.mode = TRAIN_MODE
        if global_batch_size is None:
            global_batch_size = x.shape[0]
        emit = self.tracer.emit_event
        self.stepping = True
        try:
            for i in range(1, len(self.layers)):
                emit(PYDTNN_MDL_EVENT, self.layers[i].id * PYDTNN_MDL_EVENTS + PYDTNN_MDL_FORWARD)
                x = self.layers[i].forward(x)
                emit(PYDTNN_MDL_EVENT, 0)
            loss, dx = loss_func(x, y_targ, global_batch_size)
            for i in range(len(self.layers) - 1, 0, -1):
                emit(PYDTNN_MDL_EVENT, self.layers[i].id * PYDTNN_MDL_EVENTS + PYDTNN_MDL_BACKWARD)
                dx = self.layers[i].backward(dx)
                emit(PYDTNN_MDL_EVENT, 0)
        except BaseException:
            self._join_side_stream()
            raise
        finally:
            self.stepping = False
        # each layer's update waits for that layer's gradients only (Layer.update_weights), so the updates of the
        # upper layers run while the second stream still works on the filter gradients of the lowest ones
        try:
            for i in range(len(self.layers) - 1, 0, -1):
                self.layers[i].reduce_weights_sync()
                emit(PYDTNN_MDL_EVENT, self.layers[i].id * PYDTNN_MDL_EVENTS + PYDTNN_MDL_UPDATE_DW)
                self.layers[i].update_weights(optimizer)
                emit(PYDTNN_MDL_EVENT, 0)
        finally:
            self._join_side_stream()
        return loss

    @contextlib.contextmanager
    def beside_backward(self, layer, *tensors):
        """Inside train_batch with ``enable_backward_overlap``: the body's work (the gradients of ``layer``'s
        variables) goes to the model's second stream, after everything enqueued so far on the caller's, and
        ``layer.grads_ready`` is the event that marks its end; ``tensors`` (what the body reads) are marked as in
        use by that stream, so the allocator cannot hand their memory out before it has read them.
        Otherwise, and for small problems (under 2^16 elements read: nothing to overlap but launches), the body
        runs in place."""
        if not (self.stepping and self.kwargs["enable_backward_overlap"] and tensors and tensors[0].is_cuda
                and sum(t.numel() for t in tensors) >= self._overlap_min_elements):
            yield
            return
        device = tensors[0].device
        side = _side_stream(device)
        side.wait_stream(torch.cuda.current_stream(device))
        self._side_used.add(side)
        self._side_launches += 1
        for t in tensors:
            # the allocator hands the tensor's memory out again only after the second stream has passed this point,
            # so the tensor itself can be dropped as soon as the layers are done with it
            t.record_stream(side)
        with torch.cuda.stream(side):
            yield
            layer.grads_ready = torch.cuda.Event()
            layer.grads_ready.record(side)

    def _join_side_stream(self):
        for side in self._side_used:
            torch.cuda.current_stream(side.device).wait_stream(side)
        self._side_used.clear()

    def evaluate_batch(self, x):
        """Forward pass of pydtnn/model.py:623-644."""
        self.mode = EVALUATE_MODE
        emit = self.tracer.emit_event
        for i in range(1, len(self.layers)):
            emit(PYDTNN_MDL_EVENT, self.layers[i].id * PYDTNN_MDL_EVENTS + PYDTNN_MDL_FORWARD)
            x = self.layers[i].forward(x)
            emit(PYDTNN_MDL_EVENT, 0)
        return x

    def set_tracer(self, tracer):
        """Installs a tracer (pydtnn_amd.tracers) and names its events after this model's layers."""
        self.tracer = tracer
        tracer.define_event_types(self)

    def evaluate_dataset_batch(self, x):
        """pydtnn/model.py:653-667: the fusion pass runs once, on the first evaluation."""
        if not self._fused:
            self.apply_layer_fusion()
        return self.evaluate_batch(x)


    # ------------------------------------------------------------------ weights on disk (pydtnn/model.py:351-387)
    def _walk_trainable(self, layers, prev=None):
        """Yields (layer, variable names, layer before it in its sequence) in the reference's order: block
        layers are entered path by path, and only their children carry variables."""
        for layer in layers:
            name = layer.canonical_name
            if name in ["AdditionBlock", "ConcatenationBlock"]:
                for path in layer.paths:
                    yield from self._walk_trainable(path, prev)
            else:
                keys = [g for g in layer.grad_vars] + \
                       (["running_var", "running_mean"] if name == "BatchNormalization" else [])
                yield layer, keys, prev
            prev = layer

    @staticmethod
    def _file_tensor_format(pairs, d):
        """The tensor format of the model that wrote ``d``, read off the first convolution whose filter shape
        tells the two layouts apart ((co,ci,kh,kw) against (ci,kh,kw,co)); None if no filter does."""
        for layer, keys, _ in pairs:
            base = f"{layer.id}_{layer.canonical_name}_weights"
            if layer.canonical_name != "Conv2D" or base not in d:
                continue
            co, ci, kh, kw = layer.co, layer.ci, layer.kh, layer.kw
            nchw, nhwc = (co, ci, kh, kw), (ci, kh, kw, co)
            if nchw != nhwc and tuple(d[base].shape) in (nchw, nhwc):
                return "NCHW" if tuple(d[base].shape) == nchw else "NHWC"
        return None

    def _to_model_format(self, layer, key, ary, prev, file_format):
        """An array written by a model in ``file_format`` as this model's layout wants it.  Filters go between
        (ci,kh,kw,co) and (co,ci,kh,kw) as pydtnn/tests/check_tensor_format_models.py:70-71 does
        (``transpose(3, 0, 1, 2)`` towards NCHW); the rows of an FC layer that follows the Flatten of an image
        follow the flattening order of that image, (h,w,c) or (c,h,w)."""
        mine = "NCHW" if self.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW else "NHWC"
        if file_format is None or file_format == mine or key != "weights":
            return ary
        if layer.canonical_name == "Conv2D":
            return ary.transpose(3, 0, 1, 2) if mine == "NCHW" else ary.transpose(1, 2, 3, 0)
        if layer.canonical_name == "FC" and prev is not None and prev.canonical_name == "Flatten" and \
                len(prev.prev_shape) == 3:
            from .utils import decode_tensor
            h, w, c = decode_tensor(prev.prev_shape, self.tensor_format)
            if mine == "NCHW":   # rows (h,w,c) -> (c,h,w)
                return ary.reshape(h, w, c, -1).transpose(2, 0, 1, 3).reshape(ary.shape)
            return ary.reshape(c, h, w, -1).transpose(1, 2, 0, 3).reshape(ary.shape)
        return ary

    def load_store_path(self, layers, d, mode, tensor_format=None):
        """Moves every trainable tensor, plus the running statistics of BatchNormalization, between the
        layers and the dictionary ``d`` under the reference's key ``"{layer.id}_{canonical_name}_{variable}"``
        (block layers are walked path by path).  Stored arrays keep the in-memory layout of the model's
        tensor format, as in the reference.  On load, ``tensor_format`` names the format of the model that
        wrote ``d`` when it differs from this model's; without it the format is read off the filter shapes."""
        pairs = list(self._walk_trainable(layers))
        if mode == "load" and tensor_format is None:
            tensor_format = self._file_tensor_format(pairs, d)
        for layer, keys, prev in pairs:
            name = layer.canonical_name
            if name == "BatchNormalization":
                layer.updated_running_var = True
            for key in keys:
                base = f"{layer.id}_{name}_{key}"
                if mode == "load":
                    if base not in d:
                        print(f"Could not find '{base}' for layer '{name}' in file!")
                        continue
                    ary = self._to_model_format(layer, key, np.asarray(d[base]), prev, tensor_format)
                    current = getattr(layer, key, None)
                    if current is not None and tuple(ary.shape) != tuple(current.shape):
                        raise ValueError(f"'{base}' has shape {tuple(ary.shape)}, the layer expects "
                                         f"{tuple(current.shape)}")
                    setattr(layer, key, torch.from_numpy(np.ascontiguousarray(ary)).to(self.dtype).cuda())
                elif mode == "store":
                    d[base] = getattr(layer, key).detach().cpu().numpy()

    def load_weights_and_bias(self, filename, tensor_format=None):
        d = np.load(filename)
        self.load_store_path(self.layers, d, "load", tensor_format)

    def store_weights_and_bias(self, filename):
        d = {}
        self.load_store_path(self.layers, d, "store")
        np.savez_compressed(filename, **d)


# --------------------------------------------------------------------------- loss and optimizer
class CategoricalCrossEntropy:
    """pydtnn/backends/cpu/losses/categorical_cross_entropy_cpu.py:26-35.  Returns (loss tensor, dx)."""

    def __init__(self, eps=1e-8):
        self.eps = eps

    def __call__(self, y_pred, y_targ, global_batch_size):
        return ops.categorical_cross_entropy(y_pred, y_targ, global_batch_size, self.eps)


class SGD:
    """pydtnn/optimizers/sgd.py + pydtnn/backends/cpu/optimizers/sgd_cpu.py:26-41"""

    def __init__(self, learning_rate=1e-2, momentum=0.9, nesterov=False, decay=0.0):
        self.learning_rate = learning_rate
        self.momentum = momentum
        self.nesterov = nesterov
        self.decay = decay

    def update(self, layer):
        triples = []
        for w_, dw_ in layer.grad_vars.items():
            w, dw = getattr(layer, w_), getattr(layer, dw_)
            velocity = getattr(layer, "velocity_%s" % w_, None)
            if velocity is None:
                velocity = torch.zeros_like(w)
                setattr(layer, "velocity_%s" % w_, velocity)
            triples.append((w, dw.reshape(w.shape).contiguous(), velocity))
        if triples:   # the layer's variables in one launch
            ops.sgd_momentum_multi(triples, self.learning_rate, self.momentum, self.decay, self.nesterov)
