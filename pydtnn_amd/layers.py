"""Layer classes with PyDTNN's layer protocol, backed by the MI355X kernels.

Constructor arguments, attribute names (``weights``, ``biases``, ``dw``, ``db``, ``x_cols`` /
``x_rows`` / ``cg_x``, ``need_dx``, ``grad_vars``, ``shape`` ...), the ``initialize`` /
``forward`` / ``backward`` protocol and the error behaviour mirror the reference's frontend
(pydtnn/layers/*.py) and CPU backend (pydtnn/backends/cpu/layers/*.py); tensors are
``torch.Tensor`` on the GPU.  ``Conv2D.initialize`` selects the ``i2c`` (explicit im2col + GEMM)
or ``cg`` (implicit GEMM, fused epilogue) variant exactly as
pydtnn/backends/cpu/layers/conv_2d_cpu.py:89-143 does and installs it as ``self.forward`` /
``self.backward``, so the fusion pass in ``model.py`` can test ``forward.__name__`` the way the
reference does.
"""
import numpy as np
import torch

from . import ops
from .best_of import BestOf
from . import tracers as ev
from .conv_gemm import ConvGemm, PreparedForward
from .utils import PYDTNN_TENSOR_FORMAT_NCHW, decode_tensor, encode_tensor

EVALUATE_MODE, TRAIN_MODE, UNSPECIFIED_MODE = (0, 1, 2)  # pydtnn/model.py:56


# --------------------------------------------------------------------------- initializers
# Same names and scaling rules as pydtnn/initializers/__init__.py:28-79 (fans computed from
# shape[0], shape[1] and the trailing receptive field).  Drawn with NumPy on the host, then
# uploaded.  The normal variants use a plain normal instead of SciPy's truncated normal: random
# streams are not part of the parity contract.
def _compute_fans(shape):
    if len(shape) == 2:
        return shape[0], shape[1]
    if len(shape) > 2:
        receptive_field = int(np.prod(shape[2:]))
        return shape[1] * receptive_field, shape[0] * receptive_field
    raise ValueError("The length of 'shape' must be greater or equal to 2")


def _generate_distribution(shape, scale, mode, distribution):
    fan_in, fan_out = _compute_fans(shape)
    if mode == "fan_in":
        scale /= max(1., fan_in)
    elif mode == "fan_out":
        scale /= max(1., fan_out)
    else:
        scale /= max(1., float(fan_in + fan_out) / 2)
    if distribution == "normal":
        x = np.random.normal(0.0, np.sqrt(scale), shape)
    else:
        limit = np.sqrt(3. * scale)
        x = np.random.uniform(-limit, limit, shape)
    return torch.from_numpy(x.astype(np.float32)).cuda()


initializers = {
    "glorot_uniform": lambda shape: _generate_distribution(shape, 1.0, "fan_avg", "uniform"),
    "glorot_normal": lambda shape: _generate_distribution(shape, 1.0, "fan_avg", "normal"),
    "he_uniform": lambda shape: _generate_distribution(shape, 2.0, "fan_in", "uniform"),
    "he_normal": lambda shape: _generate_distribution(shape, 2.0, "fan_in", "normal"),
    "lecun_uniform": lambda shape: _generate_distribution(shape, 1.0, "fan_in", "uniform"),
    "lecun_normal": lambda shape: _generate_distribution(shape, 1.0, "fan_in", "normal"),
    "zeros": lambda shape: torch.zeros(tuple(shape), dtype=torch.float32, device="cuda"),
    "ones": lambda shape: torch.ones(tuple(shape), dtype=torch.float32, device="cuda"),
}


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


# --------------------------------------------------------------------------- base class
class Layer:
    """pydtnn/layers/layer_and_activation_base.py:25-106"""

    def __init__(self, shape=()):
        self.nparams = 0
        self.shape = shape
        self.weights = None
        self.biases = None
        self.act = None
        self.grad_vars = {}
        self.fwd_time = np.zeros((4,), dtype=np.float32)
        self.bwd_time = np.zeros((4,), dtype=np.float32)
        self.paths = []
        self.need_dx = True
        self.id = None
        self.model = None
        self.prev_shape = None
        self.is_block_layer = False
        # set by Model.add unless ReLU folding is disabled (see Relu)
        self.relu_above = None
        self.relu_below = None

    @property
    def canonical_name(self):
        return type(self).__name__

    @property
    def _id_prefix(self):
        """pydtnn/layers/layer_and_activation_base.py:46-60: the id padded to the width of the model's last id."""
        model = getattr(self, "model", None)
        if self.id is None or model is None:
            return ""
        try:
            last = model.layers[-1]
        except IndexError:
            width = 1
        else:
            last_id = last.children[-1].id if len(last.children) else last.id
            width = len(str(last_id))
        return "{:0{width}d}_".format(self.id, width=width)

    @property
    def canonical_name_with_id(self):
        """pydtnn/layers/layer.py:32-34"""
        return f"{self._id_prefix}{self.canonical_name}"

    def __repr__(self):
        return f"{self.id if self.id is not None else '?'}_{type(self).__name__}"

    def set_model(self, parent_model):
        self.model = parent_model
        self.id = next(self.model.layer_id)

    # The neighbours do a Relu layer's work only inside the model's own training step, where the Relu layer is
    # known to be the next consumer; a forward / backward called by hand computes what the reference's does.
    def _folds_relu_above(self):
        return self.relu_above is not None and self.model.mode == TRAIN_MODE and self.model.stepping

    def _gate_below(self, dx_shape):
        if self.relu_below is None or not self.model.stepping:
            return None
        return self.relu_below.gate_for(dx_shape)

    def initialize(self, prev_shape, need_dx=True):
        self.prev_shape = prev_shape
        self.need_dx = need_dx

    def forward(self, x):
        raise NotImplementedError

    def backward(self, dy):
        raise NotImplementedError

    # Single GPU: the gradient all-reduce hooks of pydtnn/backends/cpu/layers/layer_cpu.py:38-63 have nothing to do.
    def reduce_weights_async(self):
        pass

    def wait_allreduce_async(self):
        pass

    def reduce_weights_sync(self):
        pass

    @property
    def children(self):
        children = []
        for path in self.paths:
            children += [layer for layer in path]
        return children

    def update_weights(self, optimizer):
        ready = self.__dict__.pop("grads_ready", None)   # set when the gradients were computed on another stream
        if ready is not None:
            torch.cuda.current_stream().wait_event(ready)
        optimizer.update(self)


class Input(Layer):
    """pydtnn/layers/input.py: only carries the per-sample shape (given as (h, w, c))."""

    def __init__(self, shape=(1,)):
        super().__init__(shape)

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = encode_tensor(self.shape, self.model.tensor_format)


# --------------------------------------------------------------------------- activations
class Relu(Layer):
    """pydtnn/backends/cpu/activations/relu_cpu.py:25-40.

    Inside ``Model.train_batch`` (unless ``Model(enable_relu_folding=False)``) the neighbours do this layer's work
    in their own kernels: a convolution below hands over ``(y, mask)`` already rectified (``take_folded``), and the
    layer above announces a dy it has already multiplied by the mask (``take_gated``).  Both are recognised by
    the identity of the tensor passed to forward / backward, so any other caller gets the plain computation."""

    def __init__(self, shape=(1,)):
        super().__init__(shape)
        self.mask = None
        self.y = None
        self._folded = None
        self._gated = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = prev_shape

    def take_folded(self, y, mask):
        self._folded = (y, mask)

    def take_gated(self, dx):
        self._gated = dx

    def forward(self, x):
        folded, self._folded = self._folded, None
        if folded is not None and folded[0] is x:
            self.y, self.mask = folded
            return x
        train = self.model.mode == TRAIN_MODE
        self.y, mask = ops.relu(x, with_mask=train)
        if train:
            self.mask = mask
        return self.y

    def backward(self, dy):
        gated, self._gated = self._gated, None
        if self.need_dx:
            if gated is not None and gated is dy:
                return dy
            return ops.relu_backward(dy, self.mask)

    def gate_for(self, dx_shape):
        """The mask the layer above may apply to its dx, or None."""
        if self.need_dx and self.mask is not None and tuple(self.mask.shape) == tuple(dx_shape):
            return self.mask
        return None


class Softmax(Layer):
    """pydtnn/backends/cpu/activations/softmax_cpu.py:25-39 (a (batch, classes) matrix)."""

    def __init__(self, shape=(1,)):
        super().__init__(shape)
        self.y = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = prev_shape

    def forward(self, x):
        self.y = ops.softmax(x)
        return self.y

    def backward(self, dy):
        if self.need_dx:
            return ops.softmax_backward(dy, self.y)


activations = {"relu": Relu, "softmax": Softmax}


# --------------------------------------------------------------------------- Conv2D
class Conv2D(Layer):
    """Frontend pydtnn/layers/conv_2d.py:29-78 + backend pydtnn/backends/cpu/layers/conv_2d_cpu.py:51-510."""

    def __init__(self, nfilters=1, filter_shape=(3, 3), grouping=None, padding=0, stride=1,
                 dilation=1, activation="", use_bias=True, weights_initializer="glorot_uniform",
                 biases_initializer="zeros"):
        super().__init__()
        self.co = nfilters
        self.filter_shape = filter_shape
        self.grouping = grouping
        self.padding = padding
        self.stride = stride
        self.dilation = dilation
        self.vpadding, self.hpadding = _pair(padding)
        self.vstride, self.hstride = _pair(stride)
        self.vdilation, self.hdilation = _pair(dilation)
        self.act = activations.get(activation, None)
        self.use_bias = use_bias
        self.weights_initializer = initializers[weights_initializer]
        self.biases_initializer = initializers[biases_initializer]
        self.grad_vars = {"weights": "dw"}
        if self.use_bias:
            self.grad_vars["biases"] = "db"
        self.debug = False
        self.ci = self.hi = self.wi = self.kh = self.kw = self.ho = self.wo = 0
        self.weights_shape = None
        self.cg = None
        self.x_cols = self.x_rows = self.cg_x = None
        self.dw = self.db = None
        self._prepared = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.hi, self.wi, self.ci = decode_tensor(prev_shape, self.model.tensor_format)
        self.kh, self.kw = self.filter_shape
        if self.grouping in ("depthwise", "pointwise"):
            # pydtnn/backends/cpu/layers/conv_2d_cpu.py:245-249, :515-519 raise the same way for the variants
            # the reference does not implement; grouped convolutions are outside the conv-as-GEMM path here.
            raise NotImplementedError(f"grouping='{self.grouping}' is not implemented on this backend")
        if self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
            self.weights_shape = (self.co, self.ci, *self.filter_shape)
        else:
            self.weights_shape = (self.ci, *self.filter_shape, self.co)
        self.ho = (self.hi + 2 * self.vpadding - self.vdilation * (self.kh - 1) - 1) // self.vstride + 1
        self.wo = (self.wi + 2 * self.hpadding - self.hdilation * (self.kw - 1) - 1) // self.hstride + 1
        self.shape = encode_tensor((self.ho, self.wo, self.co), self.model.tensor_format)
        self.nparams = int(np.prod(self.weights_shape)) + (self.co if self.use_bias else 0)
        self.weights = self.weights_initializer(self.weights_shape).to(self.model.dtype)
        if self.use_bias:
            self.biases = self.biases_initializer((self.co,)).to(self.model.dtype)
        if self.model.enable_conv_gemm:
            self.cg = ConvGemm(dtype=self.model.dtype, debug=self.debug, parent_layer=self)
        variant = "cg" if self.model.enable_conv_gemm else "i2c"  # conv_2d_cpu.py:89, :139-140
        if getattr(self.model, "enable_best_of", False):
            # conv_2d_cpu.py:95-130: the explicit and the implicit route race per problem size, forward alone
            # in EVALUATE_MODE and as a forward + backward pipeline in TRAIN_MODE
            variant = "best_of"
            if self.cg is None:
                self.cg = ConvGemm(dtype=self.model.dtype, debug=self.debug, parent_layer=self)
            pairs = [(v, self._get_class_forward_and_backward(v)) for v in ("i2c", "cg")]

            def problem_size(*args):
                return tuple(list(args[0].shape) + list(args[0].weights.shape))

            self._best_fw = BestOf(name="Conv2D only forward", alternatives=[(v, fb[0]) for v, fb in pairs],
                                   get_problem_size=problem_size)
            self._best_fw_bw_pipeline = BestOf(name="Conv2D forward backward",
                                               alternatives=[(v, list(fb)) for v, fb in pairs],
                                               get_problem_size=problem_size)
        forward, backward = self._get_forward_and_backward(variant)
        setattr(self, "forward", forward)
        setattr(self, "backward", backward)

    def _get_forward_and_backward(self, variant):
        tensor_format = "nchw" if self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW else "nhwc"
        return (getattr(self, f"_forward_{tensor_format}_{variant}"),
                getattr(self, f"_backward_{tensor_format}_{variant}"))

    def _get_class_forward_and_backward(self, variant):
        """Unbound functions, called as f(layer, x) (conv_2d_cpu.py:165-181)."""
        tensor_format = "nchw" if self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW else "nhwc"
        return (getattr(type(self), f"_forward_{tensor_format}_{variant}"),
                getattr(type(self), f"_backward_{tensor_format}_{variant}"))

    def _fw_bw_best_of(self, stage, x_or_y):
        """conv_2d_cpu.py:251-259"""
        if self.model.mode == TRAIN_MODE:
            return self._best_fw_bw_pipeline(stage, self, x_or_y)
        if self.model.mode == EVALUATE_MODE:
            return self._best_fw(self, x_or_y)
        raise RuntimeError("Conv2D BestOf variant requires Model.mode to be set to EVALUATE_MODE or TRAIN_MODE")

    def _forward_nchw_best_of(self, x):
        return self._fw_bw_best_of(0, x)

    def _forward_nhwc_best_of(self, x):
        return self._fw_bw_best_of(0, x)

    def _backward_nchw_best_of(self, dy):
        return self._fw_bw_best_of(1, dy)

    def _backward_nhwc_best_of(self, dy):
        return self._fw_bw_best_of(1, dy)

    def _geom(self):
        return (self.kh, self.kw, self.vpadding, self.hpadding, self.vstride, self.hstride,
                self.vdilation, self.hdilation)

    def _geom13(self, b):
        return (b, self.ci, self.hi, self.wi, self.co, self.kh, self.kw, self.vpadding, self.hpadding,
                self.vstride, self.hstride, self.vdilation, self.hdilation)

    def _cg_kwargs(self):
        return dict(vpadding=self.vpadding, hpadding=self.hpadding, vstride=self.vstride, hstride=self.hstride,
                    vdilation=self.vdilation, hdilation=self.hdilation)

    def _op(self, kind):
        """Opens the operation event `kind` of this layer (closed by _end)."""
        self.model.tracer.emit_event(ev.PYDTNN_OPS_EVENT, self.id * ev.PYDTNN_OPS_EVENTS + kind)

    def _end(self):
        self.model.tracer.emit_event(ev.PYDTNN_OPS_EVENT, 0)

    # ---------------------------------------------------------------- i2c, NHWC (conv_2d_cpu.py:183-209, :363-397)
    def _forward_nhwc_i2c(self, x):
        self._op(ev.PYDTNN_OPS_FORWARD_IM2COL)
        x_rows = ops.im2row_nhwc(x, *self._geom())
        self._end()
        if self.model.mode == TRAIN_MODE:
            self.x_rows = x_rows
        y = torch.empty((x.shape[0], self.ho, self.wo, self.co), dtype=x.dtype, device=x.device)
        # matmul + add_nhwc_cython fused: the bias is added in the GEMM's store
        self._op(ev.PYDTNN_OPS_FORWARD_MATMUL)
        ops.conv_i2c_forward(True, self._geom13(x.shape[0]), self.weights, x_rows, y,
                             self.biases if self.use_bias else None)
        self._end()
        return y

    def _backward_nhwc_i2c(self, dy):
        b = dy.shape[0]
        self.dw = torch.empty_like(self.weights)
        with self.model.beside_backward(self, dy, self.x_rows):
            self._op(ev.PYDTNN_OPS_COMP_DW_MATMUL)
            ops.conv_i2c_dw(True, self._geom13(b), dy, self.x_rows, self.dw)
            self._end()
            if self.use_bias:
                self._op(ev.PYDTNN_OPS_BACKWARD_SUM_BIASES)
                self.db = ops.bias_grad(dy, self.co, 1)
                self._end()
        if self.need_dx:
            dx = torch.empty((b, self.hi, self.wi, self.ci), dtype=dy.dtype, device=dy.device)
            self._op(ev.PYDTNN_OPS_COMP_DX_MATMUL)  # the GEMM and row2im of the explicit route
            ops.conv_i2c_dx(True, self._geom13(b), self.weights, dy, dx)
            self._end()
            return dx

    # ---------------------------------------------------------------- i2c, NCHW (conv_2d_cpu.py:264-291, :447-481)
    def _forward_nchw_i2c(self, x):
        self._op(ev.PYDTNN_OPS_FORWARD_IM2COL)
        x_cols = ops.im2col_nchw(x, *self._geom())
        self._end()
        if self.model.mode == TRAIN_MODE:
            self.x_cols = x_cols
        y = torch.empty((x.shape[0], self.co, self.ho, self.wo), dtype=x.dtype, device=x.device)
        # matmul + add_nchw_cython + best_transpose_1023 fused into the GEMM's store
        self._op(ev.PYDTNN_OPS_FORWARD_MATMUL)
        ops.conv_i2c_forward(False, self._geom13(x.shape[0]), self.weights, x_cols, y,
                             self.biases if self.use_bias else None)
        self._end()
        return y

    def _backward_nchw_i2c(self, dy):
        b = dy.shape[0]
        self.dw = torch.empty_like(self.weights)
        with self.model.beside_backward(self, dy, self.x_cols):
            self._op(ev.PYDTNN_OPS_COMP_DW_MATMUL)
            ops.conv_i2c_dw(False, self._geom13(b), dy, self.x_cols, self.dw)
            self._end()
            if self.use_bias:
                self._op(ev.PYDTNN_OPS_BACKWARD_SUM_BIASES)
                self.db = ops.bias_grad(dy, self.co, self.ho * self.wo)
                self._end()
        if self.need_dx:
            dx = torch.empty((b, self.ci, self.hi, self.wi), dtype=dy.dtype, device=dy.device)
            self._op(ev.PYDTNN_OPS_COMP_DX_MATMUL)  # the GEMM and col2im of the explicit route
            ops.conv_i2c_dx(False, self._geom13(b), self.weights, dy, dx)
            self._end()
            return dx

    def _evaluate_forward(self, x, nhwc, bn=None, relu=False):
        """EVALUATE_MODE forward through a call prepared once per (input shape, bound tensors): the geometry, the
        filter and the per-channel vectors are fixed when the layer is initialised, so a step passes only x
        (conv_2d_cpu.py:89-143 fixes them in ``initialize`` too).  With ``Model(enable_memory_cache=True)`` the
        layer also keeps its output tensor between steps, as the reference's GPU layers do
        (pydtnn/backends/gpu/layers/conv_2d_gpu.py:89-96): each call then returns the same tensor, overwritten."""
        biases_vector = self.biases if self.use_bias else None
        p = self._prepared
        if p is None or p.x_shape != x.shape or not p.binds(self.weights, biases_vector, bn, relu):
            p = self._prepared = PreparedForward(nhwc, x.shape, self.weights, self._geom(), biases_vector, bn, relu,
                                                 keep_output=bool(self.model.enable_memory_cache))
        return p(x)

    # ---------------------------------------------------------------- cg, NHWC (conv_2d_cpu.py:211-227, :399-427)
    def _folded_forward(self, conv_gemm, x, out_shape, biases_vector):
        """TRAIN_MODE forward that also does the Relu layer above: y = relu(conv(x) + b) and that layer's mask."""
        y = torch.empty(out_shape, dtype=x.dtype, device=x.device)
        mask = torch.empty(out_shape, dtype=torch.int8, device=x.device)
        conv_gemm(self.weights, x, biases=y, biases_vector=biases_vector, relu=True, relu_mask=mask,
                  **self._cg_kwargs())
        self.relu_above.take_folded(y, mask)
        return y

    def _forward_nhwc_cg(self, x):
        if self.model.mode == TRAIN_MODE:
            self.cg_x = x
        biases_vector = self.biases if self.use_bias else None
        self._op(ev.PYDTNN_OPS_FORWARD_CONVGEMM)
        if self._folds_relu_above():
            y = self._folded_forward(self.cg.conv_gemm_nhwc, x, (x.shape[0], self.ho, self.wo, self.co),
                                     biases_vector)
        elif self.model.mode == EVALUATE_MODE:
            y = self._evaluate_forward(x, True)
        else:
            y = self.cg.conv_gemm_nhwc(self.weights, x, biases_vector=biases_vector, **self._cg_kwargs())
        self._end()
        return y

    def _filter_and_bias_gradients(self, dy, conv_gemm, rows):
        res = torch.empty(self.weights.shape, dtype=dy.dtype, device=dy.device)
        with self.model.beside_backward(self, dy, self.cg_x):
            self._op(ev.PYDTNN_OPS_BACKWARD_CONVGEMM)
            conv_gemm(dy, self.cg_x, biases=res, trans=True, **self._cg_kwargs())
            self._end()
            self.dw = res
            if self.use_bias:
                self._op(ev.PYDTNN_OPS_BACKWARD_SUM_BIASES)
                self.db = ops.bias_grad(dy, self.co, rows)
                self._end()

    def _backward_nhwc_cg(self, dy):
        self._filter_and_bias_gradients(dy, self.cg.conv_gemm_nhwc, 1)
        if self.need_dx:
            dx = torch.empty((dy.shape[0], self.hi, self.wi, self.ci), dtype=dy.dtype, device=dy.device)
            gate = self._gate_below(dx.shape)
            self._op(ev.PYDTNN_OPS_BACKWARD_DECONV_GEMM)
            self.cg.deconv_gemm_nhwc(self.weights, dy, dx, gate=gate, **self._cg_kwargs())
            self._end()
            if gate is not None:
                self.relu_below.take_gated(dx)
            return dx

    # ---------------------------------------------------------------- cg, NCHW (conv_2d_cpu.py:293-308, :483-510)
    def _forward_nchw_cg(self, x):
        if self.model.mode == TRAIN_MODE:
            self.cg_x = x
        biases_vector = self.biases if self.use_bias else None
        self._op(ev.PYDTNN_OPS_FORWARD_CONVGEMM)
        if self._folds_relu_above():
            y = self._folded_forward(self.cg.conv_gemm_nchw, x, (x.shape[0], self.co, self.ho, self.wo),
                                     biases_vector)
        elif self.model.mode == EVALUATE_MODE:
            y = self._evaluate_forward(x, False)
        else:
            y = self.cg.conv_gemm_nchw(self.weights, x, biases=None, biases_vector=biases_vector,
                                       **self._cg_kwargs())
        self._end()
        return y

    def _backward_nchw_cg(self, dy):
        self._filter_and_bias_gradients(dy, self.cg.conv_gemm_nchw, self.ho * self.wo)
        if self.need_dx:
            dx = torch.empty((dy.shape[0], self.ci, self.hi, self.wi), dtype=dy.dtype, device=dy.device)
            gate = self._gate_below(dx.shape)
            self._op(ev.PYDTNN_OPS_BACKWARD_DECONV_GEMM)
            self.cg.deconv_gemm_nchw(self.weights, dy, dx, gate=gate, **self._cg_kwargs())
            self._end()
            if gate is not None:
                self.relu_below.take_gated(dx)
            return dx


# --------------------------------------------------------------------------- FC
class FC(Layer):
    """pydtnn/layers/fc.py:27-42 + pydtnn/backends/cpu/layers/fc_cpu.py:30-77.  Weights are (in, out)."""

    def __init__(self, shape=(1,), activation="", use_bias=True, weights_initializer="glorot_uniform",
                 biases_initializer="zeros"):
        super().__init__(shape)
        self.act = activations.get(activation, None)
        self.use_bias = use_bias
        self.weights_initializer = initializers[weights_initializer]
        self.biases_initializer = initializers[biases_initializer]
        self.grad_vars = {"weights": "dw"}
        if self.use_bias:
            self.grad_vars["biases"] = "db"
        self.x = None
        self.dw = None
        self.db = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.weights = self.weights_initializer((*prev_shape, *self.shape)).to(self.model.dtype)
        if self.use_bias:
            self.biases = self.biases_initializer(self.shape).to(self.model.dtype)
        self.nparams = self.weights.numel() + (self.biases.numel() if self.use_bias else 0)

    def forward(self, x):
        if self.model.mode == TRAIN_MODE:
            self.x = x
        if not self.use_bias:
            # fc_cpu.py:63 is `return res + self.biases if self.use_bias else 0`: without a bias the
            # reference returns the scalar 0.  That is a precedence slip, not a contract; return x @ W.
            return self.model.matmul(x, self.weights)
        return self.model.matmul(x, self.weights, bias=self.biases)

    def backward(self, dy):
        with self.model.beside_backward(self, dy, self.x):
            self.dw = self.model.matmul(self.x.t(), dy)
            if self.use_bias:
                self.db = ops.bias_grad(dy, dy.shape[1], 1)
        if self.need_dx:
            return self.model.matmul(dy, self.weights.t())


# --------------------------------------------------------------------------- pooling, flatten, dropout
class MaxPool2D(Layer):
    """pydtnn/layers/abstract_pool_2d_layer.py:28-57 + pydtnn/backends/cpu/layers/max_pool_2d_cpu.py:30-117."""

    def __init__(self, pool_shape=(2, 2), padding=0, stride=1, dilation=1):
        super().__init__()
        self.pool_shape = pool_shape
        self.padding, self.stride, self.dilation = padding, stride, dilation
        self.vpadding, self.hpadding = _pair(padding)
        self.vstride, self.hstride = _pair(stride)
        self.vdilation, self.hdilation = _pair(dilation)
        self.ci = self.hi = self.wi = self.kh = self.kw = self.ho = self.wo = self.co = self.n = 0
        self.idx_max = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.hi, self.wi, self.ci = decode_tensor(prev_shape, self.model.tensor_format)
        if self.pool_shape[0] == 0:
            self.pool_shape = (self.hi, self.pool_shape[1])
        if self.pool_shape[1] == 0:
            self.pool_shape = (self.pool_shape[0], self.wi)
        self.kh, self.kw = self.pool_shape
        self.co = self.ci
        self.ho = (self.hi + 2 * self.vpadding - self.vdilation * (self.kh - 1) - 1) // self.vstride + 1
        self.wo = (self.wi + 2 * self.hpadding - self.hdilation * (self.kw - 1) - 1) // self.hstride + 1
        assert self.ho > 0 and self.wo > 0, "Output dimensions must be greater than 0"
        self.shape = encode_tensor((self.ho, self.wo, self.co), self.model.tensor_format)
        self.n = int(np.prod(self.shape))

    def _geom(self):
        return (self.kh, self.kw, self.vpadding, self.hpadding, self.vstride, self.hstride,
                self.vdilation, self.hdilation)

    def forward(self, x):
        nchw = self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW
        y, idx_max = (ops.max_pool_2d_fwd_nchw if nchw else ops.max_pool_2d_fwd_nhwc)(x, *self._geom())
        if self.model.mode == TRAIN_MODE:
            self.idx_max = idx_max
        return y

    def backward(self, dy):
        if self.need_dx:
            b = dy.shape[0]
            if self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
                bwd, dims = ops.max_pool_2d_bwd_nchw, (b, self.ci, self.hi, self.wi)
            else:
                bwd, dims = ops.max_pool_2d_bwd_nhwc, (b, self.hi, self.wi, self.ci)
            gate = self._gate_below(dims)
            dx = bwd(dy, self.idx_max, *dims, *self._geom(), gate=gate)
            if gate is not None:
                self.relu_below.take_gated(dx)
            return dx


class AveragePool2D(MaxPool2D):
    """pydtnn/layers/abstract_pool_2d_layer.py:28-57 + pydtnn/backends/cpu/layers/average_pool_2d_cpu.py:30-108.
    ``pool_shape=(0, 0)`` pools each whole plane (global average pooling)."""

    def forward(self, x):
        nhwc = self.model.tensor_format != PYDTNN_TENSOR_FORMAT_NCHW
        return ops.average_pool_2d_fwd(x, nhwc, *self._geom())

    def backward(self, dy):
        if self.need_dx:
            nhwc = self.model.tensor_format != PYDTNN_TENSOR_FORMAT_NCHW
            return ops.average_pool_2d_bwd(dy, nhwc, dy.shape[0], self.ci, self.hi, self.wi, *self._geom())


class Flatten(Layer):
    """pydtnn/layers/flatten.py:26-30 + pydtnn/backends/cpu/layers/flatten_cpu.py"""

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = (int(np.prod(prev_shape)),)

    def forward(self, x):
        return x.reshape(x.shape[0], *self.shape)

    def backward(self, dy):
        if self.need_dx:
            return dy.reshape(dy.shape[0], *self.prev_shape)


class Dropout(Layer):
    """pydtnn/backends/cpu/layers/dropout_cpu.py:28-43 (mask drawn with torch's generator on the GPU)."""

    def __init__(self, rate=0.5):
        super().__init__()
        self.rate = min(1., max(0., rate))
        self.mask = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = prev_shape

    def forward(self, x):
        if self.model.mode == TRAIN_MODE and self.rate > 0:
            self.mask = torch.bernoulli(torch.full_like(x, 1 - self.rate)) / (1 - self.rate)
            return x * self.mask
        self.mask = None
        return x

    def backward(self, dy):
        if self.need_dx:
            return dy if self.mask is None else dy * self.mask


# --------------------------------------------------------------------------- BatchNormalization (inference)
class BatchNormalization(Layer):
    """pydtnn/layers/batch_normalization.py:26-62 + the EVALUATE_MODE branch of
    pydtnn/backends/cpu/layers/batch_normalization_cpu.py:40-129.  ``xn`` is kept in the model's tensor
    format (the reference keeps it as a (rows, channels) matrix); ``std`` is per channel."""

    def __init__(self, beta=0.0, gamma=1.0, momentum=0.9, epsilon=1e-5,
                 moving_mean_initializer="zeros", moving_variance_initializer="zeros", sync_stats=False):
        super().__init__()
        self.gamma_init_val = gamma
        self.beta_init_val = beta
        self.momentum = momentum
        self.epsilon = epsilon
        self.moving_mean_initializer = initializers[moving_mean_initializer]
        self.moving_variance_initializer = initializers[moving_variance_initializer]
        self.grad_vars = {"beta": "dbeta", "gamma": "dgamma"}
        self.sync_stats = sync_stats
        self.spatial = self.co = self.ci = self.hi = self.wi = 0
        self.gamma = self.beta = self.running_mean = self.running_var = None
        self.updated_running_var = False
        self.inv_std = None

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        self.shape = shape_ = prev_shape
        self.spatial = len(self.shape) > 2
        if self.spatial:
            self.hi, self.wi, self.ci = decode_tensor(self.shape, self.model.tensor_format)
            shape_ = (self.ci,)
        self.gamma = torch.full(shape_, self.gamma_init_val, dtype=self.model.dtype, device="cuda")
        self.beta = torch.full(shape_, self.beta_init_val, dtype=self.model.dtype, device="cuda")
        self.running_mean = self.moving_mean_initializer(shape_).to(self.model.dtype)
        self.running_var = self.moving_variance_initializer(shape_).to(self.model.dtype)
        self.inv_std = 1.0 / torch.sqrt(self.running_var + self.epsilon)
        self.nparams = self.gamma.numel() + self.beta.numel() + self.running_mean.numel() + self.running_var.numel()

    def _refresh_inv_std(self):
        # batch_normalization_cpu.py:92-94
        if self.updated_running_var:
            self.updated_running_var = False
            self.inv_std = 1.0 / torch.sqrt(self.running_var + self.epsilon)

    def _apply(self, x, relu):
        self._refresh_inv_std()
        bn = (self.running_mean, self.inv_std, self.gamma, self.beta)
        if self.spatial and self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
            return ops.bn_inference_nchw(x, *bn, relu=relu)
        return ops.chan_eltwise(x, channels=x.shape[-1], inner=1, bn=bn, relu=relu)

    def _view(self, t):
        """(channels, inner) of the (outer, channels, inner) view of an activation tensor."""
        if self.spatial and self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW:
            return t.shape[1], t.shape[2] * t.shape[3]
        return t.shape[-1], 1

    def forward(self, x):
        if self.model.mode == TRAIN_MODE:
            if self.sync_stats:
                raise NotImplementedError("sync_stats needs more than one process")
            channels, inner = self._view(x)
            y, self.xn, self.std = ops.bn_training_forward(x, self.gamma, self.beta, self.running_mean,
                                                           self.running_var, self.momentum, self.epsilon,
                                                           channels, inner)
            self.updated_running_var = True
            return y
        if self.model.mode != EVALUATE_MODE:
            raise ValueError("Unexpected model mode")
        return self._apply(x, relu=False)

    def backward(self, dy):
        channels, inner = self._view(dy)
        self.dgamma, self.dbeta, dx = ops.bn_training_backward(dy, self.xn, self.std, self.gamma, channels, inner,
                                                               need_dx=self.need_dx)
        return dx


class _FromParents:
    """Fused layers are built from the layers they replace by copying their ``__dict__``
    (pydtnn/layers/conv_2d_batch_normalization_relu.py:28-37): the second parent's attributes win, so after
    fusion ``ci/hi/wi`` are the BatchNormalization's (the convolution's *output* extents) and ``co`` is 0.
    Nothing below reads those; tensor extents come from the tensors themselves."""

    def _adopt(self, from_parent, from_parent2=None):
        self.__dict__.update(from_parent.__dict__)
        if from_parent2 is not None:
            self.__dict__.update(from_parent2.__dict__)
        # the parents' installed forward/backward variants must not shadow this class's own methods
        self.__dict__.pop("forward", None)
        self.__dict__.pop("backward", None)


class BatchNormalizationRelu(BatchNormalization, _FromParents):
    """pydtnn/layers/batch_normalization_relu.py + pydtnn/backends/cpu/layers/batch_normalization_relu_cpu.py:28-55"""

    def __init__(self, *args, **kwargs):
        from_parent = kwargs.pop("from_parent", None)
        if from_parent is None:
            super().__init__(*args, **kwargs)
        else:
            self._adopt(from_parent)

    def forward(self, x):
        if self.model.mode == TRAIN_MODE:
            raise RuntimeError("Fused layers cannot be used in training mode!")
        return self._apply(x, relu=True)

    def backward(self, x):
        raise RuntimeError(f"Backward method of {self.__class__.__name__} should not be called")


class _FusedConv(Conv2D, _FromParents):
    """Common part of pydtnn/backends/cpu/layers/conv_2d_relu_cpu.py:32-101,
    conv_2d_batch_normalization_cpu.py:25-97 and conv_2d_batch_normalization_relu_cpu.py:25-97: inference only,
    one implicit-GEMM call whose epilogue applies bias -> BN -> ReLU."""

    _with_bn = False
    _with_relu = False

    def __init__(self, *args, **kwargs):
        from_parent = kwargs.pop("from_parent", None)
        from_parent2 = kwargs.pop("from_parent2", None)
        if from_parent is None and from_parent2 is None:
            super().__init__(*args, **kwargs)
        else:
            # the second parent of Conv2DRelu is the Relu layer; only BN parents carry state worth copying
            self._adopt(from_parent, from_parent2 if self._with_bn else None)

    def initialize(self, prev_shape=None, need_dx=True, from_parent_dict=None):
        self.forward = {"_forward_nchw_cg": self._forward_nchw_cg,
                        "_forward_nhwc_cg": self._forward_nhwc_cg}[from_parent_dict["forward"].__name__]
        self.weights = from_parent_dict["weights"]
        self.biases = from_parent_dict["biases"]
        self.shape = from_parent_dict["shape"]

    def _epilogue_kwargs(self):
        kw = dict(self._cg_kwargs(), biases_vector=self.biases if self.use_bias else None, relu=self._with_relu)
        if self._with_bn:
            if self.updated_running_var:
                self.updated_running_var = False
                self.inv_std = 1.0 / torch.sqrt(self.running_var + self.epsilon)
            kw.update(bn_running_mean=self.running_mean, bn_inv_std=self.inv_std, bn_gamma=self.gamma,
                      bn_beta=self.beta)
        return kw

    def _bound_bn(self):
        if not self._with_bn:
            return None
        if self.updated_running_var:
            self.updated_running_var = False
            self.inv_std = 1.0 / torch.sqrt(self.running_var + self.epsilon)
        return (self.running_mean, self.inv_std, self.gamma, self.beta)

    def _forward_nchw_cg(self, x, residual=None, relu_after_residual=False):
        if self.model.mode == TRAIN_MODE:
            raise RuntimeError("Fused layers cannot be used in training mode!")
        if residual is None and self.model.mode == EVALUATE_MODE:
            return self._evaluate_forward(x, False, self._bound_bn(), self._with_relu)
        return self.cg.conv_gemm_nchw(self.weights, x, biases=None, residual=residual,
                                      relu_after_residual=relu_after_residual, **self._epilogue_kwargs())

    def _forward_nhwc_cg(self, x, residual=None, relu_after_residual=False):
        if self.model.mode == TRAIN_MODE:
            raise RuntimeError("Fused layers cannot be used in training mode!")
        if residual is None and self.model.mode == EVALUATE_MODE:
            return self._evaluate_forward(x, True, self._bound_bn(), self._with_relu)
        return self.cg.conv_gemm_nhwc(self.weights, x, biases=None, residual=residual,
                                      relu_after_residual=relu_after_residual, **self._epilogue_kwargs())

    # the sum of an addition block (and the Relu after it) can ride in this layer's store
    accepts_residual = True

    def forward_with_next(self, nxt, x, residual=None, relu_after_residual=False):
        """This layer followed by the 1 x 1 fused layer ``nxt`` as one launch (NHWC, the shapes the library builds it
        for), or None: the caller then runs the two layers one after the other, with the same bits."""
        if self.model.mode != EVALUATE_MODE or self.model.tensor_format == PYDTNN_TENSOR_FORMAT_NCHW or \
                getattr(self, "_no_pair", None) == tuple(x.shape) or not isinstance(nxt, _FusedConv) or \
                (nxt.kh, nxt.kw, nxt.vstride, nxt.hstride, nxt.vpadding, nxt.hpadding) != (1, 1, 1, 1, 0, 0):
            return None
        e1, e2 = self._epilogue_kwargs(), nxt._epilogue_kwargs()
        second = {k + "2": e2[k] for k in ("biases_vector", "relu", "bn_running_mean", "bn_inv_std", "bn_gamma", "bn_beta")
                  if k in e2}
        y = self.cg.conv_gemm_pair_nhwc(self.weights, x, nxt.weights, residual=residual,
                                        relu_after_residual=relu_after_residual, **e1, **second)
        if y is None:
            self._no_pair = tuple(x.shape)      # not a shape the fused launch is built for: do not ask again
        return y

    def backward(self, x):
        raise RuntimeError(f"Backward method of {self.__class__.__name__} should not be called")


class Conv2DRelu(_FusedConv):
    _with_relu = True


class Conv2DBatchNormalization(_FusedConv):
    _with_bn = True


class Conv2DBatchNormalizationRelu(_FusedConv):
    _with_bn = True
    _with_relu = True


# --------------------------------------------------------------------------- residual block
class AdditionBlock(Layer):
    """pydtnn/layers/abstract_block_layer.py:25-57 + pydtnn/backends/cpu/layers/addition_block_cpu.py:28-60:
    runs every path on the same input and sums the results (eltw_sum)."""

    def __init__(self, *args):
        super().__init__()
        self.paths = [list(p) for p in args]
        self.is_block_layer = True
        self.out_shapes = []

    def initialize(self, prev_shape, need_dx=True):
        super().initialize(prev_shape, need_dx)
        for p in self.paths:
            shape = self.prev_shape
            for layer in p:
                layer.set_model(self.model)
                layer.initialize(shape, self.need_dx)
                shape = layer.shape
                self.nparams += layer.nparams
            self.out_shapes.append(shape)
        assert all([o == self.out_shapes[0] for o in self.out_shapes])
        self.shape = self.out_shapes[0]

    def _folded_sum_path(self):
        """Index of the path whose last layer can add the other path's result in its own store, or None.
        Only after the model's fusion pass, in EVALUATE_MODE, for blocks of two paths (a sum of two is the
        same bits in either order; three or more would fix an order)."""
        if not getattr(self.model, "_fused", False) or self.model.mode != EVALUATE_MODE or len(self.paths) != 2:
            return None
        for i, p in enumerate(self.paths):
            if p and getattr(p[-1], "accepts_residual", False):
                return i
        return None

    def forward(self, x):
        k = self._folded_sum_path()
        if k is not None:
            other = x
            for layer in self.paths[1 - k]:
                other = layer.forward(other)
            cur = x
            path = self.paths[k]
            relu = self.relu_above is not None
            y = None
            if len(path) >= 2 and getattr(path[-2], "accepts_residual", False):
                # the path's last two convolutions in one launch where the library has one
                for layer in path[:-2]:
                    cur = layer.forward(cur)
                y = path[-2].forward_with_next(path[-1], cur, residual=other, relu_after_residual=relu)
                if y is None:
                    cur = path[-2].forward(cur)
            else:
                for layer in path[:-1]:
                    cur = layer.forward(cur)
            if y is None:
                y = path[-1].forward(cur, residual=other, relu_after_residual=relu)
            if relu:
                self.relu_above.take_folded(y, None)
            return y
        xs = [x] * len(self.paths)
        for i, p in enumerate(self.paths):
            for layer in p:
                xs[i] = layer.forward(xs[i])
            if i > 0:
                if xs[0] is x:  # an empty first path must not be summed into the caller's tensor
                    xs[0] = x.clone()
                ops.eltw_sum(xs[0], xs[i])
        return xs[0]

    def backward(self, dy):
        dxs = [dy] * len(self.paths)
        for i, p in enumerate(self.paths):
            for layer in reversed(p):
                dxs[i] = layer.backward(dxs[i])
            if i > 0:
                if dxs[0] is dy:
                    dxs[0] = dy.clone()
                ops.eltw_sum(dxs[0], dxs[i])
        return dxs[0]

    def update_weights(self, optimizer):
        for p in self.paths:
            for layer in p:
                layer.update_weights(optimizer)
