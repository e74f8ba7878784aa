"""Layer mirrors of the reference's Keras layers, as ``torch.nn.Module``s:
``AMConv2D`` (python/keras/layers/am_convolutional.py:400-558), ``denseam``
(python/keras/layers/amdenselayer.py:47-256) and the attention layers of
``ammha/multihead_attention.py``.  Bias add, activations, softmax, scaling and
reshapes are plain torch ops, exactly as they are stock TF ops in the
reference; every multiplication of activations by weights goes through the
approximate-multiplier ops."""
import math

import torch
from torch import nn

from . import functors
from .amnn_ops import amconvolution_v2
from .math_ops import matmulam


# Keras vocabulary of the reference's layers (activations.get / initializers.get,
# am_convolutional.py:128-144, amdenselayer.py:109-126): names map to torch functions.
_ACTIVATIONS = {
    "linear": None,
    "relu": torch.relu,
    "sigmoid": torch.sigmoid,
    "tanh": torch.tanh,
    "softmax": lambda x: torch.softmax(x, dim=-1),
    "softplus": nn.functional.softplus,
    "softsign": nn.functional.softsign,
    "elu": nn.functional.elu,
    "selu": nn.functional.selu,
    "gelu": nn.functional.gelu,
    "swish": nn.functional.silu,
    "exponential": torch.exp,
}


def _get_activation(activation):
    """None, a Keras activation name, or a callable -> callable or None (identity)."""
    if activation is None or callable(activation):
        return activation
    if isinstance(activation, str) and activation in _ACTIVATIONS:
        return _ACTIVATIONS[activation]
    raise ValueError(f"Unknown activation function: {activation}")


def _fusable(activation):
    """Name of the activation if the library can apply it in the producing kernel, else None."""
    if activation is None:
        return "linear"
    if activation in (torch.relu, torch.nn.functional.relu) or isinstance(activation, nn.ReLU):
        return "relu"
    return None


def _initialize_(t, initializer, fan_in, fan_out):
    """Fills ``t`` in place by a Keras initializer name, or by a callable ``f(shape)`` that
    returns the values."""
    with torch.no_grad():
        if callable(initializer):
            return t.copy_(torch.as_tensor(initializer(tuple(t.shape)), dtype=t.dtype))
        name = str(initializer).lower()
        if name == "zeros":
            return t.zero_()
        if name == "ones":
            return t.fill_(1.0)
        if name == "random_normal":
            return t.normal_(0.0, 0.05)
        if name == "random_uniform":
            return t.uniform_(-0.05, 0.05)
        scale = {"glorot": 2.0 / (fan_in + fan_out), "he": 2.0 / fan_in, "lecun": 1.0 / fan_in}
        for family, variance in scale.items():
            if name == family + "_uniform":
                limit = math.sqrt(3.0 * variance)
                return t.uniform_(-limit, limit)
            if name == family + "_normal":
                # Keras draws from a normal truncated at two standard deviations and rescales
                std = math.sqrt(variance) / 0.87962566103423978
                return nn.init.trunc_normal_(t, 0.0, std, -2.0 * std, 2.0 * std)
        raise ValueError(f"Unknown initializer: {initializer}")


class _KerasLayerArgs:
    """Constructor arguments every Keras layer of the reference accepts besides its own:
    regularizers and constraints are kept as callables (``losses()`` evaluates the
    regularizers, ``apply_constraints()`` projects the parameters); ``name``, ``dtype``,
    ``trainable`` and ``input_shape`` are honoured where they mean something here."""

    def _keras_args(self, kernel_regularizer, bias_regularizer, activity_regularizer, kernel_constraint,
                    bias_constraint, kwargs):
        for what, f in (("kernel_regularizer", kernel_regularizer), ("bias_regularizer", bias_regularizer),
                        ("activity_regularizer", activity_regularizer), ("kernel_constraint", kernel_constraint),
                        ("bias_constraint", bias_constraint)):
            if f is not None and not callable(f):
                raise ValueError(f"{what} must be a callable or None")
        self.kernel_regularizer, self.bias_regularizer = kernel_regularizer, bias_regularizer
        self.activity_regularizer = activity_regularizer
        self.kernel_constraint, self.bias_constraint = kernel_constraint, bias_constraint
        self.layer_name = kwargs.pop("name", None)
        self.trainable = bool(kwargs.pop("trainable", True))
        dtype = kwargs.pop("dtype", None)
        if dtype not in (None, "float32", torch.float32):
            raise ValueError("the approximate-multiplier ops are float32 only")
        input_shape = kwargs.pop("input_shape", None)
        kwargs.pop("batch_input_shape", None)
        if kwargs:
            raise TypeError(f"Keyword argument not understood: {sorted(kwargs)[0]}")
        self._activity_loss = None
        return input_shape

    def _finish_build(self):
        if not self.trainable:
            for p in self.parameters():
                p.requires_grad_(False)

    def _track_activity(self, out):
        if self.activity_regularizer is not None:
            self._activity_loss = self.activity_regularizer(out)
        return out

    def losses(self):
        """Regularization terms of this layer (Keras ``layer.losses``), to be added to the objective."""
        out = []
        if self.kernel_regularizer is not None and self.kernel is not None:
            out.append(self.kernel_regularizer(self.kernel))
        if self.bias_regularizer is not None and self.bias is not None:
            out.append(self.bias_regularizer(self.bias))
        if self._activity_loss is not None:
            out.append(self._activity_loss)
        return out

    def apply_constraints(self):
        """Projects kernel and bias through their constraints (Keras does so after each update)."""
        with torch.no_grad():
            if self.kernel_constraint is not None and self.kernel is not None:
                self.kernel.copy_(self.kernel_constraint(self.kernel))
            if self.bias_constraint is not None and self.bias is not None:
                self.bias.copy_(self.bias_constraint(self.bias))


def _epilogue_backward(grad, out, bias, act):
    """Gradient through act(z + bias) given its output: (dL/dz, dL/dbias)."""
    grad = grad.contiguous()
    if act == "relu":
        grad = grad * (out > 0)
    grad_bias = grad.reshape(-1, grad.shape[-1]).sum(0) if bias is not None else None
    return grad, grad_bias


class _ConvamBiasAct(torch.autograd.Function):
    """``act(Convam(input, filter) + bias)`` in one kernel (the reference runs Convam, BiasAdd
    and the activation as three ops, am_convolutional.py:248-276); the gradient is the chain
    rule through the epilogue followed by ConvamInputGrad / ConvamFilterGrad."""

    @staticmethod
    def forward(ctx, input, filters, bias, strides, padding, mant_mul_lut, act):
        out = functors.convam(mant_mul_lut, input, filters, strides, padding, bias=bias, activation=act)
        ctx.save_for_backward(input, filters, out)
        ctx.attrs = (strides, padding, mant_mul_lut, act, bias is not None)
        return out

    @staticmethod
    def backward(ctx, grad):
        input, filters, out = ctx.saved_tensors
        strides, padding, lut, act, has_bias = ctx.attrs
        grad, grad_bias = _epilogue_backward(grad, out, has_bias or None, act)
        grad_input = grad_filter = None
        if ctx.needs_input_grad[0]:
            grad_input = functors.convam_input_grad(lut, input.shape, filters, grad, strides, padding)
        if ctx.needs_input_grad[1]:
            grad_filter = functors.convam_filter_grad(lut, input, filters.shape, grad, strides, padding)
        return grad_input, grad_filter, grad_bias, None, None, None, None


class AMConv2D(nn.Module, _KerasLayerArgs):
    """2-D convolution over NHWC input with an HWIO kernel through op ``Convam``.
    Same constructor vocabulary as the Keras layer (am_convolutional.py:519-558):
    ``filters, kernel_size, strides, padding ('valid' | 'same'), data_format, dilation_rate,
    groups, activation, use_bias, kernel_initializer, bias_initializer, the regularizers and
    constraints, mant_mul_lut``.  Like the reference, only channels-last data, dilation 1
    (amnn_ops.py:196-197) and one group run through the approximate op."""

    def __init__(self, filters, kernel_size, strides=(1, 1), padding="valid", data_format=None,
                 dilation_rate=(1, 1), groups=1, activation=None, use_bias=True,
                 kernel_initializer="glorot_uniform", bias_initializer="zeros", kernel_regularizer=None,
                 bias_regularizer=None, activity_regularizer=None, kernel_constraint=None, bias_constraint=None,
                 mant_mul_lut='', in_channels=None, **kwargs):
        super().__init__()
        if not mant_mul_lut:
            raise ValueError("mant_mul_lut must name a LUT file")
        ks = (kernel_size, kernel_size) if isinstance(kernel_size, int) else tuple(kernel_size)
        st = (strides, strides) if isinstance(strides, int) else tuple(strides)
        dr = (dilation_rate, dilation_rate) if isinstance(dilation_rate, int) else tuple(dilation_rate)
        if len(ks) != 2 or len(st) != 2 or len(dr) != 2:
            raise ValueError("kernel_size, strides and dilation_rate take one or two integers")
        if filters is not None and int(filters) < 0:
            raise ValueError(f"Received a negative value for `filters`. Was expecting a positive value, got {filters}.")
        if any(d != 1 for d in dr):
            raise ValueError("Dilation is not supported in current implementation")
        if padding.lower() == "causal":
            raise ValueError("Causal padding is only supported for `Conv1D` and `SeparableConv1D`.")
        if padding.lower() not in ("valid", "same"):
            raise ValueError("padding must be 'valid' or 'same'")
        if data_format not in (None, "channels_last"):
            raise ValueError("only channels_last (NHWC) data runs through the approximate convolution")
        if groups != 1:
            raise ValueError("grouped convolution is not provided by the approximate convolution op")
        self.filters, self.kernel_size, self.strides = int(filters), ks, st
        self.padding = padding.upper()
        self.activation, self.use_bias, self.mant_mul_lut = _get_activation(activation), use_bias, mant_mul_lut
        self.kernel_initializer, self.bias_initializer = kernel_initializer, bias_initializer
        input_shape = self._keras_args(kernel_regularizer, bias_regularizer, activity_regularizer, kernel_constraint,
                                       bias_constraint, kwargs)
        self.kernel = None
        self.bias = None
        if in_channels is None and input_shape is not None:
            in_channels = input_shape[-1]
        if in_channels is not None:
            self.build(in_channels)

    def build(self, in_channels, device=None):
        kh, kw = self.kernel_size
        k = torch.empty(kh, kw, in_channels, self.filters, device=device)
        _initialize_(k, self.kernel_initializer, kh * kw * in_channels, kh * kw * self.filters)
        self.kernel = nn.Parameter(k)
        if self.use_bias:
            b = torch.empty(self.filters, device=device)
            self.bias = nn.Parameter(_initialize_(b, self.bias_initializer, self.filters, self.filters))
        self._finish_build()

    def forward(self, inputs):
        return self._track_activity(self._call(inputs))

    def _call(self, inputs):
        if self.kernel is None:
            self.build(inputs.shape[-1], inputs.device)
        act = _fusable(self.activation)
        if act is not None and (self.use_bias or act != "linear"):
            if inputs.dim() != 4 or inputs.shape[3] != self.kernel.shape[2]:
                raise ValueError("input must be NHWC with the kernel's input depth")
            return _ConvamBiasAct.apply(inputs, self.kernel, self.bias if self.use_bias else None,
                                        tuple(self.strides), self.padding, self.mant_mul_lut, act)
        out = amconvolution_v2(inputs, self.kernel, strides=list(self.strides), padding=self.padding,
                               data_format="NHWC", mant_mul_lut=self.mant_mul_lut)
        if self.use_bias:
            out = out + self.bias
        return self.activation(out) if self.activation is not None else out

    def get_config(self):
        return {"filters": self.filters, "kernel_size": self.kernel_size, "strides": self.strides,
                "padding": self.padding.lower(), "use_bias": self.use_bias, "mant_mul_lut": self.mant_mul_lut}


class _Denseam(torch.autograd.Function):
    """op ``Denseam`` with gradient op ``DenseamGrad`` (denseam.cc:36-57, 177-184;
    gradient registration amdenselayer.py:258-260)."""

    @staticmethod
    def forward(ctx, inputs, weights, mant_mul_lut):
        ctx.save_for_backward(inputs, weights)
        ctx.lut = mant_mul_lut
        return functors.denseam(mant_mul_lut, inputs, weights)

    @staticmethod
    def backward(ctx, grad):
        inputs, weights = ctx.saved_tensors
        grad_input, grad_weights = functors.denseam_grad(ctx.lut, grad.contiguous(), inputs, weights)
        return grad_input, grad_weights, None


class _DenseamBiasAct(torch.autograd.Function):
    """``act(Denseam(inputs, weights) + bias)`` in one kernel (amdenselayer.py:211-226 runs
    three ops); gradient = chain rule through the epilogue, then ``DenseamGrad``."""

    @staticmethod
    def forward(ctx, inputs, weights, bias, mant_mul_lut, act):
        out = functors.denseam(mant_mul_lut, inputs, weights, bias=bias, activation=act)
        ctx.save_for_backward(inputs, weights, out)
        ctx.attrs = (mant_mul_lut, act, bias is not None)
        return out

    @staticmethod
    def backward(ctx, grad):
        inputs, weights, out = ctx.saved_tensors
        lut, act, has_bias = ctx.attrs
        grad, grad_bias = _epilogue_backward(grad, out, has_bias or None, act)
        grad_input, grad_weights = functors.denseam_grad(lut, grad, inputs, weights)
        return grad_input, grad_weights, grad_bias, None, None


class denseam(nn.Module, _KerasLayerArgs):
    """Dense layer through op ``Denseam``: ``activation(inputs . kernel + bias)``, with the Keras
    constructor vocabulary of amdenselayer.py:93-126.  Inputs of rank > 2 are flattened to
    [-1, width] and go through the same op (the reference routes them to an exact
    ``tensordot``, amdenselayer.py:215, which silently bypasses the approximate multiplier)."""

    def __init__(self, units, activation=None, use_bias=True, kernel_initializer="glorot_uniform",
                 bias_initializer="zeros", kernel_regularizer=None, bias_regularizer=None, activity_regularizer=None,
                 kernel_constraint=None, bias_constraint=None, mant_mul_lut='', input_dim=None, **kwargs):
        super().__init__()
        if not mant_mul_lut:
            raise ValueError("mant_mul_lut must name a LUT file")
        if int(units) < 0:
            raise ValueError(f"Received an invalid value for `units`, expected a positive integer, got {units}.")
        self.units, self.use_bias, self.mant_mul_lut = int(units), use_bias, mant_mul_lut
        self.activation = _get_activation(activation)
        self.kernel_initializer, self.bias_initializer = kernel_initializer, bias_initializer
        input_shape = self._keras_args(kernel_regularizer, bias_regularizer, activity_regularizer, kernel_constraint,
                                       bias_constraint, kwargs)
        self.kernel = None
        self.bias = None
        if input_dim is None and input_shape is not None:
            input_dim = input_shape[-1]
        if input_dim is not None:
            self.build(input_dim)

    def build(self, input_dim, device=None):
        k = torch.empty(input_dim, self.units, device=device)
        _initialize_(k, self.kernel_initializer, input_dim, self.units)
        self.kernel = nn.Parameter(k)
        if self.use_bias:
            b = torch.empty(self.units, device=device)
            self.bias = nn.Parameter(_initialize_(b, self.bias_initializer, self.units, self.units))
        self._finish_build()

    def forward(self, inputs):
        return self._track_activity(self._call(inputs))

    def _call(self, inputs):
        if self.kernel is None:
            self.build(inputs.shape[-1], inputs.device)
        lead = inputs.shape[:-1]
        flat = inputs.reshape(-1, inputs.shape[-1])
        act = _fusable(self.activation)
        if act is not None and (self.use_bias or act != "linear"):
            out = _DenseamBiasAct.apply(flat, self.kernel, self.bias if self.use_bias else None, self.mant_mul_lut, act)
            return out.reshape(tuple(lead) + (self.units,))
        out = _Denseam.apply(flat, self.kernel, self.mant_mul_lut)
        out = out.reshape(tuple(lead) + (self.units,))
        if self.use_bias:
            out = out + self.bias
        return self.activation(out) if self.activation is not None else out

    def get_config(self):
        return {"units": self.units, "use_bias": self.use_bias, "mant_mul_lut": self.mant_mul_lut}


class _Attention(torch.autograd.Function):
    """The whole of DotProductAttention.call as one library call per direction; the mask is a
    constant (no gradient), as in the reference."""

    @staticmethod
    def forward(ctx, queries, keys, values, mask, divisor, mant_mul_lut):
        out, weights = functors.attention(mant_mul_lut, queries, keys, values, divisor, mask)
        ctx.save_for_backward(queries, keys, values, weights)
        ctx.attrs = (divisor, mant_mul_lut)
        return out

    @staticmethod
    def backward(ctx, grad):
        queries, keys, values, weights = ctx.saved_tensors
        divisor, lut = ctx.attrs
        gq, gk, gv = functors.attention_grad(lut, queries, keys, values, weights, grad.contiguous(), divisor)
        return gq, gk, gv, None, None, None


class DotProductAttention(nn.Module):
    """Scaled dot-product attention with both matrix products through the approximate
    multiplier (multihead_attention.py:9-30): ``matmulam(softmax(matmulam(q, k^T) / sqrt(d_k)
    + -1e9 * mask), v)``, run as one strided batch over every leading dimension."""

    def __init__(self, lut_file):
        super().__init__()
        self.lut_file = lut_file

    def forward(self, queries, keys, values, d_k, mask=None):
        return _Attention.apply(queries, keys, values, mask, math.sqrt(float(d_k)), self.lut_file)


class MultiHeadAttention(nn.Module):
    """AMMHA (multihead_attention.py:33-89): four ``denseam`` projections around
    ``DotProductAttention``."""

    def __init__(self, lut_file, h, d_k, d_v, d_model, input_dim=None):
        super().__init__()
        self.attention = DotProductAttention(lut_file)
        self.heads, self.d_k, self.d_v, self.d_model = h, d_k, d_v, d_model
        self.W_q = denseam(d_k, mant_mul_lut=lut_file, input_dim=input_dim)
        self.W_k = denseam(d_k, mant_mul_lut=lut_file, input_dim=input_dim)
        self.W_v = denseam(d_v, mant_mul_lut=lut_file, input_dim=input_dim)
        self.W_o = denseam(d_model, mant_mul_lut=lut_file, input_dim=d_v if input_dim is not None else None)

    def reshape_tensor(self, x, heads, flag):
        if flag:
            x = x.reshape(x.shape[0], x.shape[1], heads, -1).permute(0, 2, 1, 3)
        else:
            x = x.permute(0, 2, 1, 3)
            x = x.reshape(x.shape[0], x.shape[1], self.d_k)
        return x.contiguous()

    def forward(self, queries, keys, values, mask=None):
        q = self.reshape_tensor(self.W_q(queries), self.heads, True)
        k = self.reshape_tensor(self.W_k(keys), self.heads, True)
        v = self.reshape_tensor(self.W_v(values), self.heads, True)
        o = self.attention(q, k, v, self.d_k, mask)
        return self.W_o(self.reshape_tensor(o, self.heads, False))
