"""Convolution op wrapper and its gradient registration: the counterpart of the
reference's ``python/ops/amnn_ops.py`` (``amconvolution_v2`` -> op ``Convam``;
``@RegisterGradient("Convam")`` -> ops ``ConvamInputGrad`` + ``ConvamFilterGrad``,
amnn_ops.py:85-244) with ``torch.autograd`` standing in for TensorFlow's
gradient registry.  NHWC input, HWIO filters, as the reference requires."""
import torch

from . import functors

_CHANNELS_LAST_FORMATS = frozenset({"NWC", "NHC", "NHWC", "NWHC"})


def _get_sequence(value, n, channel_index, name):
    """Same normalisation as amnn_ops.py:47-83: int / short list -> a list of
    n + 2 values with 1 at the batch and channel positions."""
    if value is None:
        return [1] * (n + 2)
    if isinstance(value, int):
        value = [value]
    else:
        value = list(value)
    if len(value) == n + 2:
        return value
    if len(value) == 1:
        value = value * n
    elif len(value) != n:
        raise ValueError(f"{name} should be of length 1, {n} or {n + 2} but was {len(value)}")
    if channel_index == 1:
        return [1, 1] + value
    return [1] + value + [1]


class _Convam(torch.autograd.Function):
    """op ``Convam`` (convam.cc:427-437) with the gradient of amnn_ops.py:220-244."""

    @staticmethod
    def forward(ctx, input, filters, strides, padding, mant_mul_lut):
        ctx.save_for_backward(input, filters)
        ctx.attrs = (strides, padding, mant_mul_lut)
        return functors.convam(mant_mul_lut, input, filters, strides, padding)

    @staticmethod
    def backward(ctx, grad):
        input, filters = ctx.saved_tensors
        strides, padding, lut = ctx.attrs
        grad = grad.contiguous()
        grad_input = grad_filter = None
        if ctx.needs_input_grad[0]:
            # ConvamInputGrad(input_sizes = shape(input), filter, out_backprop)
            grad_input = functors.convam_input_grad(lut, input.shape, filters, grad, strides, padding)
        if ctx.needs_input_grad[1]:
            # ConvamFilterGrad(filter_sizes = shape(filter), input, out_backprop)
            grad_filter = functors.convam_filter_grad(lut, input, filters.shape, grad, strides, padding)
        return grad_input, grad_filter, None, None, None


def amconvolution_internal(input, filters, strides=None, padding="VALID", data_format=None, dilations=None,
                           name=None, call_from_convolution=True, num_spatial_dims=None, mant_mul_lut=''):
    if not mant_mul_lut:
        raise ValueError("mant_mul_lut: the LUT file name attr has no default (convam.cc:434)")
    if filters.dim() != 4 or input.dim() != 4:
        raise ValueError("input must be 4-dimensional NHWC and filter 4-dimensional HWIO")
    num_spatial_dims = 2
    if data_format is not None and data_format not in _CHANNELS_LAST_FORMATS:
        raise ValueError("only channels-last (NHWC) data is supported")
    channel_index = num_spatial_dims + 1
    if dilations is not None:
        dilations = _get_sequence(dilations, num_spatial_dims, channel_index, "dilations")
        if any(i != 1 for i in dilations):
            raise ValueError("Dilation is not supported in current implementation")
    strides = _get_sequence(strides, num_spatial_dims, channel_index, "strides")
    if strides[0] != 1 or strides[3] != 1:
        raise ValueError("strides in the batch and depth dimensions must be 1")
    if padding not in ("VALID", "SAME"):
        raise ValueError("padding must be 'VALID' or 'SAME'")
    if input.shape[3] != filters.shape[2]:
        raise ValueError(f"input depth must equal filter depth: {input.shape[3]} vs {filters.shape[2]}")
    return _Convam.apply(input, filters, (int(strides[1]), int(strides[2])), padding, mant_mul_lut)


def amconvolution_v2(input, filters, strides=None, padding="VALID", data_format=None, dilations=None, name=None,
                     mant_mul_lut=''):
    """``amconvolution_v2`` of the reference (amnn_ops.py:199-218)."""
    return amconvolution_internal(input, filters, strides=strides, padding=padding, data_format=data_format,
                                  dilations=dilations, name=name, mant_mul_lut=mant_mul_lut)
