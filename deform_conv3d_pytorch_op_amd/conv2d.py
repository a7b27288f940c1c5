"""The reference's plain convolution package: `Conv2dFunction`
(conv2d/conv2d_functions/conv2d_function.py:7-67) and `Conv2d`
(conv2d/conv2d_modules/conv2d_model.py:11-46), on the kernels of the 2-D deformable layer with every
offset zero (C ABI: conv2d_forward / conv2d_backward_input / conv2d_backward_weight in
include/dcn_amd.h, in place of conv2d/lib/conv2d_cuda.h:17-39).

Same call shape, `Conv2dFunction.apply(inputs, weight, bias=None, stride=(1, 1), padding=(0, 0),
dilation=(1, 1), group=1)`, and the reference's dilation-aware output size
(conv2d_function.py:16-19); backward returns (grad_input, grad_weight, grad_bias, None x 4), with
None for gradients that are not needed (the reference wraps None in Variable there).  float32 and
float64 on one MI355X; there is no CPU path.
"""
import torch
import torch.nn as nn
from torch.autograd import Function
from torch.autograd.function import once_differentiable
from torch.nn.modules.utils import _pair

from . import _lib
from .functions import _check, _device_check, _ntuple, _on_device, _stream, output_size


def _conv_geom(inputs, weight, outs, stride, padding, dilation, group):
    return ([inputs.size(0), inputs.size(1), weight.size(0)] + list(inputs.shape[2:]) + list(outs) +
            list(weight.shape[2:]) + list(padding) + list(stride) + list(dilation) + [group])


def _conv_workspace(inputs, weight, outs, group):
    L = _lib.load()
    n = int(L.conv2d_workspace_bytes(inputs.element_size(), inputs.size(0), inputs.size(1), weight.size(0),
                                     inputs.size(2) * inputs.size(3), outs[0] * outs[1],
                                     weight.size(2) * weight.size(3), group))
    _check(n > 0, "inconsistent convolution geometry")
    return torch.empty(n, dtype=torch.uint8, device=inputs.device), n


def _conv_check(inputs, weight, bias, stride, padding, dilation, group):
    """The checks of the reference's shape_check (conv2d/lib/conv2d_cuda.cpp:28-62) with its messages."""
    _check(weight.dim() == 4, "kernel dim")
    _check(inputs.dim() == 4, "input dim")
    _check(group > 0 and inputs.size(1) == weight.size(1) * group, "input c != kernel c")
    _check(weight.size(0) % group == 0, "ou c != ker c")
    _check(inputs.dtype in (torch.float32, torch.float64), "dtype must be float32 or float64")
    _device_check(inputs, weight, bias)
    outs = output_size(inputs.shape[2:], weight.shape[2:], stride, padding, dilation, standard=True)
    _check(outs[0] >= 1, "error outhh")
    _check(outs[1] >= 1, "error outww")
    return outs


class Conv2dFunction(Function):
    @staticmethod
    def forward(ctx, inputs, weight, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1), group=1):
        L = _lib.load()
        stride, padding, dilation = _ntuple(stride, 2), _ntuple(padding, 2), _ntuple(dilation, 2)
        outs = _conv_check(inputs, weight, bias, stride, padding, dilation, group)
        inputs, weight = inputs.contiguous(), weight.contiguous()
        bias_c = bias.contiguous() if bias is not None else None
        ctx.cfg = (stride, padding, dilation, group, outs)
        ctx.save_for_backward(inputs, weight)
        ctx.has_bias = bias is not None
        output = torch.empty((inputs.size(0), weight.size(0)) + outs, dtype=inputs.dtype, device=inputs.device)
        suf = "f32" if inputs.dtype == torch.float32 else "f64"
        with _on_device(inputs.device):
            ws, n = _conv_workspace(inputs, weight, outs, group)
            _lib.check(getattr(L, "conv2d_forward_" + suf)(
                inputs.data_ptr(), weight.data_ptr(), bias_c.data_ptr() if bias_c is not None else None,
                output.data_ptr(), *_conv_geom(inputs, weight, outs, stride, padding, dilation, group),
                ws.data_ptr(), n, _stream()))
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        L = _lib.load()
        inputs, weight = ctx.saved_tensors
        stride, padding, dilation, group, outs = ctx.cfg
        grad_output = grad_output.contiguous()
        grad_input = grad_weight = grad_bias = None
        suf = "f32" if inputs.dtype == torch.float32 else "f64"
        geom = _conv_geom(inputs, weight, outs, stride, padding, dilation, group)
        with _on_device(inputs.device):
            ws, n = _conv_workspace(inputs, weight, outs, group)
            if ctx.needs_input_grad[0]:
                grad_input = torch.zeros_like(inputs)
                _lib.check(getattr(L, "conv2d_backward_input_" + suf)(
                    weight.data_ptr(), grad_output.data_ptr(), grad_input.data_ptr(), *geom, ws.data_ptr(), n, _stream()))
            if ctx.needs_input_grad[1]:
                grad_weight = torch.zeros_like(weight)
                _lib.check(getattr(L, "conv2d_backward_weight_" + suf)(
                    inputs.data_ptr(), grad_output.data_ptr(), grad_weight.data_ptr(), *geom, ws.data_ptr(), n, _stream()))
        if ctx.has_bias and ctx.needs_input_grad[2]:
            grad_bias = grad_output.sum((0, 2, 3))
        return grad_input, grad_weight, grad_bias, None, None, None, None


class Conv2d(nn.Module):
    """`Conv2d(in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, bias=True,
    groups=1)` with parameters `weight` (Kaiming-normal, fan_out) and `bias` (U(-0.1, 0.1)), as
    conv2d/conv2d_modules/conv2d_model.py:11-46; `device` and `dtype` are extra keyword arguments."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, bias=True, groups=1,
                 device=None, dtype=None):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.group = groups
        if in_channels % groups != 0:
            raise ValueError('in_channels must be divisible by groups')
        if out_channels % groups != 0:
            raise ValueError('out_channels must be divisible by groups')
        kw = dict(device=device, dtype=dtype)
        self.weight = nn.Parameter(torch.empty(out_channels, in_channels // groups, *self.kernel_size, **kw))
        nn.init.kaiming_normal_(self.weight, mode='fan_out')
        if bias:
            self.bias = nn.Parameter(torch.empty(out_channels, **kw))
            nn.init.uniform_(self.bias, -0.1, 0.1)
        else:
            self.register_parameter('bias', None)

    def forward(self, inputs):
        return Conv2dFunction.apply(inputs, self.weight, self.bias, self.stride, self.padding, self.dilation, self.group)
