"""nn.Module front ends, mirroring `ConvOffset3d`
(deform3d/deform_conv3d_modules/deform_conv3d_model.py:11-50) and `ConvOffset2d`
(deform2d_double/deform_conv2d_modules/deform_conv2d_model.py:11-50).

Constructor: `(in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
channel_per_group=1, bias=True, groups=1)`, forward `(input, offset)`; parameters are named
`weight` [out, in/groups, *kernel] and `bias` [out], so state_dicts interchange.  The legacy
float 2-D module (deform2d/deform_conv2d_modules/deform_conv2d_model.py:12-18) takes
`channel_per_group` as its 6th positional argument; here that slot is `dilation` as in the other
two packages, so pass `channel_per_group` by keyword.

Initialisation: the reference draws Kaiming-normal (fan_out) and then overwrites the weight with
the constant 1 (deform_conv3d_model.py:38-39); this keeps the Kaiming draw, which is what the
float 2-D package does (deform2d ... :29).  Bias ~ U(-0.1, 0.1) as in the reference (:42).
`device` and `dtype` are extra keyword arguments (the reference hard-codes cuda float / double),
and so are `standard_output_size` (default False: the reference's dilation-blind output size; True:
the usual dilation-aware one, see functions.output_size) and `oob_offset_grad` (default 'reference';
'zero' drops the 3-D kernels' grad_offset term for samples outside the input, see functions.py).

`ConvOffset{2,3}dPack` additionally own the plain convolution that the reference's callers put in
front of the layer to produce the offsets (deform3d/test_model.py:18-30, deform2d/test_model.py:19-29):
`nn.Conv{2,3}d(in_channels, in_channels // channel_per_group * nd * prod(kernel), kernel, stride,
padding, bias=False)` on the same input; forward takes the input alone.
"""
import torch
import torch.nn as nn
from torch.nn.modules.utils import _pair, _triple

from .functions import ConvOffset2dFunction, ConvOffset3dFunction


class _ConvOffsetNd(nn.Module):
    _tuple = None
    _function = None

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 channel_per_group=1, bias=True, groups=1, device=None, dtype=None, standard_output_size=False,
                 oob_offset_grad="reference"):
        super().__init__()
        self.standard_output_size = bool(standard_output_size)
        if oob_offset_grad not in ("reference", "zero"):
            raise ValueError("oob_offset_grad must be 'reference' or 'zero'")
        self.oob_offset_grad = oob_offset_grad
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = self._tuple(kernel_size)
        self.stride = self._tuple(stride)
        self.padding = self._tuple(padding)
        self.dilation = self._tuple(dilation)
        self.channel_per_group = channel_per_group
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

    def forward(self, input, offset):
        return self._function.apply(input, offset, self.weight, self.bias, self.stride, self.padding,
                                    self.dilation, self.channel_per_group, self.group, self.standard_output_size,
                                    self.oob_offset_grad)

    def extra_repr(self):
        return ('{in_channels}, {out_channels}, kernel_size={kernel_size}, stride={stride}, padding={padding}, '
                'dilation={dilation}, channel_per_group={channel_per_group}, groups={group}, '
                'bias=' + str(self.bias is not None)).format(**self.__dict__)


class _ConvOffsetPackNd(_ConvOffsetNd):
    """The deformable layer together with its offset-producing convolution (MIOpen through
    `nn.Conv{2,3}d`).  The offset convolution uses the layer's kernel size, stride and padding
    with dilation 1: its output then has the layer's (dilation-blind) output size for every
    dilation, which the callers' own construction only achieves for dilation 1.
    `zero_init_offset=True` starts from zero offsets (the layer then equals a plain convolution
    sampled at the integer taps); the default keeps PyTorch's initialisation, as the reference's
    callers do.  Parameters: `weight`, `bias` (as ConvOffsetNd) and `conv_offset.weight`."""
    _conv = None
    _nd = None

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 channel_per_group=1, bias=True, groups=1, zero_init_offset=False, device=None, dtype=None,
                 standard_output_size=False, oob_offset_grad="reference"):
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, channel_per_group,
                         bias, groups, device=device, dtype=dtype, standard_output_size=standard_output_size,
                         oob_offset_grad=oob_offset_grad)
        if in_channels % channel_per_group != 0:
            raise ValueError('in_channels must be divisible by channel_per_group')
        taps = 1
        for k in self.kernel_size:
            taps *= k
        # with the standard output size the offset convolution takes the layer's dilation as well
        self.conv_offset = self._conv(in_channels, in_channels // channel_per_group * self._nd * taps,
                                      self.kernel_size, self.stride, self.padding,
                                      self.dilation if self.standard_output_size else 1, bias=False,
                                      device=device, dtype=dtype)
        if zero_init_offset:
            nn.init.zeros_(self.conv_offset.weight)

    def forward(self, input):
        return super().forward(input, self.conv_offset(input))


class ConvOffset3d(_ConvOffsetNd):
    _tuple = staticmethod(_triple)
    _function = ConvOffset3dFunction


class ConvOffset2d(_ConvOffsetNd):
    _tuple = staticmethod(_pair)
    _function = ConvOffset2dFunction


class ConvOffset3dPack(_ConvOffsetPackNd):
    _tuple = staticmethod(_triple)
    _function = ConvOffset3dFunction
    _conv = nn.Conv3d
    _nd = 3


class ConvOffset2dPack(_ConvOffsetPackNd):
    _tuple = staticmethod(_pair)
    _function = ConvOffset2dFunction
    _conv = nn.Conv2d
    _nd = 2
