"""autograd Functions of the deformable convolution, mirroring the reference's
`ConvOffset3dFunction` (deform3d/deform_conv3d_functions/deform_conv3d_function.py:7-77) and
`ConvOffset2dFunction` (deform2d_double/deform_conv2d_functions/deform_conv2d_function.py:7-77;
deform2d/deform_conv2d_functions/deform_conv2d_function.py:7-57 is its float, dilation-1,
group-1, bias-free subset).

Same call shape: `Fn.apply(inputs, offset, weight, bias=None, stride, padding, dilation,
channel_per_group=1, group=1)` (plus two optional trailing arguments: `standard_output_size`, see
`output_size`, and `oob_offset_grad`: 'reference' keeps the 3-D kernels' +-|grad column| term in
grad_offset for samples outside the input (deform3d/lib/deform_conv3d_cuda_kernel.cu:470-481), 'zero'
leaves it out, which makes grad_offset the derivative of the forward pass everywhere); same
dilation-blind output size by default; same shape checks and messages
as the reference's `shape_check` (deform3d/lib/deform_conv3d_cuda.cpp:24-87), raised as
RuntimeError.  Differences: no column workspace is kept on ctx (the kernels never build one),
float32 and float64 are served by the same class for both 2-D and 3-D, and gradients that are
not required come back as None instead of crashing (the reference wraps None in Variable, :76).
All tensors must live on one MI355X; there is no CPU path.
"""
import os

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib

_SUFFIX = {torch.float32: "f32", torch.float64: "f64", torch.bfloat16: "bf16", torch.float16: "f16"}


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _ntuple(v, nd):
    if isinstance(v, int):
        return (v,) * nd
    v = tuple(int(x) for x in v)
    _check(len(v) == nd, "expected %d values, got %r" % (nd, v))
    return v


def output_size(in_sizes, kernel, stride, padding, dilation=None, standard=False):
    """The reference formula, dilation not included (deform3d/lib/deform_conv3d_cuda.cpp:15-17;
    deform_conv3d_function.py:26-27).  `standard=True` gives the usual dilation-aware size
    `(in + 2p - d(k-1) - 1) // s + 1` instead (the one the reference's plain convolution uses,
    conv2d/lib/conv2d_cuda.cpp:20-22): with it every tap of every output position starts inside
    the padded input, as in an ordinary convolution."""
    if standard:
        dilation = dilation if dilation is not None else (1,) * len(kernel)
        return tuple((i + 2 * p - d * (k - 1) - 1) // s + 1
                     for i, k, s, p, d in zip(in_sizes, kernel, stride, padding, dilation))
    return tuple((i + 2 * p - k) // s + 1 for i, k, s, p in zip(in_sizes, kernel, stride, padding))


_OUT_MSG = {3: ("error output ll", "error outhh", "error outww"), 2: ("error outhh", "error outww")}
_OFF_MSG = {3: ("off l", "off h", "off w"), 2: ("off h", "off w")}


def shape_check(nd, inputs, weight, offset, output_shape, channel_per_group, group, stride, padding,
                dilation=None, standard=False):
    """Python restatement of the reference's shape_check with its messages."""
    _check(weight.dim() == nd + 2, "kernel dim")
    _check(inputs.dim() == nd + 2, "input dim")
    _check(inputs.size(1) == weight.size(1) * group, "input c != kernel c")
    _check(len(output_shape) == nd + 2, "output dim")
    _check(output_shape[0] == inputs.size(0), "output b != input b")
    _check(output_shape[1] == weight.size(0), "ou c != ker c")
    _check(offset.dim() == nd + 2, "off dim")
    _check(offset.size(0) == inputs.size(0), "off batch")
    kV = 1
    for k in weight.shape[2:]:
        kV *= k
    _check(channel_per_group > 0 and inputs.size(1) % channel_per_group == 0, "off channel")
    _check(offset.size(1) == inputs.size(1) // channel_per_group * nd * kV, "off channel")
    for a in range(nd):
        _check(offset.size(2 + a) == output_shape[2 + a], _OFF_MSG[nd][a])
    want = output_size(inputs.shape[2:], weight.shape[2:], stride, padding, dilation, standard)
    for a in range(nd):
        _check(inputs.size(2 + a) + 2 * padding[a] - weight.size(2 + a) >= 0 and want[a] >= 1 and
               want[a] == output_shape[2 + a], _OUT_MSG[nd][a])
    _check(group > 0 and weight.size(0) % group == 0, "ou c != ker c")


def _device_check(*tensors):
    t0 = tensors[0]
    _check(t0.is_cuda, "deformable convolution runs on the GPU only: tensors must be on a HIP device "
                       "(there is no CPU path in this package)")
    _check(t0.dtype in _SUFFIX, "dtype must be float32, float64, bfloat16 or float16")
    for t in tensors[1:]:
        if t is None:
            continue
        _check(t.device == t0.device, "all tensors must be on the same GPU")
        _check(t.dtype == t0.dtype, "all tensors must have the same dtype")


def _geom(nd, inputs, weight, out_sizes, stride, padding, dilation, channel_per_group, group):
    return ([inputs.size(0), inputs.size(1), weight.size(0)] + list(inputs.shape[2:]) + list(out_sizes) +
            list(weight.shape[2:]) + list(padding) + list(stride) + list(dilation) + [channel_per_group, group])


def _workspace_bytes(inputs, weight, group, out_sizes, channel_per_group):
    L = _lib.load()
    kV = inV = outV = 1
    for k in weight.shape[2:]:
        kV *= k
    for v in inputs.shape[2:]:
        inV *= v
    for v in out_sizes:
        outV *= v
    return int(L.dcn_workspace_bytes_for(inputs.element_size(), inputs.size(0), inputs.size(1), weight.size(0), inV, outV,
                                         kV, group, channel_per_group))


def _workspace(inputs, weight, group, out_sizes, channel_per_group):
    nbytes = _workspace_bytes(inputs, weight, group, out_sizes, channel_per_group)
    return torch.empty(max(nbytes, 1), dtype=torch.uint8, device=inputs.device), nbytes


def _stream():
    return torch.cuda.current_stream().cuda_stream


class _on_device:
    """`with torch.cuda.device(d)` only when d is not the current device (the context manager costs
    several microseconds, which shows on small layers)."""

    def __init__(self, device):
        self.ctx = None if torch.cuda.current_device() == device.index else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


# DCN_OVERLAP_BACKWARD=1: backward_weight next to backward_input_offset on a second stream (default: one stream)
_OVERLAP_BACKWARD = os.environ.get("DCN_OVERLAP_BACKWARD", "0") == "1"
_SIDE_STREAMS = {}


def _side_stream(device):
    """One extra stream per device, default priority, created on first use."""
    key = torch.device(device).index
    if key not in _SIDE_STREAMS:
        _SIDE_STREAMS[key] = torch.cuda.Stream(device=device)
    return _SIDE_STREAMS[key]


# Checked layer geometries: (output sizes, the C ABI's geometry arguments, workspace bytes) per
# (shapes, dtype, parameters).  A layer that passed the shape checks once skips them afterwards.
_PLANS = {}


def _plan(nd, inputs, offset, weight, out_shape, stride, padding, dilation, channel_per_group, group, standard):
    key = (nd, inputs.dtype, inputs.shape, offset.shape, weight.shape, out_shape, stride, padding, dilation,
           channel_per_group, group, standard)
    plan = _PLANS.get(key)
    if plan is None:
        _check(inputs.dim() == nd + 2, "input dim")
        _check(weight.dim() == nd + 2, "kernel dim")
        outs = output_size(inputs.shape[2:], weight.shape[2:], stride, padding, dilation, standard)
        shape = (inputs.size(0), weight.size(0)) + outs if out_shape is None else tuple(out_shape)
        shape_check(nd, inputs, weight, offset, shape, channel_per_group, group, stride, padding, dilation, standard)
        outs = tuple(shape[2:])
        plan = (shape, tuple(_geom(nd, inputs, weight, outs, stride, padding, dilation, channel_per_group, group)),
                _workspace_bytes(inputs, weight, group, outs, channel_per_group))
        if len(_PLANS) > 4096:
            _PLANS.clear()
        _PLANS[key] = plan
    return plan


def _forward(nd, inputs, offset, weight, bias, stride, padding, dilation, channel_per_group, group, standard=False):
    L = _lib.load()
    stride, padding, dilation = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(dilation, nd)
    _device_check(inputs, offset, weight, bias)
    out_shape, geom, ws_bytes = _plan(nd, inputs, offset, weight, None, stride, padding, dilation, channel_per_group, group,
                                      standard)
    if bias is not None:
        _check(bias.dim() == 1 and bias.size(0) == weight.size(0), "bias size")
    inputs, offset, weight = inputs.contiguous(), offset.contiguous(), weight.contiguous()
    device = inputs.device
    output = torch.empty(out_shape, dtype=inputs.dtype, device=device)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=device)
    fn = getattr(L, "dcn%dd_forward_%s" % (nd, _SUFFIX[inputs.dtype]))
    with _on_device(device):
        rc = fn(inputs.data_ptr(), weight.data_ptr(), offset.data_ptr(),
                bias.contiguous().data_ptr() if bias is not None else None, output.data_ptr(),
                *geom, ws.data_ptr(), ws_bytes, torch.cuda.current_stream(device).cuda_stream)
    _lib.check(rc)
    return output


def _backward(nd, inputs, offset, weight, grad_output, stride, padding, dilation, channel_per_group, group,
              need_data, need_weight, standard=False, oob_zero=False):
    L = _lib.load()
    _device_check(inputs, offset, weight, grad_output)
    _, geom, ws_bytes = _plan(nd, inputs, offset, weight, grad_output.shape, stride, padding, dilation, channel_per_group,
                              group, standard)
    inputs, offset, weight = inputs.contiguous(), offset.contiguous(), weight.contiguous()
    grad_output = grad_output.contiguous()
    suf = _SUFFIX[inputs.dtype]
    device = inputs.device
    grad_input = grad_offset = grad_weight = None
    with _on_device(device):
        main = torch.cuda.current_stream(device)
        # The two backward calls are independent.  On request (DCN_OVERLAP_BACKWARD=1) backward_weight
        # runs on a second stream of the same priority with a workspace of its own.  It is off by
        # default: a workgroup of the fused backward kernel takes nearly all of a CU's LDS, so the
        # two kernels never share a CU; they only take turns, which upsets the order in which the
        # fused kernel works through its items (whole rounds first, split items last) and measured
        # slower than one stream (4.02 against 3.69 ms per step at 64 -> 64 channels, 16x56x56).
        side = _side_stream(device) if (need_data and need_weight and _OVERLAP_BACKWARD) else None
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=device)
        ws_w = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=device) if side is not None else ws
        if need_weight:
            grad_weight = torch.zeros_like(weight)          # beta = 1 accumulation, as in the reference
        if need_data:
            # the kernels accumulate into grad_input (as the reference's atomicAdd does) and store
            # every element of grad_offset
            grad_input = torch.zeros_like(inputs)
            grad_offset = torch.empty_like(offset)
        if side is not None:
            side.wait_stream(main)           # the operands and the zero fills above are ready
        if need_data:
            args = (inputs.data_ptr(), weight.data_ptr(), offset.data_ptr(), grad_output.data_ptr(),
                    grad_input.data_ptr(), grad_offset.data_ptr(), *geom, ws.data_ptr(), ws_bytes, main.cuda_stream)
            if nd == 3 and oob_zero:        # the reference's 2-D kernels have no out-of-range term
                _check(suf in ("f32", "f64"), "oob_offset_grad='zero' is available in float32 and float64 only")
                _lib.check(getattr(L, "dcn3d_backward_input_offset_flags_%s" % suf)(*args, _lib.FLAG_OOB_OFFSET_GRAD_ZERO))
            else:
                _lib.check(getattr(L, "dcn%dd_backward_input_offset_%s" % (nd, suf))(*args))
        if need_weight:
            fn = getattr(L, "dcn%dd_backward_weight_%s" % (nd, suf))
            _lib.check(fn(inputs.data_ptr(), offset.data_ptr(), grad_output.data_ptr(), grad_weight.data_ptr(),
                          *geom, ws_w.data_ptr(), ws_bytes, (side or main).cuda_stream))
        if side is not None:
            main.wait_stream(side)           # everything issued later on the caller's stream sees grad_weight
    return grad_input, grad_offset, grad_weight


class _ConvOffsetNdFunction(Function):
    ND = 0

    @classmethod
    def _fwd(cls, ctx, inputs, offset, weight, bias, stride, padding, dilation, channel_per_group, group,
             standard_output_size=False, oob_offset_grad="reference"):
        nd = cls.ND
        ctx.standard = bool(standard_output_size)
        if oob_offset_grad not in ("reference", "zero"):
            raise ValueError("oob_offset_grad must be 'reference' or 'zero'")
        ctx.oob_zero = oob_offset_grad == "zero"
        ctx.stride, ctx.padding, ctx.dilation = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(dilation, nd)
        ctx.channel_per_group, ctx.group = int(channel_per_group), int(group)
        ctx.has_bias = bias is not None
        ctx.save_for_backward(inputs, offset, weight)
        return _forward(nd, inputs, offset, weight, bias, ctx.stride, ctx.padding, ctx.dilation,
                        ctx.channel_per_group, ctx.group, ctx.standard)

    @classmethod
    def _bwd(cls, ctx, grad_output):
        inputs, offset, weight = ctx.saved_tensors
        need = ctx.needs_input_grad
        # grad_input and grad_offset come out of one kernel, as in the reference (:52)
        gi, go, gw = _backward(cls.ND, inputs, offset, weight, grad_output, ctx.stride, ctx.padding, ctx.dilation,
                               ctx.channel_per_group, ctx.group, need[0] or need[1], need[2], ctx.standard,
                               ctx.oob_zero)
        gb = None
        if ctx.has_bias and need[3]:
            gb = grad_output.sum(dim=[0] + list(range(2, 2 + cls.ND)))
        return (gi if need[0] else None, go if need[1] else None, gw, gb, None, None, None, None, None, None, None)


class ConvOffset3dFunction(_ConvOffsetNdFunction):
    ND = 3

    @staticmethod
    def forward(ctx, inputs, offset, weight, bias=None, stride=(1, 1, 1), padding=(0, 0, 0), dilation=(1, 1, 1),
                channel_per_group=1, group=1, standard_output_size=False, oob_offset_grad="reference"):
        return ConvOffset3dFunction._fwd(ctx, inputs, offset, weight, bias, stride, padding, dilation,
                                         channel_per_group, group, standard_output_size, oob_offset_grad)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        return ConvOffset3dFunction._bwd(ctx, grad_output)


class ConvOffset2dFunction(_ConvOffsetNdFunction):
    ND = 2

    @staticmethod
    def forward(ctx, inputs, offset, weight, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
                channel_per_group=1, group=1, standard_output_size=False, oob_offset_grad="reference"):
        return ConvOffset2dFunction._fwd(ctx, inputs, offset, weight, bias, stride, padding, dilation,
                                         channel_per_group, group, standard_output_size, oob_offset_grad)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        return ConvOffset2dFunction._bwd(ctx, grad_output)
