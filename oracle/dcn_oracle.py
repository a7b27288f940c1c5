"""ctypes front end of the CPU oracle (oracle/dcn_oracle.cpp).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module; the
shipped package never does.  Tensors are CPU torch tensors (float32 or float64, contiguous).

The Python-side semantics follow the reference's autograd Functions
(deform3d/deform_conv3d_functions/deform_conv3d_function.py:26-32,41-42,52-77 and
deform2d_double/deform_conv2d_functions/deform_conv2d_function.py:25-31,41-42,52-77):
dilation-blind output size, zero-filled outputs, bias added after the GEMMs, grad_bias as the
sum of grad_output over everything but channels.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libdcn_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.dcn_oracle_output_size.restype = ctypes.c_int
        _lib = L
    return _lib


def _tup(v, nd):
    if isinstance(v, int):
        return (v,) * nd
    v = tuple(int(x) for x in v)
    assert len(v) == nd
    return v


def output_size(in_sizes, k, stride, pad):
    L = lib()
    return tuple(L.dcn_oracle_output_size(int(i), int(p), int(kk), int(s))
                 for i, p, kk, s in zip(in_sizes, pad, k, stride))


def geometry(inputs, weight, stride, padding, dilation, channel_per_group, group):
    """Returns (nd, 24-int ctypes array, out_sizes)."""
    nd = inputs.dim() - 2
    assert nd in (2, 3)
    stride, padding, dilation = _tup(stride, nd), _tup(padding, nd), _tup(dilation, nd)
    ins = tuple(inputs.shape[2:])
    ks = tuple(weight.shape[2:])
    outs = output_size(ins, ks, stride, padding)
    pad3 = lambda t, fill: (fill,) * (3 - nd) + tuple(t)
    g = [nd, inputs.shape[0], inputs.shape[1], weight.shape[0]]
    g += pad3(ins, 1) + pad3(outs, 1) + pad3(ks, 1) + pad3(padding, 0) + pad3(stride, 1) + pad3(dilation, 1)
    g += [int(channel_per_group), int(group)]
    return nd, (ctypes.c_int * 24)(*[int(x) for x in g]), outs


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _dt(t):
    assert t.dtype in (torch.float32, torch.float64) and t.is_contiguous() and t.device.type == "cpu"
    return 0 if t.dtype == torch.float32 else 1


def _columns(inputs, weight, outs):
    kV = 1
    for k in weight.shape[2:]:
        kV *= k
    outV = 1
    for o in outs:
        outV *= o
    return inputs.new_zeros(inputs.shape[1] * kV, outV)


def forward(inputs, offset, weight, bias=None, stride=1, padding=0, dilation=1,
            channel_per_group=1, group=1, acc64=True):
    nd, geom, outs = geometry(inputs, weight, stride, padding, dilation, channel_per_group, group)
    dt = _dt(inputs)
    assert _dt(offset) == dt and _dt(weight) == dt
    kV = weight[0, 0].numel()
    assert inputs.shape[1] == weight.shape[1] * group, "input c != kernel c"
    assert tuple(offset.shape) == (inputs.shape[0], inputs.shape[1] // channel_per_group * nd * kV) + outs, "off shape"
    out = inputs.new_zeros((inputs.shape[0], weight.shape[0]) + outs)
    col = _columns(inputs, weight, outs)
    lib().dcn_oracle_forward(dt, int(acc64), geom, _p(inputs), _p(weight), _p(offset), _p(out), _p(col))
    if bias is not None:
        out += bias.view((1, -1) + (1,) * nd)
    return out


def backward(inputs, offset, weight, grad_output, bias=None, stride=1, padding=0, dilation=1,
             channel_per_group=1, group=1, acc64=True):
    """Returns (grad_input, grad_offset, grad_weight, grad_bias or None)."""
    nd, geom, outs = geometry(inputs, weight, stride, padding, dilation, channel_per_group, group)
    dt = _dt(inputs)
    grad_output = grad_output.contiguous()
    assert tuple(grad_output.shape) == (inputs.shape[0], weight.shape[0]) + outs
    col = _columns(inputs, weight, outs)
    gin = torch.zeros_like(inputs)
    goff = torch.zeros_like(offset)
    gw = torch.zeros_like(weight)
    L = lib()
    L.dcn_oracle_backward_input_offset(dt, int(acc64), geom, _p(inputs), _p(weight), _p(offset),
                                       _p(grad_output), _p(gin), _p(goff), _p(col))
    L.dcn_oracle_backward_weight(dt, int(acc64), geom, _p(inputs), _p(offset), _p(grad_output),
                                 _p(gw), _p(col))
    gb = None
    if bias is not None:
        gb = grad_output.sum(dim=[0] + list(range(2, 2 + nd)))
    return gin, goff, gw, gb


# --- single stages on one sample (no batch dim), for pinning each part on its own -------------

def im2col(im, off, weight_shape, stride, padding, dilation, channel_per_group):
    """im [C,(D,)H,W], off [DG*kV*nd, *out] -> col [C*kV, outV]."""
    x = im.unsqueeze(0)
    w = im.new_zeros((1, im.shape[0]) + tuple(weight_shape))
    nd, geom, outs = geometry(x, w, stride, padding, dilation, channel_per_group, 1)
    col = _columns(x, w, outs)
    lib().dcn_oracle_im2col(_dt(im), geom, _p(im), _p(off), _p(col))
    return col


def col2im_input(col, off, im_shape, weight_shape, stride, padding, dilation, channel_per_group):
    x = col.new_zeros((1,) + tuple(im_shape))
    w = col.new_zeros((1, im_shape[0]) + tuple(weight_shape))
    nd, geom, outs = geometry(x, w, stride, padding, dilation, channel_per_group, 1)
    gim = col.new_zeros(tuple(im_shape))
    lib().dcn_oracle_col2im_input(_dt(col), geom, _p(col), _p(off), _p(gim))
    return gim


def col2im_offset(col, im, off, weight_shape, stride, padding, dilation, channel_per_group):
    x = im.unsqueeze(0)
    w = im.new_zeros((1, im.shape[0]) + tuple(weight_shape))
    nd, geom, outs = geometry(x, w, stride, padding, dilation, channel_per_group, 1)
    goff = torch.zeros_like(off)
    lib().dcn_oracle_col2im_offset(_dt(col), geom, _p(col), _p(im), _p(off), _p(goff))
    return goff


# --- the reference's sequencing with the host BLAS for its three GEMMs ------------------------
# deform3d/lib/deform_conv3d_cuda.cpp:105-158 (forward), :186-253 (backward to input and offset) and
# :278-330 (backward to weight) loop over the samples, build the column buffer of a sample with
# deformable_im2col, and call one cuBLAS GEMM per convolution group.  This is that loop with
# torch.mm (the host BLAS) in the place of cuBLAS and the oracle's C++ stages for the rest; the
# benchmark times it as the CPU baseline.

def step_blas(inputs, offset, weight, grad_output, stride=1, padding=0, dilation=1, channel_per_group=1, group=1):
    """Forward + backward of the reference algorithm on the host: (output, grad_input, grad_offset, grad_weight)."""
    N, C_in, C_out = inputs.shape[0], inputs.shape[1], weight.shape[0]
    wshape = tuple(weight.shape[2:])
    kV = weight[0, 0].numel()
    M, Kg = C_out // group, (C_in // group) * kV
    w2 = weight.reshape(group, M, Kg)
    out = gin = goff = None
    gw = torch.zeros_like(w2)
    for n in range(N):
        col = im2col(inputs[n], offset[n], wshape, stride, padding, dilation, channel_per_group)      # [C_in*kV, outV]
        outV = col.shape[1]
        if out is None:
            outs = tuple(grad_output.shape[2:])
            out = inputs.new_empty((N, C_out) + outs)
            gin, goff = torch.zeros_like(inputs), torch.zeros_like(offset)
        colg = col.view(group, Kg, outV)
        go = grad_output[n].reshape(group, M, outV)
        gcol = torch.empty_like(colg)
        for g in range(group):
            out[n].view(group, M, outV)[g] = torch.mm(w2[g], colg[g])              # G1
            gcol[g] = torch.mm(w2[g].t(), go[g])                                   # G2
            gw[g] += torch.mm(go[g], colg[g].t())                                  # G3 (the reference rebuilds the columns first)
        gcol = gcol.view(C_in * kV, outV)
        gin[n] = col2im_input(gcol, offset[n], inputs.shape[1:], wshape, stride, padding, dilation, channel_per_group)
        goff[n] = col2im_offset(gcol, inputs[n], offset[n], wshape, stride, padding, dilation, channel_per_group)
    return out, gin, goff, gw.view_as(weight)
