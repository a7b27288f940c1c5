"""Stand-ins for the reference's cffi modules: `deform_conv3d_op`
(deform3d/deform_conv3d_op/__init__.py:1-12; the three symbols of
deform3d/lib/deform_conv3d_cuda.h:12-34, the module-level functions below) and the two
`deform_conv2d_op` modules (deform2d_double/lib/deform_conv2d_cuda.h:12-34: double, with dilation and
groups -> class deform_conv2d_double_op; deform2d/lib/deform_conv2d_cuda.h:12-31: float, no dilation,
no groups -> class deform_conv2d_float_op), each with the reference's argument order, bound to
libdcn_amd.so with ctypes.  `columns` is accepted and ignored (no column buffer exists), the
return value is 1 as in the reference, and errors raise RuntimeError where the reference raises
through THError.  This is the file a maintainer of the reference would drop in to keep the
reference's own Function and Module code; tests/test_gpu_binding.py drives it the way
deform3d/deform_conv3d_functions/deform_conv3d_function.py:20-77 does.
"""
import ctypes

import torch

from deform_conv3d_pytorch_op_amd._lib import SO_PATH

_L = ctypes.CDLL(SO_PATH)
_L.dcn_workspace_bytes.restype = ctypes.c_size_t
_L.dcn_workspace_bytes.argtypes = [ctypes.c_int] * 4 + [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int]
_L.dcn_last_error.restype = ctypes.c_char_p
_vp = ctypes.c_void_p


def _geom(inp, weight, out, pad, stride, dil, cpg, group):
    return ([inp.size(0), inp.size(1), weight.size(0)] + list(inp.shape[2:]) + list(out.shape[2:]) +
            list(weight.shape[2:]) + list(pad) + list(stride) + list(dil) + [cpg, group])


def _workspace(inp, weight, out, group):
    n = _L.dcn_workspace_bytes(inp.element_size(), inp.size(0), inp.size(1), weight.size(0), inp[0, 0].numel(), out[0, 0].numel(),
                               weight[0, 0].numel(), group)
    return torch.empty(n, dtype=torch.uint8, device=inp.device), n


def _check(rc):
    if rc != 0:
        raise RuntimeError(_L.dcn_last_error().decode())


def _call(fn, ptrs, ints, ws, n):
    stream = torch.cuda.current_stream().cuda_stream
    _check(fn(*[_vp(p) for p in ptrs], *[ctypes.c_int(int(v)) for v in ints], _vp(ws.data_ptr()),
              ctypes.c_size_t(n), _vp(stream)))
    return 1


def deform_conv_forward_cuda(input, weight, offset, columns, output, pl, ph, pw, sl, sh, sw, dl, dh, dw, cpg, group):
    ws, n = _workspace(input, weight, output, group)
    return _call(_L.dcn3d_forward_f32,
                 [input.data_ptr(), weight.data_ptr(), offset.data_ptr(), None, output.data_ptr()],
                 _geom(input, weight, output, (pl, ph, pw), (sl, sh, sw), (dl, dh, dw), cpg, group), ws, n)


def deform_conv_backward_input_offset_cuda(input, weight, offset, grad_output, columns, grad_input, grad_offset,
                                           pl, ph, pw, sl, sh, sw, dl, dh, dw, cpg, group):
    ws, n = _workspace(input, weight, grad_output, group)       # grad_input must be zero-filled, as in the reference
    return _call(_L.dcn3d_backward_input_offset_f32,
                 [input.data_ptr(), weight.data_ptr(), offset.data_ptr(), grad_output.data_ptr(),
                  grad_input.data_ptr(), grad_offset.data_ptr()],
                 _geom(input, weight, grad_output, (pl, ph, pw), (sl, sh, sw), (dl, dh, dw), cpg, group), ws, n)


def deform_conv_backward_weight_cuda(input, offset, grad_output, columns, grad_weight,
                                     pl, ph, pw, sl, sh, sw, dl, dh, dw, cpg, group):
    ws, n = _workspace(input, grad_weight, grad_output, group)  # grad_weight is accumulated into (beta = 1)
    return _call(_L.dcn3d_backward_weight_f32,
                 [input.data_ptr(), offset.data_ptr(), grad_output.data_ptr(), grad_weight.data_ptr()],
                 _geom(input, grad_weight, grad_output, (pl, ph, pw), (sl, sh, sw), (dl, dh, dw), cpg, group), ws, n)


def _make_2d(suffix, with_dilation_and_groups):
    """The three symbols of a 2-D package as static methods, in the reference's argument order."""
    fwd = getattr(_L, "dcn2d_forward_" + suffix)
    bwd = getattr(_L, "dcn2d_backward_input_offset_" + suffix)
    bww = getattr(_L, "dcn2d_backward_weight_" + suffix)

    def split(tail):
        if with_dilation_and_groups:      # pad_h, pad_w, stride_h, stride_w, dilation_h, dilation_w, channel_per_deformable_group, group
            ph, pw, sh, sw, dh, dw, cpg, group = tail
        else:                             # pad_h, pad_w, stride_h, stride_w, channel_per_deformable_group
            ph, pw, sh, sw, cpg = tail
            dh = dw = group = 1
        return (ph, pw), (sh, sw), (dh, dw), cpg, group

    class Op:
        @staticmethod
        def deform_conv_forward_cuda(input, weight, offset, columns, output, *tail):
            pad, stride, dil, cpg, group = split(tail)
            ws, n = _workspace(input, weight, output, group)
            return _call(fwd, [input.data_ptr(), weight.data_ptr(), offset.data_ptr(), None, output.data_ptr()],
                         _geom(input, weight, output, pad, stride, dil, cpg, group), ws, n)

        @staticmethod
        def deform_conv_backward_input_offset_cuda(input, weight, offset, grad_output, columns, grad_input, grad_offset, *tail):
            pad, stride, dil, cpg, group = split(tail)
            ws, n = _workspace(input, weight, grad_output, group)
            return _call(bwd, [input.data_ptr(), weight.data_ptr(), offset.data_ptr(), grad_output.data_ptr(),
                               grad_input.data_ptr(), grad_offset.data_ptr()],
                         _geom(input, weight, grad_output, pad, stride, dil, cpg, group), ws, n)

        @staticmethod
        def deform_conv_backward_weight_cuda(input, offset, grad_output, columns, grad_weight, *tail):
            pad, stride, dil, cpg, group = split(tail)
            ws, n = _workspace(input, grad_weight, grad_output, group)
            return _call(bww, [input.data_ptr(), offset.data_ptr(), grad_output.data_ptr(), grad_weight.data_ptr()],
                         _geom(input, grad_weight, grad_output, pad, stride, dil, cpg, group), ws, n)
    return Op


deform_conv2d_double_op = _make_2d("f64", True)      # deform2d_double/lib/deform_conv2d_cuda.h:12-34
deform_conv2d_float_op = _make_2d("f32", False)      # deform2d/lib/deform_conv2d_cuda.h:12-31
