"""The reference-shaped binding (tests/reference_binding.py: the three symbols of
deform3d/lib/deform_conv3d_cuda.h:12-34 in the reference's argument order) driven in the order
and with the buffers the reference's Function uses
(deform3d/deform_conv3d_functions/deform_conv3d_function.py:20-77): a column buffer that is
allocated and passed but never used, zero-filled grad_input / grad_offset / grad_weight, bias
added by the caller, return value 1.  Results are compared with the CPU oracle to the float32
tolerances (1e-4 forward, 1e-3 gradients, relative to the largest reference value).
"""
import pytest
import torch

from oracle import dcn_oracle as orc
from tests.cases import make_case

pytestmark = pytest.mark.gpu

#  N, Cin, Cout, in, k, stride, pad, dil, cpg, groups, off_scale
CASES = {
    "gradient_script_shape": (2, 2, 4, 7, 3, 2, 2, 2, 2, 2, 1.0),           # deform3d/test_gradient.py:9-20
    "two_deformable_groups": (2, 12, 10, (5, 9, 8), 3, 1, 1, 1, 6, 1, 2.0),
    "groups_rect_kernel": (1, 6, 3, (4, 7, 5), (2, 3, 1), (1, 2, 1), (1, 2, 0), (1, 2, 1), 2, 3, 2.0),
}


def _rel(got, want):
    scale = want.abs().max().item()
    return (got.cpu().double() - want.double()).abs().max().item() / (scale if scale > 0 else 1.0)


@pytest.mark.parametrize("name", sorted(CASES))
def test_reference_call_sequence_matches_oracle(name):
    from tests import reference_binding as op
    print("reference binding", name, flush=True)
    c = make_case(3, *CASES[name], dtype=torch.float32, seed=5)
    dev = torch.device("cuda:0")
    inputs, offset, weight, bias, grad_output = (c[k].to(dev) for k in ("x", "off", "w", "b", "gout"))
    pad, stride, dil, cpg, group = c["pad"], c["stride"], c["dil"], c["cpg"], c["groups"]
    tail = (*pad, *stride, *dil, cpg, group)

    output = inputs.new_zeros((inputs.size(0), weight.size(0)) + c["outs"])
    columns = inputs.new_zeros(inputs.size(1) * weight[0, 0].numel(), output[0, 0].numel())
    assert op.deform_conv_forward_cuda(inputs, weight, offset, columns, output, *tail) == 1
    output += bias.view((1, -1, 1, 1, 1)).expand_as(output)

    grad_input, grad_offset = torch.zeros_like(inputs), torch.zeros_like(offset)
    assert op.deform_conv_backward_input_offset_cuda(inputs, weight, offset, grad_output, columns, grad_input,
                                                     grad_offset, *tail) == 1
    grad_weight = torch.zeros_like(weight)
    assert op.deform_conv_backward_weight_cuda(inputs, offset, grad_output, columns, grad_weight, *tail) == 1
    torch.cuda.synchronize()
    assert float(columns.abs().max()) == 0.0          # the column buffer is never touched

    cfg = (c["stride"], c["pad"], c["dil"], cpg, group)
    want_out = orc.forward(c["x"], c["off"], c["w"], c["b"], *cfg)
    want_gin, want_goff, want_gw, _ = orc.backward(c["x"], c["off"], c["w"], c["gout"], c["b"], *cfg)
    assert _rel(output, want_out) <= 1e-4
    assert _rel(grad_input, want_gin) <= 1e-3
    assert _rel(grad_offset, want_goff) <= 1e-3
    assert _rel(grad_weight, want_gw) <= 1e-3


def test_reference_binding_raises_on_inconsistent_extents():
    from tests import reference_binding as op
    dev = torch.device("cuda:0")
    inputs = torch.zeros(1, 4, 5, 5, 5, device=dev)
    weight = torch.zeros(4, 4, 3, 3, 3, device=dev)
    offset = torch.zeros(1, 81, 5, 5, 5, device=dev)
    output = torch.zeros(1, 4, 4, 5, 5, device=dev)          # output length 4 where the formula gives 5
    columns = torch.zeros(1, device=dev)
    with pytest.raises(RuntimeError, match="error output ll"):
        op.deform_conv_forward_cuda(inputs, weight, offset, columns, output, 1, 1, 1, 1, 1, 1, 1, 1, 1, 4, 1)


#  N, Cin, Cout, in, k, stride, pad, dil, cpg, groups, off_scale
CASES_2D_DOUBLE = {
    "gradient_script_shape": (2, 2, 4, 7, 1, 2, 2, 2, 2, 2, 1.0),           # deform2d_double/test_gradient.py:7-19
    "dilated_grouped": (1, 16, 8, 10, 3, 1, 2, 2, 4, 2, 3.0),
    "rect_kernel": (1, 6, 4, (8, 6), (3, 2), (2, 1), (2, 1), (2, 1), 3, 1, 2.0),
}
CASES_2D_FLOAT = {                                                          # dilation 1, one group: all the float package has
    "model_script_like": (2, 8, 6, (9, 10), 3, 1, 1, 1, 4, 1, 2.0),         # deform2d/test_model.py: 3x3, pad 1
    "strided": (1, 6, 5, (11, 8), (3, 2), (2, 1), (1, 0), 1, 6, 1, 1.5),
}


def _drive_2d(op, c, tail, dtype, tol_fwd, tol_grad, bias):
    dev = torch.device("cuda:0")
    inputs, offset, weight, grad_output = (c[k].to(dev) for k in ("x", "off", "w", "gout"))
    output = inputs.new_zeros((inputs.size(0), weight.size(0)) + c["outs"])
    columns = inputs.new_zeros(weight.size(1) * weight[0, 0].numel(), output[0, 0].numel())
    assert op.deform_conv_forward_cuda(inputs, weight, offset, columns, output, *tail) == 1
    if bias:
        output += c["b"].to(dev).view((1, -1, 1, 1)).expand_as(output)
    grad_input, grad_offset = torch.zeros_like(inputs), torch.zeros_like(offset)
    assert op.deform_conv_backward_input_offset_cuda(inputs, weight, offset, grad_output, columns, grad_input,
                                                     grad_offset, *tail) == 1
    grad_weight = torch.zeros_like(weight)
    assert op.deform_conv_backward_weight_cuda(inputs, offset, grad_output, columns, grad_weight, *tail) == 1
    torch.cuda.synchronize()
    assert float(columns.abs().max()) == 0.0
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    b = c["b"] if bias else None
    want_out = orc.forward(c["x"], c["off"], c["w"], b, *cfg)
    want_gin, want_goff, want_gw, _ = orc.backward(c["x"], c["off"], c["w"], c["gout"], b, *cfg)
    assert _rel(output, want_out) <= tol_fwd
    assert _rel(grad_input, want_gin) <= tol_grad
    assert _rel(grad_offset, want_goff) <= tol_grad
    assert _rel(grad_weight, want_gw) <= tol_grad


@pytest.mark.parametrize("name", sorted(CASES_2D_DOUBLE))
def test_reference_call_sequence_2d_double(name):
    """deform2d_double's three symbols (deform2d_double/lib/deform_conv2d_cuda.h:12-34) in the order of
    deform2d_double/deform_conv2d_functions/deform_conv2d_function.py:20-77, float64 to 1e-10."""
    from tests.reference_binding import deform_conv2d_double_op as op
    print("reference binding 2-D double", name, flush=True)
    c = make_case(2, *CASES_2D_DOUBLE[name], dtype=torch.float64, seed=7)
    tail = (*c["pad"], *c["stride"], *c["dil"], c["cpg"], c["groups"])
    _drive_2d(op, c, tail, torch.float64, 1e-10, 1e-10, bias=True)


@pytest.mark.parametrize("name", sorted(CASES_2D_FLOAT))
def test_reference_call_sequence_2d_float(name):
    """deform2d's three symbols (deform2d/lib/deform_conv2d_cuda.h:12-31: no dilation, no groups, no
    bias) in the order of deform2d/deform_conv2d_functions/deform_conv2d_function.py:14-57."""
    from tests.reference_binding import deform_conv2d_float_op as op
    print("reference binding 2-D float", name, flush=True)
    c = make_case(2, *CASES_2D_FLOAT[name], dtype=torch.float32, seed=8)
    tail = (*c["pad"], *c["stride"], c["cpg"])
    _drive_2d(op, c, tail, torch.float32, 1e-4, 1e-3, bias=False)
