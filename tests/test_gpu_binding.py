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
