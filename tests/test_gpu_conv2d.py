"""The plain convolution row (the reference's conv2d package) on the GPU: `Conv2d` / `Conv2dFunction`
against torch's own convolution on the shape of the reference's script (conv2d/test_model.py:8-49:
batch 2, 4 -> 8 channels, 75 x 75, kernel 3, stride 1, pad 1, dilation 3, 4 groups, all-ones
grad_output) and against the CPU oracle's deformable layer at zero offsets (the two are the same
arithmetic; the oracle's output is cropped to the dilation-aware size).  float32 to 1e-4 forward /
1e-3 gradients of the tensor's largest value, float64 to 1e-10."""
import pytest
import torch
import torch.nn.functional as F

from oracle import dcn_oracle as orc

pytestmark = pytest.mark.gpu

#        N, Cin, Cout, in, k, stride, pad, dil, groups
CASES = {
    "reference_script": (2, 4, 8, (75, 75), 3, 1, 1, 3, 4),               # conv2d/test_model.py:8-19
    "strided_rect": (3, 6, 10, (17, 12), (3, 2), (2, 1), (1, 0), (1, 2), 2),
    "wide": (1, 48, 40, (20, 22), 3, 1, 1, 1, 1),
}


def _rel(got, want):
    scale = want.abs().max().item()
    return (got.detach().cpu().double() - want.detach().cpu().double()).abs().max().item() / (scale if scale > 0 else 1.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_conv2d_matches_torch_and_zero_offset_oracle(name, dtype):
    import deform_conv3d_pytorch_op_amd as dcn
    print("conv2d", name, dtype, flush=True)
    N, cin, cout, ins, k, stride, pad, dil, groups = CASES[name]
    tol_f, tol_g = (1e-4, 1e-3) if dtype == torch.float32 else (1e-10, 1e-10)
    dev = torch.device("cuda:0")
    torch.manual_seed(1)
    m = dcn.Conv2d(cin, cout, k, stride, pad, dil, bias=True, groups=groups, device=dev, dtype=dtype)
    x = torch.randn((N, cin) + ins, dtype=dtype, device=dev, requires_grad=True)
    y = m(x)
    gout = torch.ones_like(y) if name == "reference_script" else torch.randn_like(y)
    y.backward(gout)
    torch.cuda.synchronize()
    # torch's convolution in float64 on the host
    xr = x.detach().cpu().double().requires_grad_(True)
    wr = m.weight.detach().cpu().double().requires_grad_(True)
    br = m.bias.detach().cpu().double().requires_grad_(True)
    yr = F.conv2d(xr, wr, br, m.stride, m.padding, m.dilation, groups)
    assert tuple(y.shape) == tuple(yr.shape)
    yr.backward(gout.cpu().double())
    assert _rel(y, yr) <= tol_f
    assert _rel(x.grad, xr.grad) <= tol_g
    assert _rel(m.weight.grad, wr.grad) <= tol_g
    assert _rel(m.bias.grad, br.grad) <= tol_g
    # the oracle's deformable layer with zero offsets, cropped to the dilation-aware output size
    kk = m.kernel_size
    blind = tuple((i + 2 * p - kq) // s + 1 for i, kq, s, p in zip(ins, kk, m.stride, m.padding))
    off = torch.zeros((N, 2 * kk[0] * kk[1]) + blind, dtype=torch.float64)
    want = orc.forward(x.detach().cpu().double(), off, m.weight.detach().cpu().double(), m.bias.detach().cpu().double(),
                       m.stride, m.padding, m.dilation, cin, groups)
    assert _rel(y, want[:, :, :y.shape[2], :y.shape[3]]) <= tol_f


def test_conv2d_gating_and_errors():
    import deform_conv3d_pytorch_op_amd as dcn
    dev = torch.device("cuda:0")
    x = torch.randn(1, 4, 9, 9, device=dev)
    w = torch.randn(6, 2, 3, 3, device=dev, requires_grad=True)
    y = dcn.Conv2dFunction.apply(x, w, None, (1, 1), (1, 1), (1, 1), 2)      # no grad for the input
    y.sum().backward()
    assert w.grad is not None and x.grad is None
    with pytest.raises(RuntimeError, match="input c != kernel c"):
        dcn.Conv2dFunction.apply(x, torch.randn(6, 3, 3, 3, device=dev), None, (1, 1), (1, 1), (1, 1), 2)
    with pytest.raises(ValueError, match="in_channels must be divisible by groups"):
        dcn.Conv2d(5, 4, 3, groups=2)
