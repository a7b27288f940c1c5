"""CPU-side tests: the C-ABI library loads and exports every declared symbol, the Python front
end reproduces the reference's checks and messages, the oracle matches the committed fixtures.
No compute call is made on the HIP library here (there is no GPU)."""
import ctypes
import glob
import os
import re

import numpy as np
import pytest
import torch

from oracle import dcn_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from deform_conv3d_pytorch_op_amd import _lib
    L = _lib.load()
    header = open(os.path.join(ROOT, "include", "dcn_amd.h")).read()
    declared = set(re.findall(r"\b((?:dcn(?:2d|3d)?|conv2d)_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert L.dcn_version() == 1
    assert L.dcn_arch() == b"gfx950"
    assert L.dcn_last_error() == b""


def test_workspace_query():
    from deform_conv3d_pytorch_op_amd import _lib
    L = _lib.load()
    n4 = L.dcn_workspace_bytes(4, 2, 64, 64, 1000, 900, 27, 1)
    n8 = L.dcn_workspace_bytes(8, 2, 64, 64, 1000, 900, 27, 1)
    assert n4 >= 64 * 64 * 27 * 4 + 2 * 2 * 64 * 1000 * 4 and n8 >= 64 * 64 * 27 * 8 + 2 * 2 * 64 * 1000 * 8
    assert L.dcn_workspace_bytes(4, 2, 64, 64, 1000, 900, 27, 0) == 0


def test_argument_validation_needs_no_gpu():
    # validation runs before anything touches the device
    from deform_conv3d_pytorch_op_amd import _lib
    L = _lib.load()
    geom = [1, 4, 4, 6, 6, 5, 6, 3, 3, 1, 1, 1, 1, 1, 1, 4, 1]       # output_h 5 contradicts the formula (6)
    rc = L.dcn2d_forward_f32(None, None, None, None, None, *geom, None, 0, None)
    assert rc == -1 and L.dcn_last_error() == b"error outhh"
    geom[5] = 6
    rc = L.dcn2d_forward_f32(None, None, None, None, None, *geom, None, 0, None)
    assert rc == -1 and L.dcn_last_error() == b"null tensor pointer"
    geom[15] = 3                                                       # 4 channels, 3 per deformable group
    rc = L.dcn2d_backward_weight_f64(None, None, None, None, *geom, None, 0, None)
    assert rc == -1 and L.dcn_last_error() == b"off channel"


def test_front_end_checks_and_messages():
    import deform_conv3d_pytorch_op_amd as dcn
    from deform_conv3d_pytorch_op_amd.functions import shape_check, output_size
    x = torch.randn(1, 4, 6, 6)
    w = torch.randn(4, 4, 3, 3)
    off = torch.zeros(1, 18, 6, 6)
    ok = (1, 4, 6, 6)
    shape_check(2, x, w, off, ok, 4, 1, (1, 1), (1, 1))
    cases = [
        (dict(weight=torch.randn(4, 4, 3)), "kernel dim"),
        (dict(inputs=torch.randn(4, 6, 6)), "input dim"),
        (dict(group=2), "input c != kernel c"),
        (dict(output_shape=(2, 4, 6, 6)), "output b != input b"),
        (dict(output_shape=(1, 5, 6, 6)), "ou c != ker c"),
        (dict(offset=torch.zeros(1, 18, 6)), "off dim"),
        (dict(offset=torch.zeros(2, 18, 6, 6)), "off batch"),
        (dict(offset=torch.zeros(1, 17, 6, 6)), "off channel"),
        (dict(offset=torch.zeros(1, 18, 5, 6)), "off h"),
        (dict(offset=torch.zeros(1, 18, 6, 5)), "off w"),
        (dict(output_shape=(1, 4, 5, 6), offset=torch.zeros(1, 18, 5, 6)), "error outhh"),
    ]
    for kw, msg in cases:
        a = dict(inputs=x, weight=w, offset=off, output_shape=ok, channel_per_group=4, group=1)
        a.update(kw)
        with pytest.raises(RuntimeError, match=msg):
            shape_check(2, a["inputs"], a["weight"], a["offset"], a["output_shape"], a["channel_per_group"],
                        a["group"], (1, 1), (1, 1))
    # dilation-blind output size: in 28, k 3, pad 2, dilation 2 -> 30 (BASELINE configs[2])
    assert output_size((28, 28), (3, 3), (1, 1), (2, 2)) == (30, 30)
    assert output_size((16, 112, 112), (3, 3, 3), (1, 2, 2), (1, 1, 1)) == (16, 56, 56)
    with pytest.raises(ValueError, match="in_channels must be divisible by groups"):
        dcn.ConvOffset3d(3, 4, 3, groups=2)
    with pytest.raises(ValueError, match="out_channels must be divisible by groups"):
        dcn.ConvOffset2d(4, 3, 3, groups=2)
    m = dcn.ConvOffset3d(4, 6, (1, 3, 3), stride=(1, 2, 2), padding=1, channel_per_group=2, groups=2)
    assert m.kernel_size == (1, 3, 3) and m.stride == (1, 2, 2) and m.padding == (1, 1, 1) and m.group == 2
    assert tuple(m.weight.shape) == (6, 2, 1, 3, 3) and tuple(m.bias.shape) == (6,)
    assert float(m.bias.abs().max()) <= 0.1
    # CPU tensors are refused loudly: there is no CPU path in the package
    with pytest.raises(RuntimeError, match="GPU only"):
        m(torch.randn(1, 4, 3, 6, 6), torch.zeros(1, 2 * 3 * 9, 5, 3, 3))


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "*.npz"))),
                         ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_golden_fixtures(path):
    d = np.load(path)
    nd = d["x"].ndim - 2
    g = [int(v) for v in d["geom"]]
    cfg = (tuple(g[:nd]), tuple(g[nd:2 * nd]), tuple(g[2 * nd:3 * nd]), g[3 * nd], g[3 * nd + 1])
    x, off, w, gout = (torch.from_numpy(d[k]) for k in ("x", "off", "w", "gout"))
    b = torch.from_numpy(d["b"]) if "b" in d else None
    out = orc.forward(x, off, w, b, *cfg)
    gin, goff, gw, gb = orc.backward(x, off, w, gout, b, *cfg)
    for got, key in ((out, "out"), (gin, "gin"), (goff, "goff"), (gw, "gw")):
        assert np.abs(got.numpy() - d[key]).max() < 1e-12, key
    if b is not None:
        assert np.abs(gb.numpy() - d["gb"]).max() < 1e-12


def test_reference_function_script_values():
    # deform3d/test_function.py:6-25, worked by hand: with pad 1 and dilation 2 the taps of each
    # axis sit at o-1, o+1, o+3.  The rows of the input are [1,2,1] along h and constant along l, w.
    d = np.load(os.path.join(ROOT, "tests", "golden", "3d_ref_function_script.npz"))
    out = d["out"][0, 0]
    # position (0,0,0): only tap index 1 (coordinate 1) is inside on each axis -> x[1,1,1] = 2
    assert out[0, 0, 0] == 2.0
    # position (1,1,1): taps at 0 and 2 on each axis: 8 samples, rows h=0 and h=2 hold 1 -> 8
    assert out[1, 1, 1] == 8.0
    # position (1,0,1): l in {0,2}, h = 1, w in {0,2}: 4 samples of value 2 -> 8
    assert out[1, 0, 1] == 8.0
    assert d["gw"].shape == (1, 1, 3, 3, 3)
    # grad_offset by hand.  Weight and grad_output are all ones, so every grad-column value is 1.
    # A tap at integer coordinate p on an axis: p in {0, 1, 2} is inside; the high corner differs
    # from the low one only for p = 1 (for p <= 0 and p >= size - 1 it collapses).  The input varies
    # along h only ([1, 2, 1]), so an inside sample has d/dl = d/dw = 0 and d/dh = x[2] - x[1] = -1
    # when p_h = 1, else 0.  A sample with any axis outside gets, per axis, -|1| for p <= -1, +|1|
    # for p >= 3 (the length extent, deform3d/lib/deform_conv3d_cuda_kernel.cu:470-481), else 0.
    goff = d["goff"].reshape(27, 3, 3, 3, 3)                    # [tap][axis][ol][oh][ow]
    want = np.zeros_like(goff)
    for kl in range(3):
        for kh in range(3):
            for kw in range(3):
                tap = (kl * 3 + kh) * 3 + kw
                for ol in range(3):
                    for oh in range(3):
                        for ow in range(3):
                            p = (ol - 1 + 2 * kl, oh - 1 + 2 * kh, ow - 1 + 2 * kw)
                            if all(0 <= v <= 2 for v in p):
                                want[tap, 1, ol, oh, ow] = -1.0 if p[1] == 1 else 0.0
                            else:
                                for a in range(3):
                                    want[tap, a, ol, oh, ow] = -1.0 if p[a] <= -1 else (1.0 if p[a] >= 3 else 0.0)
    assert np.array_equal(goff, want)
    assert (want != 0).sum() > 100          # taps at -1 and at 3 (and beyond) do occur


def test_pack_modules_construction():
    """The modules that own the offset convolution: parameter names, offset channels, offset size."""
    import deform_conv3d_pytorch_op_amd as dcn
    m = dcn.ConvOffset3dPack(8, 6, (3, 3, 1), stride=(1, 2, 1), padding=(1, 1, 0), dilation=2, channel_per_group=4, groups=2)
    assert sorted(m.state_dict()) == ["bias", "conv_offset.weight", "weight"]
    assert tuple(m.conv_offset.weight.shape) == (8 // 4 * 3 * 9, 8, 3, 3, 1)
    x = torch.randn(2, 8, 5, 8, 4)
    # the offset convolution (dilation 1) has the layer's dilation-blind output size
    assert tuple(m.conv_offset(x).shape[2:]) == dcn.output_size((5, 8, 4), (3, 3, 1), (1, 2, 1), (1, 1, 0))
    m2 = dcn.ConvOffset2dPack(4, 4, 3, padding=1, channel_per_group=2, bias=False, zero_init_offset=True)
    assert sorted(m2.state_dict()) == ["conv_offset.weight", "weight"]
    assert float(m2.conv_offset.weight.abs().max()) == 0.0
    with pytest.raises(ValueError):
        dcn.ConvOffset2dPack(6, 4, 3, channel_per_group=4)
    with pytest.raises(RuntimeError):          # no CPU path: the layer itself needs the GPU
        m2(torch.randn(1, 4, 5, 5))


def test_standard_output_size_formula():
    from deform_conv3d_pytorch_op_amd import output_size
    # reference formula: dilation ignored
    assert output_size((8, 8, 8), (3, 3, 3), (1, 1, 1), (3, 3, 3)) == (12, 12, 12)
    # dilation-aware: torch's convolution size
    assert output_size((8, 8, 8), (3, 3, 3), (1, 1, 1), (3, 3, 3), (3, 3, 3), standard=True) == (8, 8, 8)
    for i, k, s, p, d in [(10, 3, 2, 1, 2), (7, 1, 3, 0, 4), (9, 2, 1, 0, 3), (16, 5, 2, 4, 2)]:
        want = torch.nn.functional.conv1d(torch.zeros(1, 1, i), torch.zeros(1, 1, k), stride=s, padding=p, dilation=d).shape[-1]
        assert output_size((i,), (k,), (s,), (p,), (d,), standard=True) == (want,)
        # never larger than the reference's size, equal for dilation 1
        assert want <= output_size((i,), (k,), (s,), (p,))[0]
        assert output_size((i,), (k,), (s,), (p,), (1,), standard=True) == output_size((i,), (k,), (s,), (p,))


def test_pack_module_offset_convolution_follows_output_size_mode():
    from deform_conv3d_pytorch_op_amd import ConvOffset2dPack
    blind = ConvOffset2dPack(4, 4, 3, padding=2, dilation=2)
    std = ConvOffset2dPack(4, 4, 3, padding=2, dilation=2, standard_output_size=True)
    assert blind.conv_offset.dilation == (1, 1) and std.conv_offset.dilation == (2, 2)
    x = torch.zeros(1, 4, 9, 9)
    assert blind.conv_offset(x).shape[2:] == (11, 11) and std.conv_offset(x).shape[2:] == (9, 9)


def test_oob_offset_grad_argument_is_validated():
    from deform_conv3d_pytorch_op_amd import ConvOffset3d, ConvOffset3dPack
    assert ConvOffset3d(2, 2, 3, oob_offset_grad="zero").oob_offset_grad == "zero"
    assert ConvOffset3dPack(2, 2, 3).oob_offset_grad == "reference"
    with pytest.raises(ValueError):
        ConvOffset3d(2, 2, 3, oob_offset_grad="clean")
