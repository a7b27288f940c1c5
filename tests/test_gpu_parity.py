"""GPU parity tests: the HIP path (through the C ABI, via ctypes) against the CPU oracle on the
same seeded inputs, against the committed golden fixtures, and -- at BASELINE.json's sizes --
through size-independent identities.  Tolerances are the ones north_star states: float64 1e-10
relative; float32 1e-4 relative forward and 1e-3 on gradients.  "Relative" is the largest
absolute deviation over the largest absolute reference value of that tensor.
"""
import glob
import math
import os

import numpy as np
import pytest
import torch

from oracle import dcn_oracle as orc
from tests.cases import SMALL_CASES, make_case, random_spec

pytestmark = pytest.mark.gpu

TOL = {torch.float64: dict(fwd=1e-10, grad=1e-10), torch.float32: dict(fwd=1e-4, grad=1e-3)}


def _dcn():
    import deform_conv3d_pytorch_op_amd as dcn
    return dcn


def rel_err(got, want):
    want = want.double()
    scale = want.abs().max().item()
    return (got.detach().cpu().double() - want).abs().max().item() / (scale if scale > 0 else 1.0)


def run_gpu(c, need_bias=True):
    dcn = _dcn()
    fn = dcn.ConvOffset3dFunction if c["nd"] == 3 else dcn.ConvOffset2dFunction
    dev = torch.device("cuda:0")
    x, off, w = (c[k].to(dev).requires_grad_(True) for k in ("x", "off", "w"))
    b = c["b"].to(dev).requires_grad_(True) if c["b"] is not None else None
    out = fn.apply(x, off, w, b, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    out.backward(c["gout"].to(dev))
    torch.cuda.synchronize()
    return out, x.grad, off.grad, w.grad, (b.grad if b is not None else None)


def run_oracle(c):
    out = orc.forward(c["x"], c["off"], c["w"], c["b"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    gin, goff, gw, gb = orc.backward(c["x"], c["off"], c["w"], c["gout"], c["b"], c["stride"], c["pad"], c["dil"],
                                     c["cpg"], c["groups"])
    return out, gin, goff, gw, gb


def compare(c, dtype, tag):
    got = run_gpu(c)
    want = run_oracle(c)
    names = ("output", "grad_input", "grad_offset", "grad_weight", "grad_bias")
    for name, g, w in zip(names, got, want):
        if w is None:
            continue
        tol = TOL[dtype]["fwd" if name == "output" else "grad"]
        e = rel_err(g, w)
        assert e <= tol, "%s %s: relative error %.3e > %.1e" % (tag, name, e, tol)


@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["f64", "f32"])
@pytest.mark.parametrize("name", sorted(SMALL_CASES))
def test_small_cases_match_oracle(name, dtype):
    print("case", name, dtype, flush=True)
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=3)
    compare(c, dtype, name)


@pytest.mark.parametrize("seed", range(96))
def test_random_geometries_match_oracle(seed):
    """Seeded random small geometries (2-D / 3-D, odd channel counts, all divisors as deformable-group
    widths, rectangular kernels, per-axis stride / padding / dilation), float64 and float32."""
    spec = random_spec(seed)
    print("random geometry", seed, spec, flush=True)
    for dtype in (torch.float64, torch.float32):
        compare(make_case(*spec, dtype=dtype, seed=100 + seed), dtype, "random_%d" % seed)


@pytest.mark.parametrize("seed", range(48))
def test_random_medium_geometries_match_oracle(seed):
    """The same with extents of several position tiles per axis (halo tiling, channel splits, partial
    tiles at the rim) and up to 72 input channels."""
    spec = random_spec(seed, medium=True)
    print("random medium geometry", seed, spec, flush=True)
    for dtype in (torch.float64, torch.float32):
        compare(make_case(*spec, dtype=dtype, seed=200 + seed), dtype, "random_medium_%d" % seed)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))),
                         ids=lambda p: os.path.basename(p)[:-4])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["f64", "f32"])
def test_golden_fixtures(path, dtype):
    print("fixture", os.path.basename(path), dtype, flush=True)
    d = np.load(path)
    nd = d["x"].ndim - 2
    g = [int(v) for v in d["geom"]]
    c = dict(nd=nd, stride=tuple(g[:nd]), pad=tuple(g[nd:2 * nd]), dil=tuple(g[2 * nd:3 * nd]), cpg=g[3 * nd],
             groups=g[3 * nd + 1])
    for k in ("x", "off", "w", "gout"):
        c[k] = torch.from_numpy(d[k]).to(dtype)
    c["b"] = torch.from_numpy(d["b"]).to(dtype) if "b" in d else None
    got = run_gpu(c)
    want = [d["out"], d["gin"], d["goff"], d["gw"], d["gb"] if "b" in d else None]
    # float32: the fixture was computed in float64 from float64 inputs, so only inputs that are
    # exactly representable in float32 keep every inside/outside decision; all fixtures with
    # random data are therefore checked in float64 only.
    exact = all(np.array_equal(d[k], d[k].astype(np.float32).astype(np.float64)) for k in ("x", "off", "w", "gout"))
    if dtype == torch.float32 and not exact:
        pytest.skip("fixture data is not float32-representable")
    for name, gt, wt in zip(("output", "grad_input", "grad_offset", "grad_weight", "grad_bias"), got, want):
        if wt is None:
            continue
        tol = TOL[dtype]["fwd" if name == "output" else "grad"]
        assert rel_err(gt, torch.from_numpy(wt)) <= tol, name


def test_gradcheck_2d_float64():
    # BASELINE configs[0] geometry (deform2d float64, k3 p1, one deformable group) at reduced
    # extent; offsets kept 0.05 away from integer coordinates, where the sampler has kinks.
    print("gradcheck 2d", flush=True)
    dcn = _dcn()
    g = torch.Generator().manual_seed(7)
    dev = "cuda:0"
    x = torch.randn(2, 4, 6, 6, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    off = torch.rand(2, 18, 6, 6, generator=g, dtype=torch.float64) * 3 - 1.5
    off = torch.where((off - off.round()).abs() < 0.05, off + 0.1, off).to(dev).requires_grad_(True)
    w = torch.randn(4, 4, 3, 3, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    b = torch.randn(4, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    assert torch.autograd.gradcheck(dcn.ConvOffset2dFunction.apply, (x, off, w, b, (1, 1), (1, 1), (1, 1), 4, 1),
                                    eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=1e-9)


def test_gradcheck_2d_float64_c1_shape():
    # BASELINE configs[0] at its full shape: N=2, C 8 -> 8, 16x16, k3 p1, one deformable group,
    # offsets U[-1.5, 1.5] (kept 0.05 away from integer coordinates, where the sampler has kinks).
    # Full Jacobians (fast_mode off): 13.9k perturbed inputs against 4096 outputs.
    print("gradcheck 2d c1 shape", flush=True)
    dcn = _dcn()
    g = torch.Generator().manual_seed(17)
    dev = "cuda:0"
    x = torch.randn(2, 8, 16, 16, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    off = torch.rand(2, 18, 16, 16, generator=g, dtype=torch.float64) * 3 - 1.5
    off = torch.where((off - off.round()).abs() < 0.05, off + 0.1, off).to(dev).requires_grad_(True)
    w = (torch.randn(8, 8, 3, 3, generator=g, dtype=torch.float64) * math.sqrt(2.0 / 72)).to(dev).requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c: dcn.ConvOffset2dFunction.apply(a, b, c, None, (1, 1), (1, 1), (1, 1), 8, 1),
                                    (x, off, w), eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=1e-9, fast_mode=False)


def test_gradcheck_2d_reference_script_shape():
    # deform2d_double/test_gradient.py:7-53
    print("gradcheck 2d ref", flush=True)
    dcn = _dcn()
    g = torch.Generator().manual_seed(5)
    dev = "cuda:0"
    x = torch.rand(2, 2, 7, 7, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    off = torch.rand(2, 2, 6, 6, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    w = torch.rand(4, 1, 1, 1, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    b = torch.rand(4, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    assert torch.autograd.gradcheck(dcn.ConvOffset2dFunction.apply, (x, off, w, b, (2, 2), (2, 2), (2, 2), 2, 2),
                                    eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=1e-9)


def test_gradcheck_3d_float64_in_range():
    # the 3-D out-of-range grad-offset branches are not a derivative, so gradcheck is run where
    # every sample stays inside the volume
    print("gradcheck 3d", flush=True)
    dcn = _dcn()
    g = torch.Generator().manual_seed(9)
    dev = "cuda:0"
    x = torch.randn(1, 2, 5, 5, 5, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    off = (torch.rand(1, 48, 4, 4, 4, generator=g, dtype=torch.float64) * 0.8 + 0.1).to(dev).requires_grad_(True)
    w = torch.randn(2, 1, 2, 2, 2, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    b = torch.randn(2, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    assert torch.autograd.gradcheck(dcn.ConvOffset3dFunction.apply,
                                    (x, off, w, b, (1, 1, 1), (0, 0, 0), (1, 1, 1), 1, 2),
                                    eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=1e-9)


def _inside_mask(c):
    """[N, DG, kV, outV] bool: the sample of (deformable group, tap, position) lies inside the input
    (-1 < coordinate < size on every axis), worked out here from the offsets in float64."""
    nd = c["nd"]
    N = c["x"].shape[0]
    kV, outV = math.prod(c["k"]), math.prod(c["outs"])
    off = c["off"].double().reshape(N, -1, kV, nd, outV)
    grids = torch.meshgrid(*[torch.arange(o, dtype=torch.float64) for o in c["outs"]], indexing="ij")
    taps = torch.meshgrid(*[torch.arange(k, dtype=torch.float64) for k in c["k"]], indexing="ij")
    ok = torch.ones(off.shape[0], off.shape[1], kV, outV, dtype=torch.bool)
    for a in range(nd):
        base = grids[a].reshape(1, 1, 1, outV) * c["stride"][a] - c["pad"][a]
        tap = taps[a].reshape(1, 1, kV, 1) * c["dil"][a]
        p = base + tap + off[:, :, :, a, :]
        ok &= (p > -1) & (p < c["ins"][a])
    return ok


@pytest.mark.parametrize("name", ["3d_basic", "3d_dilation3", "3d_c5_like"])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["f64", "f32"])
def test_oob_offset_grad_zero_drops_only_the_out_of_range_term(name, dtype):
    """oob_offset_grad='zero': grad_offset of a sample outside the input is exactly zero, that of a
    sample inside is what the reference mode gives (which the oracle pins), and nothing else moves."""
    dcn = _dcn()
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=21)
    inside = _inside_mask(c)
    assert 0 < int((~inside).sum()) < inside.numel()          # the case has samples of both kinds
    dev = torch.device("cuda:0")
    res = {}
    for mode in ("reference", "zero"):
        x, off, w = (c[k].to(dev).requires_grad_(True) for k in ("x", "off", "w"))
        out = dcn.ConvOffset3dFunction.apply(x, off, w, None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"],
                                             False, mode)
        out.backward(c["gout"].to(dev))
        torch.cuda.synchronize()
        res[mode] = (out.detach().cpu(), x.grad.cpu(), off.grad.cpu(), w.grad.cpu())
    tol = TOL[dtype]["grad"]
    assert torch.equal(res["zero"][0], res["reference"][0])
    assert rel_err(res["zero"][1], res["reference"][1]) <= tol
    assert rel_err(res["zero"][3], res["reference"][3]) <= tol
    N, kV, nd, outV = c["x"].shape[0], math.prod(c["k"]), c["nd"], math.prod(c["outs"])
    go_ref = res["reference"][2].reshape(N, -1, kV, nd, outV)
    go_zero = res["zero"][2].reshape(N, -1, kV, nd, outV)
    m = inside.unsqueeze(3).expand_as(go_ref)
    assert torch.count_nonzero(go_zero[~m]) == 0
    assert go_ref[~m].abs().max() > 0                           # the reference mode does put something there
    scale = go_ref.abs().max().item()
    assert (go_zero[m].double() - go_ref[m].double()).abs().max().item() <= tol * scale


def test_gradcheck_3d_float64_oob_zero():
    # with the out-of-range term left out grad_offset is a derivative everywhere, so gradcheck also
    # passes with samples outside the volume (offsets up to 3 voxels on a 5^3 input, padding 1)
    print("gradcheck 3d oob zero", flush=True)
    dcn = _dcn()
    g = torch.Generator().manual_seed(10)
    dev = "cuda:0"
    x = torch.randn(1, 2, 5, 5, 5, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    off = ((torch.rand(1, 48, 6, 6, 6, generator=g, dtype=torch.float64) * 2 - 1) * 3).to(dev).requires_grad_(True)
    w = torch.randn(2, 1, 2, 2, 2, generator=g, dtype=torch.float64).to(dev).requires_grad_(True)
    fn = lambda x_, o_, w_: dcn.ConvOffset3dFunction.apply(x_, o_, w_, None, (1, 1, 1), (1, 1, 1), (1, 1, 1), 1, 2,
                                                           False, "zero")
    assert torch.autograd.gradcheck(fn, (x, off, w), eps=1e-6, atol=1e-5, rtol=1e-3, nondet_tol=1e-9)


def test_modules_forward_backward():
    print("modules", flush=True)
    dcn = _dcn()
    dev = "cuda:0"
    torch.manual_seed(0)
    m3 = dcn.ConvOffset3d(4, 6, 3, stride=1, padding=1, dilation=1, channel_per_group=2, bias=True, groups=2).to(dev)
    x = torch.randn(2, 4, 4, 5, 6, device=dev, requires_grad=True)
    off = torch.randn(2, 2 * 3 * 27, 4, 5, 6, device=dev, requires_grad=True)
    y = m3(x, off)
    y.sum().backward()
    want = orc.forward(x.detach().cpu(), off.detach().cpu(), m3.weight.detach().cpu(), m3.bias.detach().cpu(),
                       1, 1, 1, 2, 2)
    assert rel_err(y, want) < 1e-4
    assert m3.weight.grad is not None and m3.bias.grad is not None and x.grad is not None and off.grad is not None
    m2 = dcn.ConvOffset2d(4, 4, 3, padding=1, channel_per_group=4, bias=False).to(dev).double()
    x2 = torch.randn(1, 4, 6, 6, device=dev, dtype=torch.float64)
    y2 = m2(x2, torch.zeros(1, 18, 6, 6, device=dev, dtype=torch.float64))
    want2 = torch.nn.functional.conv2d(x2, m2.weight, None, 1, 1)
    assert rel_err(y2, want2.cpu()) < 1e-12
    assert sorted(m3.state_dict()) == ["bias", "weight"]


@pytest.mark.parametrize("name", ["3d_basic", "2d_basic", "3d_c5_like"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
def test_non_finite_and_huge_offsets(name, dtype):
    """Offsets that are NaN, infinite or far beyond the integer range select no voxel (every window
    test of the sampler is false for them): those samples add nothing, on the GPU as in the oracle."""
    print("special offsets", name, dtype, flush=True)
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=5)
    flat = c["off"].view(-1)
    idx = torch.randperm(flat.numel(), generator=torch.Generator().manual_seed(1))[:64]
    vals = torch.tensor([float("nan"), float("inf"), -float("inf"), 1e30, -1e30, 3e9, -3e9, 1e5], dtype=dtype)
    flat[idx] = vals[torch.arange(64) % 8]
    got = run_gpu(c)
    want = run_oracle(c)
    for nm, g, w in zip(("output", "grad_input", "grad_offset", "grad_weight", "grad_bias"), got, want):
        assert torch.isfinite(g).all(), nm
        assert rel_err(g, w) < TOL[dtype]["fwd" if nm == "output" else "grad"], nm


@pytest.mark.parametrize("where", ["grad_output", "weight"])
@pytest.mark.parametrize("name", ["3d_basic", "2d_basic", "3d_c4_like"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
def test_non_finite_grad_output_and_weight_propagate(name, dtype, where):
    """NaN / infinite entries of grad_output or of the weight reach the gradients as in the
    reference's float atomics: where the oracle's gradient is not finite the GPU's is not finite
    either, and where it is finite the values agree."""
    print("non-finite", name, dtype, where, flush=True)
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=6)
    t = c["gout"] if where == "grad_output" else c["w"]
    flat = t.view(-1)
    idx = torch.randperm(flat.numel(), generator=torch.Generator().manual_seed(2))[:3]
    flat[idx] = torch.tensor([float("nan"), float("inf"), -float("inf")], dtype=dtype)
    got = run_gpu(c)
    want = run_oracle(c)
    for nm, g, w in zip(("output", "grad_input", "grad_offset", "grad_weight", "grad_bias"), got, want):
        g = g.detach().cpu().double()
        w = w.double()
        fin = torch.isfinite(w)
        assert torch.equal(torch.isfinite(g), fin), "%s: non-finite mask differs (%d vs %d finite)" % (
            nm, int(torch.isfinite(g).sum()), int(fin.sum()))
        if fin.any():
            scale = w[fin].abs().max().item()
            tol = TOL[dtype]["fwd" if nm == "output" else "grad"]
            assert (g[fin] - w[fin]).abs().max().item() <= tol * (scale if scale > 0 else 1.0), nm


@pytest.mark.parametrize("name", ["2d_c3_like", "2d_rect_kernel_stride_dil", "3d_dilation3", "3d_basic"])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32], ids=["f64", "f32"])
def test_standard_output_size_is_a_crop_of_the_reference_layer(name, dtype):
    """Output position o samples around o*stride - pad + tap*dilation whichever size formula is in
    force, and the dilation-aware size never exceeds the dilation-blind one: the layer with
    `standard_output_size` is the reference's layer cropped to the leading positions of every axis.
    So the oracle, run at the reference's size with grad_output zero outside the crop, fixes the
    output, grad_input and grad_weight, and (cropped) grad_offset."""
    dcn = _dcn()
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=11)
    nd = c["nd"]
    std = dcn.output_size(c["ins"], c["k"], c["stride"], c["pad"], c["dil"], standard=True)
    assert all(1 <= s <= o for s, o in zip(std, c["outs"]))
    crop = (slice(None), slice(None)) + tuple(slice(0, s) for s in std)
    gout_full = torch.zeros_like(c["gout"])
    gout_full[crop] = c["gout"][crop]
    co = dict(c, gout=gout_full)
    want_out, want_gin, want_goff, want_gw, want_gb = run_oracle(co)

    fn = dcn.ConvOffset3dFunction if nd == 3 else dcn.ConvOffset2dFunction
    dev = torch.device("cuda:0")
    x, w, b = (c[k].to(dev).requires_grad_(True) for k in ("x", "w", "b"))
    off = c["off"][crop].contiguous().to(dev).requires_grad_(True)
    out = fn.apply(x, off, w, b, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"], True)
    assert tuple(out.shape[2:]) == std
    out.backward(c["gout"][crop].contiguous().to(dev))
    torch.cuda.synchronize()
    tol = TOL[dtype]
    assert rel_err(out, want_out[crop]) <= tol["fwd"]
    assert rel_err(x.grad, want_gin) <= tol["grad"]
    assert rel_err(off.grad, want_goff[crop]) <= tol["grad"]
    assert rel_err(w.grad, want_gw) <= tol["grad"]
    assert rel_err(b.grad, want_gb) <= tol["grad"]


@pytest.mark.parametrize("nd", [2, 3])
def test_standard_output_size_zero_offsets_equal_dilated_convolution(nd):
    """With zero offsets and the dilation-aware size the layer is torch's dilated convolution."""
    dcn = _dcn()
    dev = torch.device("cuda:0")
    torch.manual_seed(5)
    ins = (9, 10) if nd == 2 else (7, 8, 9)
    Layer = dcn.ConvOffset2dPack if nd == 2 else dcn.ConvOffset3dPack
    layer = Layer(6, 8, 3, stride=1, padding=2, dilation=2, channel_per_group=3, groups=2, zero_init_offset=True,
                  device=dev, dtype=torch.float64, standard_output_size=True)
    x = torch.randn((2, 6) + ins, device=dev, dtype=torch.float64, requires_grad=True)
    out = layer(x)
    conv = torch.nn.functional.conv2d if nd == 2 else torch.nn.functional.conv3d
    x2 = x.detach().clone().requires_grad_(True)
    w2 = layer.weight.detach().clone().requires_grad_(True)
    want = conv(x2, w2, layer.bias.detach(), stride=1, padding=2, dilation=2, groups=2)
    assert out.shape == want.shape
    g = torch.randn_like(want)
    out.backward(g)
    want.backward(g)
    assert rel_err(out, want.detach().cpu()) <= 1e-10
    assert rel_err(x.grad, x2.grad.cpu()) <= 1e-10
    assert rel_err(layer.weight.grad, w2.grad.cpu()) <= 1e-10


class _OracleLayer(torch.autograd.Function):
    """The CPU oracle as an autograd node, so that a CPU graph (offset convolution -> layer) can be
    differentiated end to end as the reference for the Pack modules."""

    @staticmethod
    def forward(ctx, x, off, w, b, cfg):
        ctx.save_for_backward(x, off, w, b)
        ctx.cfg = cfg
        return orc.forward(x.detach(), off.detach(), w.detach(), b.detach(), *cfg)

    @staticmethod
    def backward(ctx, g):
        x, off, w, b = ctx.saved_tensors
        gin, goff, gw, gb = orc.backward(x.detach(), off.detach(), w.detach(), g.contiguous(), b.detach(), *ctx.cfg)
        return gin, goff, gw, gb, None


@pytest.mark.parametrize("nd", [2, 3])
def test_pack_module_end_to_end(nd):
    """ConvOffset{2,3}dPack (offset convolution + layer) against the same graph on the CPU: torch's
    convolution for the offsets, the oracle for the layer; float64, all four gradients."""
    print("pack module", nd, flush=True)
    dcn = _dcn()
    dev = "cuda:0"
    torch.manual_seed(3)
    if nd == 3:
        m = dcn.ConvOffset3dPack(6, 4, 3, stride=(1, 2, 1), padding=1, dilation=(1, 1, 2), channel_per_group=3, groups=2,
                                 dtype=torch.float64)
        x = torch.randn(2, 6, 4, 7, 6, dtype=torch.float64)
    else:
        m = dcn.ConvOffset2dPack(4, 6, (3, 2), stride=1, padding=(1, 0), dilation=1, channel_per_group=2, groups=2,
                                 dtype=torch.float64)
        x = torch.randn(2, 4, 7, 6, dtype=torch.float64)
    with torch.no_grad():
        m.conv_offset.weight.mul_(4.0)                 # offsets of a few voxels, some samples out of range
    ref = {k: v.detach().clone().requires_grad_(True) for k, v in m.named_parameters()}
    xr = x.clone().requires_grad_(True)
    conv = torch.nn.functional.conv3d if nd == 3 else torch.nn.functional.conv2d
    off_r = conv(xr, ref["conv_offset.weight"], None, m.stride, m.padding)
    cfg = (m.stride, m.padding, m.dilation, m.channel_per_group, m.group)
    out_r = _OracleLayer.apply(xr, off_r, ref["weight"], ref["bias"], cfg)
    gout = torch.randn_like(out_r)
    out_r.backward(gout)

    m = m.to(dev)
    xg = x.to(dev).requires_grad_(True)
    out = m(xg)
    out.backward(gout.to(dev))
    assert rel_err(out, out_r) < 1e-10
    assert rel_err(xg.grad, xr.grad) < 1e-10
    for k, v in m.named_parameters():
        assert rel_err(v.grad, ref[k].grad) < 1e-10, k


def test_forward_and_grad_weight_are_deterministic():
    """No float atomics on these two paths: repeated calls give identical bits.  (grad_input and
    grad_offset end in float atomics and may differ in the last bits from run to run.)"""
    c = make_case(*SMALL_CASES["3d_c4_like"], dtype=torch.float32, seed=4)
    first = run_gpu(c)
    for _ in range(3):
        again = run_gpu(c)
        assert torch.equal(first[0], again[0])
        assert torch.equal(first[3], again[3])
        assert rel_err(again[1], first[1].cpu()) < 1e-5 and rel_err(again[2], first[2].cpu()) < 1e-5


@pytest.mark.parametrize("nd", [2, 3])
def test_halo_plan_follows_the_offsets(nd):
    """The forward call records which of its planned LDS halo sizes the device chose, as a 32-bit
    index in the workspace at byte offset (workspace_bytes - 256) rounded down to a multiple of 256
    (include/dcn_amd.h): plan 0, margin 2, for offsets within +-1; plan 1 (margin 3, in 2-D 4) for
    offsets up to +-2.6, of which a fifth reach past +-2; plan 2 (margin 4, in 2-D 6) for offsets
    up to +-3.7 (+-5.9).  The output agrees with the oracle whichever plan runs."""
    if os.environ.get("DCN_HALO_MARGIN") or os.environ.get("DCN_ADAPTIVE_MARGIN") == "0":
        pytest.skip("one fixed halo margin is forced: nothing is chosen")
    from deform_conv3d_pytorch_op_amd import _lib
    from deform_conv3d_pytorch_op_amd.functions import _geom
    L = _lib.load()
    dev = torch.device("cuda:0")
    spec = (3, 2, 16, 16, (8, 16, 24), 3, 1, 1, 1, 8, 1) if nd == 3 else (2, 2, 32, 16, (40, 48), 3, 1, 1, 1, 16, 1)
    chosen = {}
    for label, scale in (("narrow", 1.0), ("wide", 2.6), ("widest", 3.7 if nd == 3 else 5.9)):
        print("halo plan", nd, label, flush=True)
        c = make_case(*spec, scale, dtype=torch.float32, seed=21, bias=False)
        x, off, w = (c[k].to(dev) for k in ("x", "off", "w"))
        geom = _geom(nd, x, w, c["outs"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
        nbytes = L.dcn_workspace_bytes_for(4, x.shape[0], x.shape[1], w.shape[0], math.prod(c["ins"]), math.prod(c["outs"]),
                                           math.prod(c["k"]), c["groups"], c["cpg"])
        ws = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=dev)
        out = torch.empty((x.shape[0], w.shape[0]) + c["outs"], dtype=torch.float32, device=dev)
        rc = getattr(L, "dcn%dd_forward_f32" % nd)(x.data_ptr(), w.data_ptr(), off.data_ptr(), None, out.data_ptr(), *geom,
                                                   ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, L.dcn_last_error()
        torch.cuda.synchronize()
        at = (nbytes - 256) // 256 * 256
        chosen[label] = int.from_bytes(bytes(ws[at:at + 4].cpu().tolist()), "little")
        want = orc.forward(c["x"], c["off"], c["w"], None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
        assert rel_err(out, want) < TOL[torch.float32]["fwd"], label
    assert chosen == {"narrow": 0, "wide": 1, "widest": 2}, chosen


def test_hip_graph_replay():
    """Forward + backward captured into a HIP graph (the C ABI allocates nothing, clears memory with
    kernels only and never synchronises); every replay, with eager work and synchronisations in
    between, must reproduce the eager result on fresh inputs."""
    print("hip graph", flush=True)
    dcn = _dcn()
    dev = torch.device("cuda:0")
    c = make_case(*SMALL_CASES["3d_c4_like"], dtype=torch.float32, seed=11)
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    sx, soff, sw = (c[k].to(dev).clone().requires_grad_(True) for k in ("x", "off", "w"))
    sg = c["gout"].to(dev).clone()

    def run():
        out = dcn.ConvOffset3dFunction.apply(sx, soff, sw, None, *cfg)
        gx, go, gw = torch.autograd.grad(out, (sx, soff, sw), sg)
        return out, gx, go, gw

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                          # warm-up outside capture (lazy initialisation, allocator)
            run()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for rep in range(3):
        c2 = make_case(*SMALL_CASES["3d_c4_like"], dtype=torch.float32, seed=20 + rep)
        with torch.no_grad():
            sx.copy_(c2["x"]); soff.copy_(c2["off"]); sw.copy_(c2["w"]); sg.copy_(c2["gout"])
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in captured]
        want = run()                                 # eager work between the replays
        torch.cuda.synchronize()
        for name, g, w_ in zip(("output", "grad_input", "grad_offset", "grad_weight"), got, want):
            assert rel_err(g, w_.cpu()) < 1e-5, (rep, name)      # float atomics: order differs run to run


def test_needs_input_grad_gating():
    dcn = _dcn()
    dev = "cuda:0"
    c = make_case(*SMALL_CASES["2d_basic"], dtype=torch.float64, seed=1)
    x, off, w = c["x"].to(dev), c["off"].to(dev), c["w"].to(dev).requires_grad_(True)
    out = dcn.ConvOffset2dFunction.apply(x, off, w, None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    out.backward(c["gout"].to(dev))
    assert w.grad is not None
    x2 = c["x"].to(dev).requires_grad_(True)
    out = dcn.ConvOffset2dFunction.apply(x2, off, w.detach(), None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    out.backward(c["gout"].to(dev))
    assert x2.grad is not None


# ---------------------------------------------------------------------------------------------
# BASELINE.json sizes: the whole batch at full size against the oracle (all four tensors), and the
# bilinear-form identities <out, g> = <x, grad_input> = <W, grad_weight> (fixed offsets, no bias).

FULL = {
    "c2_2d_f32": (2, 8, 256, 256, 56, 3, 1, 1, 1, 256, 1, 2.0),
    "c3_2d_f32_grouped_dilated": (2, 4, 512, 512, 28, 3, 1, 2, 2, 128, 2, None),
    "c4_3d_f32": (3, 4, 64, 64, (16, 56, 56), 3, 1, 1, 1, 64, 1, 1.5),
    "c5_3d_f32_strided": (3, 2, 128, 128, (16, 112, 112), 3, (1, 2, 2), 1, 1, 32, 1, 2.0),
}


def full_case(name, seed=0):
    args = FULL[name]
    kw = dict(dtype=torch.float32, seed=seed, bias=False)
    if args[-1] is None:
        return make_case(*args[:-1], 1.0, off_dist="normal_mix", **kw)
    return make_case(*args, **kw)


@pytest.mark.parametrize("name", sorted(FULL))
def test_full_size_parity_and_identities(name):
    print("full-size", name, flush=True)
    c = full_case(name)
    out, gin, goff, gw, _ = run_gpu(c)
    # identities, accumulated in float64 on the host
    o64, g64 = out.detach().cpu().double(), c["gout"].double()
    lhs = (o64 * g64).sum().item()
    via_x = (c["x"].double() * gin.cpu().double()).sum().item()
    via_w = (c["w"].double() * gw.cpu().double()).sum().item()
    scale = (o64.abs() * g64.abs()).sum().item()
    assert abs(lhs - via_x) / scale < 1e-5, (lhs, via_x, scale)
    assert abs(lhs - via_w) / scale < 1e-5, (lhs, via_w, scale)
    # the oracle on the same tensors, whole batch, full extent
    print("full-size oracle", name, flush=True)
    want = run_oracle(c)
    for nm, g, w in zip(("output", "grad_input", "grad_offset", "grad_weight"), (out, gin, goff, gw), want):
        tol = TOL[torch.float32]["fwd" if nm == "output" else "grad"]
        e = rel_err(g, w)
        print("  %s %s rel err %.2e" % (name, nm, e), flush=True)
        assert e <= tol, "%s %s: relative error %.3e" % (name, nm, e)


def test_linearity_in_weight_and_input_full_c4():
    # out(x, a*W1 + W2) = a*out(x, W1) + out(x, W2) at the headline size
    print("linearity c4", flush=True)
    dcn = _dcn()
    dev = "cuda:0"
    c = full_case("c4_3d_f32", seed=2)
    x, off, w1 = c["x"].to(dev), c["off"].to(dev), c["w"].to(dev)
    w2 = torch.randn_like(w1) * w1.std()
    f = lambda xx, ww: dcn.ConvOffset3dFunction.apply(xx, off, ww, None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    a = 0.5
    lhs = f(x, a * w1 + w2)
    rhs = a * f(x, w1) + f(x, w2)
    assert ((lhs - rhs).abs().max() / rhs.abs().max()).item() < 1e-4


def test_error_paths_on_gpu_tensors():
    dcn = _dcn()
    dev = "cuda:0"
    x = torch.randn(1, 4, 6, 6, device=dev)
    w = torch.randn(4, 4, 3, 3, device=dev)
    with pytest.raises(RuntimeError, match="off channel"):
        dcn.ConvOffset2dFunction.apply(x, torch.zeros(1, 17, 6, 6, device=dev), w, None, (1, 1), (1, 1), (1, 1), 4, 1)
    with pytest.raises(RuntimeError, match="off h"):
        dcn.ConvOffset2dFunction.apply(x, torch.zeros(1, 18, 5, 6, device=dev), w, None, (1, 1), (1, 1), (1, 1), 4, 1)
    with pytest.raises(RuntimeError, match="input c != kernel c"):
        dcn.ConvOffset2dFunction.apply(x, torch.zeros(1, 18, 6, 6, device=dev), w, None, (1, 1), (1, 1), (1, 1), 4, 2)


def test_every_sample_of_a_block_lands_in_one_cell():
    """The worst case for the paired fixed-point LDS cells of the float32 fused backward kernel: the
    offsets send all 27 taps of all 256 positions of a position block to the same voxel (integer
    coordinates, so one corner carries the whole weight), and grad_output is parallel to every
    weight column, which makes the Cauchy-Schwarz bound on the grad-column values an equality.
    That cell then receives (positions x taps) terms, each at the bound the scale was chosen for."""
    N, C, M, size = 1, 8, 16, (4, 8, 8)
    g = torch.Generator().manual_seed(5)
    v = torch.randn(M, generator=g, dtype=torch.float64)
    w = v.view(M, 1, 1, 1, 1).expand(M, C, 3, 3, 3).contiguous()           # every (channel, tap) column is v
    gout = v.view(1, M, 1, 1, 1).expand(N, M, *size).contiguous()           # every position's grad_output is v
    x = torch.randn((N, C) + size, generator=g, dtype=torch.float64)
    target = (1.0, 2.0, 3.0)
    off = torch.zeros(N, 27, 3, *size, dtype=torch.float64)                 # one deformable group
    for tap in range(27):
        k = (tap // 9, (tap // 3) % 3, tap % 3)
        for a in range(3):
            pos = torch.arange(size[a], dtype=torch.float64).view([-1 if b == a else 1 for b in range(3)])
            off[:, tap, a] = target[a] - (pos - 1 + k[a])                   # stride 1, pad 1, dilation 1
    off = off.view(N, 81, *size)
    c = dict(x=x.float(), off=off.float(), w=w.float(), b=None, gout=gout.float(), stride=(1, 1, 1), pad=(1, 1, 1),
             dil=(1, 1, 1), cpg=C, groups=1, ins=size, k=(3, 3, 3), outs=size, nd=3)
    got, want = run_gpu(c), run_oracle(c)
    hit = want[1][0, :, 1, 2, 3]
    assert float(hit.abs().min()) > 0.9 * 256 * 27 * float(v.dot(v))        # all terms arrived in that voxel
    for name, a, b in zip(("output", "grad_input", "grad_offset", "grad_weight"), got, want):
        tol = 1e-4 if name == "output" else 1e-3
        e = rel_err(a, b)
        assert e <= tol, "%s: relative error %.3e" % (name, e)


@pytest.mark.parametrize("name", ["3d_basic", "2d_basic", "3d_c4_like", "2d_chunk16_small_m"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
def test_non_finite_input_next_to_rim_samples(name, dtype):
    """NaN / infinite INPUT voxels beside the rim.  For a coordinate in a collapse zone (p <= 0 or
    p >= size - 1 on an axis) the reference puts the high corner on the low one and never reads the
    neighbouring voxel (deform3d/lib/deform_conv3d_cuda_kernel.cu:24-26), so a non-finite neighbour
    leaves the sample finite; inside the volume a corner of weight 0 still turns the sample into NaN
    (0 * inf), in the reference as here.  The non-finite masks of every result must equal the
    oracle's, and the finite entries must agree to the usual tolerances."""
    print("non-finite input", name, dtype, flush=True)
    c = make_case(*SMALL_CASES[name], dtype=dtype, seed=8)
    nd = c["nd"]
    x = c["x"]
    # second and second-to-last voxel of every axis in a few channels: the cells a collapsed corner would have read
    bad = [float("inf"), -float("inf"), float("nan")]
    k = 0
    for a in range(nd):
        for pos in (1, x.shape[2 + a] - 2):
            idx = [slice(None)] * x.dim()
            idx[1] = k % x.shape[1]
            idx[2 + a] = pos
            x[tuple(idx)] = bad[k % 3]
            k += 1
    # offsets pushed towards the rim so that many samples fall into the collapse zones on some axis
    c["off"] = c["off"] * 1.5
    got = run_gpu(c)
    want = run_oracle(c)
    n_bad = 0
    for nm, g, w in zip(("output", "grad_input", "grad_offset", "grad_weight", "grad_bias"), got, want):
        g = g.detach().cpu().double()
        w = w.double()
        fin = torch.isfinite(w)
        n_bad += int((~fin).sum())
        assert torch.equal(torch.isfinite(g), fin), "%s: non-finite mask differs (%d vs %d finite of %d)" % (
            nm, int(torch.isfinite(g).sum()), int(fin.sum()), fin.numel())
        if fin.any():
            scale = w[fin].abs().max().item()
            tol = TOL[dtype]["fwd" if nm == "output" else "grad"]
            assert (g[fin] - w[fin]).abs().max().item() <= tol * (scale if scale > 0 else 1.0), nm
    assert n_bad > 0                      # the case does produce non-finite results somewhere


HEAVY_EPS = {"paired": 2e-5, "single": 2e-6}


@pytest.mark.parametrize("name", ["3d_chunk8_two_blocks", "3d_c4_like", "2d_chunk16_small_m", "3d_m100_chunk4"])
def test_heavy_tailed_grad_output_keeps_small_gradients(name):
    """grad_output whose per-position magnitude spans four decades inside every position block (real
    training gradients are heavy-tailed).  The float32 grad_input of the fused backward kernel is summed
    in LDS as fixed point with one scale per workgroup, so its error is absolute in that scale: every
    element must satisfy |got - ref| <= 1e-3 |ref| + eps * max|ref| with eps = 2e-5 for the paired
    32-bit cells (2e-6 with DCN_FUSED_PAIR=0, the 64-bit cells), where the per-tensor tolerance of the
    other tests would allow 1e-3 * max|ref| everywhere."""
    print("heavy-tailed grad_output", name, flush=True)
    c = make_case(*SMALL_CASES[name], dtype=torch.float32, seed=9)
    g = torch.Generator().manual_seed(10)
    pos_shape = (c["gout"].shape[0], 1) + tuple(c["gout"].shape[2:])
    decades = torch.rand(pos_shape, generator=g) * 4.0                 # 1 .. 1e4, independent per position
    c["gout"] = (c["gout"] * torch.pow(10.0, decades)).float().contiguous()
    got = run_gpu(c)
    want = run_oracle(c)
    eps = HEAVY_EPS["single" if os.environ.get("DCN_FUSED_PAIR") == "0" else "paired"]
    gin, ref = got[1].detach().cpu().double(), want[1].double()
    top = ref.abs().max().item()
    excess = ((gin - ref).abs() - 1e-3 * ref.abs()).max().item() / top
    print("  grad_input: largest |err| - 1e-3|ref| = %.3e of max|ref|" % excess, flush=True)
    assert excess <= eps, "grad_input: %.3e of max|ref| beyond 1e-3 |ref|" % excess
    for nm, gt, wt in zip(("output", "grad_input", "grad_offset", "grad_weight"), got, want):
        assert rel_err(gt, wt) <= TOL[torch.float32]["fwd" if nm == "output" else "grad"], nm


def test_backward_plan_follows_the_offsets_up_to_the_path_without_lds():
    """backward_input_offset records the plan the device chose 64 bytes into the last whole 256-byte
    block of its workspace (include/dcn_amd.h): 0 for offsets within +-1, a wider halo for +-2.6, and 3
    -- the path without LDS tiling, coalesced atomics on a channels-last copy -- when the offsets
    (+-9) throw most samples beyond the widest halo.  The gradients agree with the oracle whichever
    path runs, and grad_input is accumulated into by all of them."""
    if os.environ.get("DCN_HALO_MARGIN") or os.environ.get("DCN_ADAPTIVE_MARGIN") == "0" or \
            os.environ.get("DCN_GLOBAL_PLAN") == "0" or os.environ.get("DCN_SCATTER") or os.environ.get("DCN_COORD"):
        pytest.skip("the choice is switched off by a knob")
    from deform_conv3d_pytorch_op_amd import _lib
    from deform_conv3d_pytorch_op_amd.functions import _geom
    L = _lib.load()
    dev = torch.device("cuda:0")
    spec = (3, 2, 16, 16, (8, 16, 24), 3, 1, 1, 1, 8, 1)
    chosen = {}
    for label, scale in (("narrow", 1.0), ("wide", 2.6), ("huge", 9.0)):
        print("backward plan", label, flush=True)
        c = make_case(*spec, scale, dtype=torch.float32, seed=22, bias=False)
        x, off, w, gout = (c[k].to(dev) for k in ("x", "off", "w", "gout"))
        geom = _geom(3, x, w, c["outs"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
        nbytes = L.dcn_workspace_bytes_for(4, x.shape[0], x.shape[1], w.shape[0], math.prod(c["ins"]), math.prod(c["outs"]),
                                           math.prod(c["k"]), c["groups"], c["cpg"])
        ws = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=dev)
        gin = torch.ones_like(x)                        # accumulated into
        goff = torch.full_like(off, 7.0)                # overwritten
        rc = L.dcn3d_backward_input_offset_f32(x.data_ptr(), w.data_ptr(), off.data_ptr(), gout.data_ptr(), gin.data_ptr(),
                                               goff.data_ptr(), *geom, ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, L.dcn_last_error()
        torch.cuda.synchronize()
        at = (nbytes - 256) // 256 * 256 + 64
        chosen[label] = int.from_bytes(bytes(ws[at:at + 4].cpu().tolist()), "little")
        want_gin, want_goff, _, _ = orc.backward(c["x"], c["off"], c["w"], c["gout"], None, c["stride"], c["pad"], c["dil"],
                                                 c["cpg"], c["groups"])
        assert rel_err(gin - 1.0, want_gin) < TOL[torch.float32]["grad"], label
        assert rel_err(goff, want_goff) < TOL[torch.float32]["grad"], label
    assert chosen["narrow"] == 0 and chosen["wide"] in (1, 2) and chosen["huge"] == 3, chosen
