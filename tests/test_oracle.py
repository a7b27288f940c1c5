"""Pins the CPU oracle (oracle/dcn_oracle.cpp) without the reference's code.

The reference holds no golden vectors, so each part of the oracle is pinned by something that
does not share its formulas: a grid_sample/einsum composite and its autograd, F.conv for zero
offsets, brute-force shifted-tap sums for integer offsets, the im2col/col2im adjoint identity,
torch.autograd.gradcheck, and hand-computed values on the reference's own script shapes.
"""
import itertools
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import dcn_oracle as orc
from tests import composite_ref as comp
from tests.cases import SMALL_CASES, make_case

torch.manual_seed(0)


def make_case(nd, N, C_in, C_out, ins, k, stride, pad, dil, cpg, groups, off_scale, dtype=torch.float64,
              seed=0, bias=True):
    g = torch.Generator().manual_seed(seed)
    t = lambda v: (v,) * nd if isinstance(v, int) else tuple(v)
    ins, k, stride, pad, dil = t(ins), t(k), t(stride), t(pad), t(dil)
    outs = comp.output_size(ins, k, stride, pad)
    kV = math.prod(k)
    x = torch.randn((N, C_in) + ins, generator=g, dtype=dtype)
    off = (torch.rand((N, C_in // cpg * nd * kV) + outs, generator=g, dtype=dtype) * 2 - 1) * off_scale
    w = torch.randn((C_out, C_in // groups) + k, generator=g, dtype=dtype) * 0.3
    b = torch.randn(C_out, generator=g, dtype=dtype) if bias else None
    gout = torch.randn((N, C_out) + outs, generator=g, dtype=dtype)
    return dict(x=x, off=off, w=w, b=b, gout=gout, stride=stride, pad=pad, dil=dil, cpg=cpg, groups=groups,
                ins=ins, k=k, outs=outs, nd=nd)


CASES = [
    # nd, N, Cin, Cout, in, k, stride, pad, dil, cpg, groups, off_scale
    (2, 2, 4, 6, (7, 9), 3, 1, 1, 1, 2, 2, 3.0),
    (2, 1, 6, 4, (8, 6), (3, 2), (2, 1), (2, 1), (2, 1), 3, 1, 2.0),
    (2, 2, 2, 4, 7, 1, 2, 2, 2, 2, 2, 1.0),          # deform2d_double/test_gradient.py:7-19 shape
    (3, 2, 4, 4, (5, 6, 7), 3, 1, 1, 1, 2, 2, 3.0),
    (3, 1, 6, 3, (4, 7, 5), (2, 3, 1), (1, 2, 1), (1, 2, 0), (1, 2, 1), 2, 3, 2.0),
    (3, 2, 2, 4, 7, 3, 2, 2, 2, 2, 2, 1.0),          # deform3d/test_gradient.py:9-20 shape
]


def oracle_fwd(c, acc64=True):
    return orc.forward(c["x"], c["off"], c["w"], c["b"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"],
                       acc64=acc64)


def oracle_bwd(c, acc64=True):
    return orc.backward(c["x"], c["off"], c["w"], c["gout"], c["b"], c["stride"], c["pad"], c["dil"], c["cpg"],
                        c["groups"], acc64=acc64)


def inside_mask(c):
    """[N, DG, kV, *out] bool: the reference's strict (-1, size) window on every axis."""
    DG = c["x"].shape[1] // c["cpg"]
    p = comp.sample_coords(c["off"], c["ins"], c["k"], c["stride"], c["pad"], c["dil"], DG)
    m = torch.ones_like(p[:, :, :, 0], dtype=torch.bool)
    for a in range(c["nd"]):
        m &= (p[:, :, :, a] > -1) & (p[:, :, :, a] < c["ins"][a])
    return m, p


# ---------------------------------------------------------------------------------------------
# sampler: hand cases through a 1x1(x1) kernel whose single tap is moved by the offset

@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_sampler_hand_cases_2d(dtype):
    H, W = 4, 5
    im = torch.arange(H * W, dtype=dtype).reshape(1, H, W) + 1
    # (ph, pw) -> expected value
    bil = lambda h, w: ((im[0, int(h), int(w)] * (1 - (w - int(w))) + im[0, int(h), int(w) + 1] * (w - int(w))) * (1 - (h - int(h)))
                        + (im[0, int(h) + 1, int(w)] * (1 - (w - int(w))) + im[0, int(h) + 1, int(w) + 1] * (w - int(w))) * (h - int(h)))
    cases = {
        (0.0, 0.0): im[0, 0, 0], (2.0, 3.0): im[0, 2, 3], (3.0, 4.0): im[0, 3, 4],      # integer coords
        (1.25, 2.5): bil(1.25, 2.5), (0.5, 0.75): bil(0.5, 0.75),                        # textbook bilinear
        (-0.5, 1.0): im[0, 0, 1], (-0.999, 0.0): im[0, 0, 0],                            # low rim replicates
        (1.0, -0.25): im[0, 1, 0],
        (3.5, 2.0): im[0, 3, 2], (2.0, 4.75): im[0, 2, 4], (3.999, 4.999): im[0, 3, 4],  # high rim replicates
        (-1.0, 1.0): 0.0, (1.0, -1.0): 0.0, (4.0, 1.0): 0.0, (1.0, 5.0): 0.0,            # strict window
        (-1.5, 2.0): 0.0, (2.0, 7.0): 0.0,
    }
    for (ph, pw), want in cases.items():
        off = torch.zeros(2, H, W, dtype=dtype)
        off[0, 0, 0], off[1, 0, 0] = ph, pw        # position (0,0): base coordinate is (0,0)
        col = orc.im2col(im, off, (1, 1), 1, 0, 1, 1)
        assert abs(float(col[0, 0]) - float(want)) < 1e-5, (ph, pw, float(col[0, 0]), float(want))


def test_sampler_hand_cases_3d():
    D, H, W = 3, 4, 5
    im = torch.randn(1, D, H, W, dtype=torch.float64)

    def tri(l, h, w):
        l0, h0, w0 = int(l), int(h), int(w)
        r = 0.0
        for dl, dh, dw in itertools.product((0, 1), repeat=3):
            wt = (l - l0 if dl else 1 - (l - l0)) * (h - h0 if dh else 1 - (h - h0)) * (w - w0 if dw else 1 - (w - w0))
            if wt != 0:
                r += wt * float(im[0, l0 + dl, h0 + dh, w0 + dw])
        return r

    cases = {
        (1.0, 2.0, 3.0): float(im[0, 1, 2, 3]), (0.5, 1.25, 2.75): tri(0.5, 1.25, 2.75),
        (1.5, 0.0, 0.5): tri(1.5, 0.0, 0.5),
        (-0.5, 1.0, 1.0): float(im[0, 0, 1, 1]), (2.5, 3.5, 4.5): float(im[0, 2, 3, 4]),
        (1.0, -0.75, 2.0): float(im[0, 1, 0, 2]),
        (-1.0, 1.0, 1.0): 0.0, (3.0, 1.0, 1.0): 0.0, (1.0, 4.0, 1.0): 0.0, (1.0, 1.0, 5.0): 0.0, (1.0, 1.0, -1.0): 0.0,
    }
    for (pl, ph, pw), want in cases.items():
        off = torch.zeros(3, D, H, W, dtype=torch.float64)
        off[0, 0, 0, 0], off[1, 0, 0, 0], off[2, 0, 0, 0] = pl, ph, pw
        col = orc.im2col(im, off, (1, 1, 1), 1, 0, 1, 1)
        assert abs(float(col[0, 0]) - want) < 1e-12, (pl, ph, pw)


# ---------------------------------------------------------------------------------------------
# forward

@pytest.mark.parametrize("case", CASES)
def test_forward_matches_grid_sample_composite(case):
    c = make_case(*case)
    got = oracle_fwd(c)
    want = comp.deform_conv(c["x"], c["off"], c["w"], c["b"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    m, _ = inside_mask(c)
    assert 0.05 < m.double().mean() < 0.98 or case[-1] <= 1.0   # the case mixes inside and outside samples
    assert (got - want).abs().max() < 1e-12


@pytest.mark.parametrize("nd,dil,stride,groups", [(2, 1, 1, 1), (2, 2, 1, 2), (2, 3, 2, 1), (3, 1, 1, 1), (3, 2, 1, 2),
                                                   (3, (1, 2, 2), (1, 2, 1), 1)])
def test_zero_offset_is_plain_convolution(nd, dil, stride, groups):
    c = make_case(nd, 2, 4, 6, (7, 8) if nd == 2 else (5, 6, 7), 3, stride, 1, dil, 2, groups, 0.0)
    got = oracle_fwd(c)
    # the reference's dilation-blind output size evaluates (d-1)(k-1) extra trailing taps over
    # implicit zeros: pad the input on the right by that much and crop the library result.
    conv = F.conv2d if nd == 2 else F.conv3d
    rp = []
    for a in reversed(range(nd)):
        rp += [0, (c["dil"][a] - 1) * (c["k"][a] - 1)]
    want = conv(F.pad(c["x"], rp), c["w"], c["b"], c["stride"], c["pad"], c["dil"], groups)
    assert got.shape == want.shape
    assert (got - want).abs().max() < 1e-12


def test_integer_offsets_are_shifted_taps_bruteforce():
    # 2-D, one deformable group: offset (dh, dw) per tap, constant over positions, so that
    # out[m,ho,wo] = sum_{c,kh,kw} W[m,c,kh,kw] * xpad[c, ho-pad+kh+dh, wo-pad+kw+dw] with zero outside.
    c = make_case(2, 1, 3, 2, (6, 7), 3, 1, 1, 1, 3, 1, 0.0, bias=False)
    shifts = torch.randint(-2, 3, (9, 2))
    c["off"] = shifts.to(torch.float64).reshape(1, 18, 1, 1).expand(1, 18, 6, 7).contiguous()
    got = oracle_fwd(c)
    want = torch.zeros_like(got)
    x, w = c["x"], c["w"]
    for m, ho, wo in itertools.product(range(2), range(6), range(7)):
        s = 0.0
        for ci, kh, kw in itertools.product(range(3), range(3), range(3)):
            dh, dw = shifts[kh * 3 + kw].tolist()
            h, ww = ho - 1 + kh + dh, wo - 1 + kw + dw
            if 0 <= h < 6 and 0 <= ww < 7:
                s += float(w[m, ci, kh, kw]) * float(x[0, ci, h, ww])
        want[0, m, ho, wo] = s
    assert (got - want).abs().max() < 1e-12


def test_reference_script_shape_3d_ones():
    # deform3d/test_function.py:6-25: 1x1x3x3x3 input with rows [1,2,1] over h, all-ones 3x3x3
    # weight, zero offsets, pad 1, stride 1, dilation 2 -> taps at {-1, 1, 3} per axis, i.e.
    # only the middle tap (coordinate 1) of each axis is inside: every output equals x[1,1,1]=2
    # at position (0,0,0); in general out[o] = sum over taps with 0<=o-1+2k<3 of x[...].
    x = torch.tensor([[1.0, 1, 1], [2.0, 2, 2], [1.0, 1, 1]]).repeat(3, 1, 1).reshape(1, 1, 3, 3, 3)
    off = torch.zeros(1, 81, 3, 3, 3)
    w = torch.ones(1, 1, 3, 3, 3)
    got = orc.forward(x, off, w, None, 1, 1, 2, 1, 1)
    want = torch.zeros(3, 3, 3)
    for o in itertools.product(range(3), repeat=3):
        s = 0.0
        for k in itertools.product(range(3), repeat=3):
            p = [o[a] - 1 + 2 * k[a] for a in range(3)]
            if all(0 <= q < 3 for q in p):
                s += float(x[0, 0, p[0], p[1], p[2]])
        want[o] = s
    assert torch.equal(got[0, 0], want)
    assert float(got[0, 0, 0, 0, 0]) == 2.0


# ---------------------------------------------------------------------------------------------
# backward

@pytest.mark.parametrize("case", CASES)
def test_backward_matches_autograd_of_composite(case):
    c = make_case(*case)
    x, off, w, b = (c[k].clone().requires_grad_(True) for k in ("x", "off", "w", "b"))
    out = comp.deform_conv(x, off, w, b, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    out.backward(c["gout"])
    gin, goff, gw, gb = oracle_bwd(c)
    assert (gin - x.grad).abs().max() < 1e-11
    assert (gw - w.grad).abs().max() < 1e-11
    assert (gb - b.grad).abs().max() < 1e-11
    m, p = inside_mask(c)                                  # [N,DG,kV,*out]
    nd = c["nd"]
    goff_v = goff.reshape(p.shape)
    ref_v = off.grad.reshape(p.shape)
    mm = m.unsqueeze(3).expand_as(goff_v)
    assert (goff_v[mm] - ref_v[mm]).abs().max() < 1e-11
    if nd == 2:
        # 2-D: samples outside the window get exactly zero (deform2d_double kernel.cu:324-365)
        assert goff_v[~mm].abs().max() == 0 if (~mm).any() else True
    else:
        # 3-D: the reference's out-of-range branches, kernel.cu:470-481, stated in words:
        # S = sum over the group's channels of |grad-column|; axis a gets -S when its coordinate
        # is <= -1, +S when it is >= the LENGTH extent (also for h and w), else 0.
        N, C = c["x"].shape[:2]
        G, cpg = c["groups"], c["cpg"]
        kV = math.prod(c["k"])
        M = c["w"].shape[0] // G
        wg = c["w"].reshape(G, M, C // G, kV)
        gcol = torch.einsum("gmck,ngmp->ngckp", wg, c["gout"].reshape(N, G, M, -1)).reshape(N, C // cpg, cpg, kV, -1)
        S = gcol.abs().sum(2).reshape(m.shape)
        want = torch.zeros_like(goff_v)
        for a in range(3):
            want[:, :, :, a] = torch.where(p[:, :, :, a] <= -1, -S, torch.where(p[:, :, :, a] >= c["ins"][0], S, torch.zeros_like(S)))
        assert (goff_v[~mm] - want[~mm]).abs().max() < 1e-11


@pytest.mark.parametrize("nd", [2, 3])
def test_im2col_col2im_adjoint(nd):
    c = make_case(nd, 1, 4, 4, (6, 7) if nd == 2 else (4, 5, 6), 3, 1, 1, 1, 2, 1, 2.5)
    im, off = c["x"][0], c["off"][0]
    col = orc.im2col(im, off, c["k"], c["stride"], c["pad"], c["dil"], c["cpg"])
    g = torch.randn_like(col)
    back = orc.col2im_input(g, off, im.shape, c["k"], c["stride"], c["pad"], c["dil"], c["cpg"])
    assert abs(float((col * g).sum() - (im * back).sum())) < 1e-10


class _OracleFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, off, w, b, stride, pad, dil, cpg, groups):
        ctx.save_for_backward(x, off, w, b)
        ctx.cfg = (stride, pad, dil, cpg, groups)
        return orc.forward(x.detach(), off.detach(), w.detach(), b.detach(), *ctx.cfg)

    @staticmethod
    def backward(ctx, gout):
        x, off, w, b = ctx.saved_tensors
        gin, goff, gw, gb = orc.backward(x.detach(), off.detach(), w.detach(), gout.contiguous(), b.detach(), *ctx.cfg)
        return gin, goff, gw, gb, None, None, None, None, None


def test_gradcheck_2d_reference_shape():
    # deform2d_double/test_gradient.py:7-53 -- the gradcheck the reference's author reports passing.
    g = torch.Generator().manual_seed(5)
    x = torch.rand(2, 2, 7, 7, generator=g, dtype=torch.float64, requires_grad=True)
    off = torch.rand(2, 2, 6, 6, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.rand(4, 1, 1, 1, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.rand(4, generator=g, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_OracleFn.apply, (x, off, w, b, (2, 2), (2, 2), (2, 2), 2, 2),
                                    eps=1e-6, atol=1e-5, rtol=1e-3)


def test_gradcheck_2d_c1_shape_small():
    # BASELINE configs[0] geometry (k3 p1, 1 deformable group) at reduced extent; offsets
    # U[-1.5,1.5] kept away from integer coordinates where the sampler has kinks.
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1, 4, 6, 6, generator=g, dtype=torch.float64, requires_grad=True)
    off = (torch.rand(1, 18, 6, 6, generator=g, dtype=torch.float64) * 3 - 1.5)
    frac = off - off.round()
    off = torch.where(frac.abs() < 0.05, off + 0.1, off).requires_grad_(True)
    w = torch.randn(4, 4, 3, 3, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(4, generator=g, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_OracleFn.apply, (x, off, w, b, (1, 1), (1, 1), (1, 1), 4, 1),
                                    eps=1e-6, atol=1e-5, rtol=1e-3)


def test_gradcheck_3d_in_range():
    # 3-D passes gradcheck only while every sample stays inside the volume (the out-of-range
    # branches are not a derivative): small offsets, pad 0.
    g = torch.Generator().manual_seed(9)
    x = torch.randn(1, 2, 5, 5, 5, generator=g, dtype=torch.float64, requires_grad=True)
    off = (torch.rand(1, 2 * 8 * 3, 4, 4, 4, generator=g, dtype=torch.float64) * 0.8 + 0.1).requires_grad_(True)
    w = torch.randn(2, 1, 2, 2, 2, generator=g, dtype=torch.float64, requires_grad=True)
    b = torch.randn(2, generator=g, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(_OracleFn.apply, (x, off, w, b, (1, 1, 1), (0, 0, 0), (1, 1, 1), 1, 2),
                                    eps=1e-6, atol=1e-5, rtol=1e-3)


def test_oob_branch_hand_case_3d():
    # One channel, 1x1x1 kernel, D=2 < H=W=6, unit weight, grad_output = v at one position.
    # gcol = v.  Push the sample out low on l -> grad_offset_l = -|v|; high on l (p_l >= 2) ->
    # +|v|; out on l with 2 <= p_h < 6 -> axis h also gets +|v| (it is tested against D);
    # out on l with p_w <= -1 -> axis w gets -|v|.
    x = torch.randn(1, 1, 2, 6, 6, dtype=torch.float64)
    w = torch.ones(1, 1, 1, 1, 1, dtype=torch.float64)
    v = -0.7
    gout = torch.zeros(1, 1, 2, 6, 6, dtype=torch.float64)
    gout[0, 0, 0, 1, 1] = v

    def run(ol, oh, ow):
        off = torch.zeros(1, 3, 2, 6, 6, dtype=torch.float64)
        off[0, 0, 0, 1, 1], off[0, 1, 0, 1, 1], off[0, 2, 0, 1, 1] = ol, oh, ow
        _, goff, _, _ = orc.backward(x, off, w, gout, None, 1, 0, 1, 1, 1)
        return [float(goff[0, a, 0, 1, 1]) for a in range(3)]

    a = abs(v)
    assert run(-1.0, 0.0, 0.0) == [-a, 0.0, 0.0]          # p = (-1, 1, 1)
    assert run(2.0, 0.0, 0.0) == [a, 0.0, 0.0]            # p = (2, 1, 1)
    assert run(2.0, 1.0, 0.0) == [a, a, 0.0]              # p = (2, 2, 1): h tested against D=2
    assert run(-3.0, 3.5, -2.0) == [-a, a, -a]            # p = (-3, 4.5, -1)
    assert run(0.5, 5.0, 0.0) == [0.0, a, 0.0]            # p = (0.5, 6, 1): only h is out
    assert run(0.5, 0.0, 0.0)[0] != 0.0                   # inside: a real derivative on l


def test_float_oracle_close_to_double():
    c64 = make_case(3, 2, 4, 4, (5, 6, 7), 3, 1, 1, 1, 2, 2, 1.5)
    c32 = {k: (v.float() if torch.is_tensor(v) else v) for k, v in c64.items()}
    # compare on the float-rounded inputs so only arithmetic differs
    c64r = {k: (v.double() if torch.is_tensor(v) else v) for k, v in c32.items()}
    for acc64 in (True, False):
        d = (oracle_fwd(c32, acc64).double() - oracle_fwd(c64r)).abs().max()
        assert d < 1e-4
        for a, b in zip(oracle_bwd(c32, acc64), oracle_bwd(c64r)):
            assert (a.double() - b).abs().max() < 1e-3


def test_blas_sequencing_equals_the_oracle_loops():
    """The reference's per-sample loop with torch.mm for its three GEMMs (the timed CPU baseline) gives
    what the oracle's own loops give."""
    for name in ("3d_basic", "2d_c3_like", "3d_mixed"):
        c = make_case(*SMALL_CASES[name], dtype=torch.float64, seed=21, bias=False)
        cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
        out, gin, goff, gw = orc.step_blas(c["x"], c["off"], c["w"], c["gout"], *cfg)
        want_out = orc.forward(c["x"], c["off"], c["w"], None, *cfg)
        want = orc.backward(c["x"], c["off"], c["w"], c["gout"], None, *cfg)
        for got, ref in ((out, want_out), (gin, want[0]), (goff, want[1]), (gw, want[2])):
            assert (got - ref).abs().max().item() <= 1e-12 * max(1.0, ref.abs().max().item()), name
