"""Independent restatement of the deformable convolution out of library routines only.

It shares no code with the oracle: the sampled column tensor is
`grid_sample(mode='bilinear', padding_mode='border', align_corners=True)` times the mask
`-1 < p < size` on every axis, and the output is an einsum with the weight.  'border' clamps
the coordinate to [0, size-1], which reproduces the reference's replicate-in-rim rule
(deform3d/lib/deform_conv3d_cuda_kernel.cu:21-26,123-124); 5-D grid_sample is trilinear.
Autograd through this composite yields grad_input, grad_weight and the in-range part of
grad_offset (the mask has zero gradient and border mode has zero grid-gradient where clamped).
Requires every input extent > 1.
"""
import torch
import torch.nn.functional as F


def output_size(ins, ks, stride, pad):
    return tuple((i + 2 * p - k) // s + 1 for i, k, s, p in zip(ins, ks, stride, pad))


def sample_coords(offset, ins, ks, stride, pad, dil, DG):
    """offset [N, DG*kV*nd, *out] -> p [N, DG, kV, nd, *out] (absolute sampling coordinates)."""
    nd = len(ins)
    N = offset.shape[0]
    outs = tuple(offset.shape[2:])
    kV = 1
    for k in ks:
        kV *= k
    off = offset.reshape((N, DG, kV, nd) + outs)
    base = torch.zeros((kV, nd) + outs, dtype=offset.dtype)
    taps = torch.cartesian_prod(*[torch.arange(k) for k in ks]).reshape(kV, nd)
    for a in range(nd):
        shape = [1] * nd
        shape[a] = outs[a]
        o = (torch.arange(outs[a]) * stride[a] - pad[a]).reshape(shape)
        base[:, a] = (o.unsqueeze(0) + (taps[:, a] * dil[a]).reshape((kV,) + (1,) * nd)).to(offset.dtype)
    return off + base


def columns(x, offset, ks, stride, pad, dil, cpg):
    """Sampled column tensor [N, C, kV, *out] built from grid_sample."""
    N, C = x.shape[:2]
    ins = tuple(x.shape[2:])
    nd = len(ins)
    DG = C // cpg
    p = sample_coords(offset, ins, ks, stride, pad, dil, DG)          # [N,DG,kV,nd,*out]
    outs = tuple(p.shape[4:])
    kV = p.shape[2]
    outV = 1
    for o in outs:
        outV *= o
    inside = torch.ones_like(p[:, :, :, 0], dtype=torch.bool)
    for a in range(nd):
        inside = inside & (p[:, :, :, a] > -1) & (p[:, :, :, a] < ins[a])
    # grid_sample wants the last dim ordered (w, h[, l]) and normalised to [-1, 1]
    norm = [2 * p[:, :, :, a] / (ins[a] - 1) - 1 for a in range(nd)]
    grid = torch.stack(norm[::-1], dim=-1)                            # [N,DG,kV,*out,nd]
    xg = x.reshape((N * DG, cpg) + ins)
    if nd == 2:
        g = grid.reshape(N * DG, kV * outs[0], outs[1], 2)
    else:
        g = grid.reshape(N * DG, kV * outs[0], outs[1], outs[2], 3)
    s = F.grid_sample(xg, g, mode="bilinear", padding_mode="border", align_corners=True)
    s = s.reshape((N, DG, cpg, kV) + outs)
    s = s * inside.unsqueeze(2).to(x.dtype)
    return s.reshape((N, C, kV) + outs)


def deform_conv(x, offset, weight, bias=None, stride=1, pad=0, dil=1, cpg=1, groups=1):
    nd = x.dim() - 2
    t = lambda v: (v,) * nd if isinstance(v, int) else tuple(v)
    stride, pad, dil = t(stride), t(pad), t(dil)
    ks = tuple(weight.shape[2:])
    col = columns(x, offset, ks, stride, pad, dil, cpg)               # [N,C,kV,*out]
    N, C = x.shape[:2]
    outs = tuple(col.shape[3:])
    kV = col.shape[2]
    Cg = C // groups
    M = weight.shape[0] // groups
    colg = col.reshape(N, groups, Cg * kV, -1)
    wg = weight.reshape(groups, M, Cg * kV)
    out = torch.einsum("gmk,ngkp->ngmp", wg, colg).reshape((N, weight.shape[0]) + outs)
    if bias is not None:
        out = out + bias.view((1, -1) + (1,) * nd)
    return out
