"""Seeded synthetic problem instances: the inputs of the benchmark, of smoke() and of the tests."""
import math

import torch


def _t(v, nd):
    return (v,) * nd if isinstance(v, int) else tuple(v)


def output_size(ins, ks, stride, pad):
    return tuple((i + 2 * p - k) // s + 1 for i, k, s, p in zip(ins, ks, stride, pad))


def make_case(nd, N, C_in, C_out, ins, k, stride, pad, dil, cpg, groups, off_scale, dtype=torch.float64,
              seed=0, bias=True, off_dist="uniform"):
    g = torch.Generator().manual_seed(seed)
    ins, k, stride, pad, dil = _t(ins, nd), _t(k, nd), _t(stride, nd), _t(pad, nd), _t(dil, nd)
    outs = output_size(ins, k, stride, pad)
    kV = math.prod(k)
    x = torch.randn((N, C_in) + ins, generator=g, dtype=torch.float64)
    oshape = (N, C_in // cpg * nd * kV) + outs
    if off_dist == "uniform":
        off = (torch.rand(oshape, generator=g, dtype=torch.float64) * 2 - 1) * off_scale
    else:   # N(0,1) with 10 % of the entries replaced by U[-6,6]  (BASELINE configs[2])
        off = torch.randn(oshape, generator=g, dtype=torch.float64)
        mask = torch.rand(oshape, generator=g, dtype=torch.float64) < 0.1
        wide = (torch.rand(oshape, generator=g, dtype=torch.float64) * 2 - 1) * 6
        off = torch.where(mask, wide, off)
    fan_out = C_out * kV
    w = torch.randn((C_out, C_in // groups) + k, generator=g, dtype=torch.float64) * math.sqrt(2.0 / fan_out)
    b = torch.randn(C_out, generator=g, dtype=torch.float64) if bias else None
    gout = torch.randn((N, C_out) + outs, generator=g, dtype=torch.float64)
    cast = lambda t: None if t is None else t.to(dtype).contiguous()
    return dict(x=cast(x), off=cast(off), w=cast(w), b=cast(b), gout=cast(gout), stride=stride, pad=pad, dil=dil,
                cpg=cpg, groups=groups, ins=ins, k=k, outs=outs, nd=nd)


# nd, N, Cin, Cout, in, k, stride, pad, dil, cpg, groups, off_scale
SMALL_CASES = {
    "2d_basic": (2, 2, 4, 6, (7, 9), 3, 1, 1, 1, 2, 2, 3.0),
    "2d_rect_kernel_stride_dil": (2, 1, 6, 4, (8, 6), (3, 2), (2, 1), (2, 1), (2, 1), 3, 1, 2.0),
    "2d_ref_gradient_script": (2, 2, 2, 4, 7, 1, 2, 2, 2, 2, 2, 1.0),      # deform2d_double/test_gradient.py:7-19
    "2d_c1": (2, 2, 8, 8, 16, 3, 1, 1, 1, 8, 1, 1.5),                     # BASELINE configs[0]
    "2d_wide_m": (2, 1, 40, 72, (9, 11), 3, 1, 1, 1, 20, 1, 2.0),          # several MFMA row tiles, 2 deformable groups
    "2d_many_m_chunks": (2, 1, 6, 300, (6, 7), 3, 1, 1, 1, 6, 1, 1.0),     # M > 8 row tiles of 32
    "2d_c3_like": (2, 1, 16, 8, 10, 3, 1, 2, 2, 4, 2, 3.0),                # groups 2, 4 deformable groups, dilation 2
    "2d_cpg_straddles_groups": (2, 1, 12, 4, 6, 3, 1, 1, 1, 12, 2, 1.5),   # one deformable group over two conv groups
    "2d_long_reduction": (2, 1, 8, 400, (6, 7), 3, 1, 1, 1, 8, 1, 1.0),           # M = 400: the long-reduction form of the fused kernel's GEMM loop in both precisions
    "2d_chunk8_ragged": (2, 2, 22, 10, (9, 8), 3, 1, 1, 1, 11, 1, 2.0),            # 11-channel segments: chunks of 8 + 3
    "2d_cpg_unaligned": (2, 1, 12, 6, 6, 2, 1, 0, 1, 4, 2, 1.5),           # cpg 4, 6 channels per conv group
    "3d_basic": (3, 2, 4, 4, (5, 6, 7), 3, 1, 1, 1, 2, 2, 3.0),
    "3d_mixed": (3, 1, 6, 3, (4, 7, 5), (2, 3, 1), (1, 2, 1), (1, 2, 0), (1, 2, 1), 2, 3, 2.0),
    "3d_ref_gradient_script": (3, 2, 2, 4, 7, 3, 2, 2, 2, 2, 2, 1.0),      # deform3d/test_gradient.py:9-20
    "3d_c4_like": (3, 2, 40, 40, (4, 9, 10), 3, 1, 1, 1, 40, 1, 1.5),      # one deformable group, >1 channel tile
    "3d_c5_like": (3, 1, 16, 24, (4, 12, 12), 3, (1, 2, 2), 1, 1, 4, 1, 2.0),   # strided, 4 deformable groups
    "3d_wide_m": (3, 1, 8, 136, (3, 6, 6), 3, 1, 1, 1, 8, 1, 2.0),        # more reduction steps than one pass of tap slots takes
    "2d_k5_depthwise": (2, 1, 6, 6, (9, 9), 5, 1, 2, 1, 1, 6, 1.0),         # 25 taps, one channel per group and per deformable group
    "3d_k1_stride3": (3, 2, 5, 7, (5, 7, 6), 1, 3, 0, 1, 5, 1, 2.0),         # a single tap, odd channel counts, stride > kernel
    "3d_dilation3": (3, 1, 4, 4, (8, 8, 8), 3, 1, 3, 3, 2, 1, 2.5),          # dilation-blind output 12^3: many taps out of range
    "3d_short_length": (3, 1, 4, 4, (2, 8, 8), (1, 3, 3), 1, (0, 1, 1), 1, 4, 1, 4.0),  # D < H: out-of-range branch vs length extent
    "3d_chunk8_ragged": (3, 1, 20, 40, (5, 9, 10), 3, 1, 1, 1, 10, 1, 2.0),     # 10-channel segments: chunks of 8 + 2, 20 reduction steps (not a multiple of 16)
    "3d_chunk8_two_blocks": (3, 2, 16, 24, (6, 10, 18), 3, 1, 1, 1, 16, 1, 1.5),   # several position blocks per axis, 8-channel chunks, 12 reduction steps
    "3d_k5": (3, 1, 8, 6, (6, 7, 7), 5, 1, 2, 1, 8, 1, 1.5),                  # 125 taps: too many terms per LDS cell for the paired float cells
    "2d_k7": (2, 1, 8, 10, (12, 11), 7, 1, 3, 1, 8, 1, 2.0),                   # 49 taps
    "3d_m72_chunk8": (3, 1, 16, 72, (4, 8, 9), 3, 1, 1, 1, 8, 1, 1.5),        # 36 reduction steps: the grad_output operand does not fit the registers
    "3d_m100_chunk4": (3, 1, 8, 100, (4, 8, 9), 3, 1, 1, 1, 4, 1, 1.5),       # 50 reduction steps, 4-channel chunks: the operand takes two register sets
    "2d_chunk16_small_m": (2, 1, 32, 24, (12, 13), 3, 1, 1, 1, 16, 1, 1.5),    # 16-channel chunks (float32), grad_output operand in registers, two deformable groups
    "2d_chunk16_ragged": (2, 2, 44, 100, (10, 9), 3, 1, 1, 1, 22, 1, 2.0),     # 22-channel segments: chunks of 16 + 6, 50 reduction steps
    "2d_chunk16_k1": (2, 1, 16, 8, (9, 10), 1, 1, 0, 1, 16, 1, 1.0),           # a single tap: one pass of two tap slots, one of them empty
}


def random_spec(seed, medium=False):
    """A small random geometry (the SMALL_CASES tuple layout), reproducible from `seed`: odd channel
    counts, every divisor as channels per deformable group, rectangular kernels, strides, pads and
    dilations per axis.  `medium`: extents of several position tiles per axis and more channels."""
    import random
    r = random.Random((5000 if medium else 1000) + seed)
    nd = r.choice((2, 3))
    groups = r.choice((1, 1, 2, 3))
    cg = r.randint(1, 12) if not medium else r.randint(4, 24)
    c_in = groups * cg
    cpg = r.choice([d for d in range(1, c_in + 1) if c_in % d == 0])
    c_out = groups * r.randint(1, 40 if nd == 2 else 24)
    k = tuple(r.randint(1, 3) for _ in range(nd))
    stride = tuple(r.randint(1, 2) for _ in range(nd))
    dil = tuple(r.randint(1, 2) for _ in range(nd))
    pad = tuple(r.randint(0, 2) for _ in range(nd))
    if medium:
        ins = tuple(r.randint(14, 40 if nd == 2 else 20) for _ in range(nd))
        return (nd, r.randint(1, 2), c_in, c_out, ins, k, stride, pad, dil, cpg, groups, r.choice((0.5, 1.5, 3.0)))
    ins = tuple(r.randint(max(3, kk - 2 * p), 12 if nd == 2 else 8) for kk, p in zip(k, pad))
    return (nd, r.randint(1, 3), c_in, c_out, ins, k, stride, pad, dil, cpg, groups, r.choice((0.5, 2.0, 4.0)))
