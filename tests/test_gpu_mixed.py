"""16-bit storage entry points (dcn*_bf16, dcn*_f16) through the package's Functions: every tensor is
stored as bfloat16 / binary16.  Backward to weight: like the forward pass, the columns are sampled in float32
from the 16-bit input, rounded to the storage format and multiplied with grad_output in 16-bit matrix
instructions with float32 accumulation (layers with an odd number of input channels: widened and computed by
the float32 kernel).  Backward to input and offset: the fused kernel reads the
16-bit tensors, forms the grad columns with 16-bit matrix instructions (exact products, float32 sums) and
each result is rounded once.  Forward: the columns are sampled in float32,
rounded to the storage format and multiplied with the weights in 16-bit matrix instructions with
float32 accumulation.  Oracle mode: the CPU oracle in float32 with double accumulation on the same
16-bit-rounded inputs: the kernels form the sampling coordinates in float32, as the reference does
(deform3d/lib/deform_conv3d_cuda_kernel.cu:110-124), and a 16-bit offset such as -7e-7 next to an integer
coordinate rounds onto that integer in float32 but not in float64 -- a float64 oracle then samples the
other side of a corner, or inside instead of outside, for single samples in a few percent of the
geometries of a wide sweep.
A gradient then differs from the oracle by the float32 kernels' error plus one rounding to the
storage format, half an ulp of the element (2^-9 of its magnitude for bfloat16, 2^-12 for
binary16); an output element additionally by the rounding of its sampled columns.  Tolerances,
relative to the tensor's largest magnitude: bfloat16 5e-3, binary16 1e-3 forward / 2e-3 gradients.
The reference has no such mode (deform3d/lib/deform_conv3d_cuda_kernel.cu:162-172 instantiates float only).
"""
import pytest
import torch

from oracle import dcn_oracle as orc
from tests.cases import SMALL_CASES, make_case, random_spec
from tests.test_gpu_parity import rel_err, run_gpu

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: dict(fwd=5e-3, grad=5e-3), torch.float16: dict(fwd=1e-3, grad=2e-3)}
CASES = ["2d_basic", "2d_c3_like", "2d_wide_m", "2d_chunk8_ragged", "3d_basic", "3d_mixed", "3d_c4_like", "3d_c5_like",
         "3d_short_length"]
MEDIUM = {   # several position blocks, more than one channel chunk
    "3d_medium": (3, 2, 24, 40, (6, 20, 18), 3, 1, 1, 1, 12, 1, 2.0),
    "2d_medium": (2, 2, 48, 64, (30, 34), 3, 1, 1, 1, 16, 2, 2.0),
}


def _compare(c, dtype, tag):
    got = run_gpu(c)
    for g in got:
        assert g is None or g.dtype == dtype
    wide = {k: (v.float() if torch.is_tensor(v) else v) for k, v in c.items()}       # (float32 coordinates: see above)
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    want = (orc.forward(wide["x"], wide["off"], wide["w"], wide["b"], *cfg),) + tuple(
        orc.backward(wide["x"], wide["off"], wide["w"], wide["gout"], wide["b"], *cfg))
    for name, g, w in zip(("output", "grad_input", "grad_offset", "grad_weight", "grad_bias"), got, want):
        if w is None:
            continue
        tol = TOL[dtype]["fwd" if name == "output" else "grad"]
        e = rel_err(g.float(), w)
        assert e <= tol, "%s %s: relative error %.3e > %.1e" % (tag, name, e, tol)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", CASES)
def test_16bit_storage_small_cases_match_oracle(name, dtype):
    print("16-bit case", name, dtype, flush=True)
    _compare(make_case(*SMALL_CASES[name], dtype=dtype, seed=7), dtype, name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("name", sorted(MEDIUM))
def test_16bit_storage_medium_cases_match_oracle(name, dtype):
    print("16-bit case", name, dtype, flush=True)
    _compare(make_case(*MEDIUM[name], dtype=dtype, seed=8), dtype, name)


@pytest.mark.parametrize("seed", range(160))
def test_16bit_storage_random_geometries_match_oracle(seed):
    """Seeded random small (even seeds) and medium (odd seeds) geometries in both 16-bit formats.
    (Seeds 33, 91, 93, 119, 141, 149 hold 16-bit offsets of about -1e-6 beside integer coordinates: single
    samples there differ from an oracle with float64 coordinates, see the module text.)"""
    spec = random_spec(seed, medium=bool(seed % 2))
    print("16-bit random geometry", seed, spec, flush=True)
    for dtype in (torch.bfloat16, torch.float16):
        _compare(make_case(*spec, dtype=dtype, seed=300 + seed), dtype, "random16_%d" % seed)


def test_16bit_gradients_against_the_float32_gradients():
    """backward_input_offset reads the 16-bit tensors itself and multiplies them in 16-bit matrix instructions
    with float32 accumulation -- the products of 16-bit values are exact in float32, so only the order of the
    sums differs from the float32 kernel -- and rounds each result once.  Every bfloat16 element of grad_input
    and grad_offset therefore lies within one rounding (2^-8 of its magnitude) of the float32 gradient on the
    widened inputs, plus what the float32 sums themselves vary by: 1e-6 of the tensor's largest value for the
    order of the sums, 1e-5 for grad_input, whose terms pass through the fixed-point LDS cells (a grad column
    that differs in its last bit may round to the neighbouring fixed-point step).  The forward pass and
    backward_weight round their sampled columns to bfloat16 for the matrix instruction: output and grad_weight
    are close to the float32 results (5e-3 of the largest value), not within one rounding."""
    import deform_conv3d_pytorch_op_amd as dcn
    c = make_case(*SMALL_CASES["3d_c4_like"], dtype=torch.bfloat16, seed=9)
    dev = torch.device("cuda:0")
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    grads = {}
    for dt in (torch.bfloat16, torch.float32):
        x, off, w, b = (c[k].to(dev).to(dt).requires_grad_(True) for k in ("x", "off", "w", "b"))
        out = dcn.ConvOffset3dFunction.apply(x, off, w, b, *cfg)
        out.backward(c["gout"].to(dev).to(dt))
        grads[dt] = (out.detach(), x.grad, off.grad, w.grad)
    for name, g16, g32 in zip(("grad_input", "grad_offset"), grads[torch.bfloat16][1:3], grads[torch.float32][1:3]):
        slack = 2.0 ** -8 * g32.abs() + (1e-5 if name == "grad_input" else 1e-6) * g32.abs().max()
        assert bool(((g16.float() - g32).abs() <= slack).all()), name
    for name, k in (("output", 0), ("grad_weight", 3)):
        v16, v32 = grads[torch.bfloat16][k].float(), grads[torch.float32][k]
        assert (v16 - v32).abs().max().item() <= 5e-3 * v32.abs().max().item(), name


def test_oob_zero_switch_is_float_only():
    import deform_conv3d_pytorch_op_amd as dcn
    c = make_case(*SMALL_CASES["3d_basic"], dtype=torch.float16, seed=1)
    dev = torch.device("cuda:0")
    x, off, w = (c[k].to(dev).requires_grad_(True) for k in ("x", "off", "w"))
    out = dcn.ConvOffset3dFunction.apply(x, off, w, None, c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"], False, "zero")
    with pytest.raises(RuntimeError, match="float32 and float64 only"):
        out.backward(c["gout"].to(dev))
