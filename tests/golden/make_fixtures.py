"""Writes the golden fixtures tests/golden/*.npz from the CPU oracle.

Run from the repository root after tests/test_oracle.py is green (the oracle then agrees with the
independent grid_sample composite):  python tests/golden/make_fixtures.py

The reference (lshiwjx/deform_conv3d_pytorch_op) holds no golden vectors and cannot be imported
(torch.utils.ffi is gone, it needs nvcc and a CUDA device), so these vectors come from the
build's oracle in float64.  Shapes follow the reference's own scripts where it has them
(deform3d/test_function.py:6-25, deform3d/test_gradient.py:9-20, deform2d_double/test_gradient.py:7-19,
deform2d_double/test_model.py:8-30) plus one case per out-of-range branch of the 3-D grad-offset.
Each file holds the inputs, the geometry and the expected output and gradients.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import dcn_oracle as orc          # noqa: E402
from tests.cases import make_case, SMALL_CASES  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def save(name, c):
    # inputs are rounded to float32-representable values first, so that the float32 build sees
    # exactly the data the float64 expectations were computed from (same inside / outside decisions)
    c = dict(c)
    for k in ("x", "off", "w", "gout", "b"):
        if c.get(k) is not None:
            c[k] = c[k].float().double()
    out = orc.forward(c["x"], c["off"], c["w"], c["b"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    gin, goff, gw, gb = orc.backward(c["x"], c["off"], c["w"], c["gout"], c["b"], c["stride"], c["pad"], c["dil"],
                                     c["cpg"], c["groups"])
    d = dict(x=c["x"].numpy(), off=c["off"].numpy(), w=c["w"].numpy(), gout=c["gout"].numpy(),
             geom=np.array(list(c["stride"]) + list(c["pad"]) + list(c["dil"]) + [c["cpg"], c["groups"]]),
             out=out.numpy(), gin=gin.numpy(), goff=goff.numpy(), gw=gw.numpy())
    if c["b"] is not None:
        d["b"] = c["b"].numpy()
        d["gb"] = gb.numpy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **d)
    print(name, {k: v.shape for k, v in d.items() if k != "geom"})


def main():
    for name in ("2d_ref_gradient_script", "3d_ref_gradient_script", "2d_c3_like", "3d_short_length", "3d_mixed"):
        save(name, make_case(*SMALL_CASES[name], seed=11))
    # deform3d/test_function.py:6-25 verbatim: rows [1,2,1], ones weight, zero offsets, dilation 2
    x = torch.tensor([[1.0, 1, 1], [2.0, 2, 2], [1.0, 1, 1]], dtype=torch.float64).repeat(3, 1, 1).reshape(1, 1, 3, 3, 3)
    c = dict(x=x, off=torch.zeros(1, 81, 3, 3, 3, dtype=torch.float64), w=torch.ones(1, 1, 3, 3, 3, dtype=torch.float64),
             b=None, gout=torch.ones(1, 1, 3, 3, 3, dtype=torch.float64), stride=(1, 1, 1), pad=(1, 1, 1),
             dil=(2, 2, 2), cpg=1, groups=1)
    save("3d_ref_function_script", c)
    # deform2d_double/test_model.py:8-30: ones input, zero offsets, pad 2, dilation 2, groups 2
    c = dict(x=torch.ones(1, 2, 5, 5, dtype=torch.float64), off=torch.zeros(1, 36, 7, 7, dtype=torch.float64),
             w=torch.ones(2, 1, 3, 3, dtype=torch.float64), b=torch.tensor([0.05, -0.05], dtype=torch.float64),
             gout=torch.ones(1, 2, 7, 7, dtype=torch.float64), stride=(1, 1), pad=(2, 2), dil=(2, 2), cpg=1, groups=2)
    save("2d_ref_model_script", c)


if __name__ == "__main__":
    main()
