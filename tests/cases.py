"""Seeded problem instances shared by the CPU and GPU tests (they live in the package, beside the
benchmark configurations that use the same generator)."""
from deform_conv3d_pytorch_op_amd.synthetic import SMALL_CASES, make_case, output_size, random_spec  # noqa: F401
