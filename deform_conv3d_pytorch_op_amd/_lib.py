"""ctypes binding of libdcn_amd.so, the hand-written HIP library for gfx950 (C ABI in
include/dcn_amd.h).  This takes the place of the reference's cffi loader
(deform3d/deform_conv3d_op/__init__.py:1-12, deform2d_double/deform_conv2d_op/__init__.py).

There is no fallback: if the shared library is missing the import of an operator fails with an
error that says how to build it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "csrc", "libdcn_amd.so")

_c_int, _c_vp, _c_sz = ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t
_lib = None

N_GEOM = {3: 23, 2: 17}     # number of int arguments of DCN3D_GEOMETRY / DCN2D_GEOMETRY
N_CONV2D_GEOM = 16          # ... of CONV2D_GEOMETRY


class DcnError(RuntimeError):
    """Raised when libdcn_amd.so rejects a call; the text comes from dcn_last_error()."""


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ImportError(
            "libdcn_amd.so is not built (expected at %s). Build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` from the repository root or "
            "`python -m deform_conv3d_pytorch_op_amd.build`; there is no CPU or PyTorch fallback." % SO_PATH)
    L = ctypes.CDLL(SO_PATH)
    L.dcn_version.restype = _c_int
    L.dcn_arch.restype = ctypes.c_char_p
    L.dcn_last_error.restype = ctypes.c_char_p
    L.dcn_workspace_bytes.restype = _c_sz
    L.dcn_workspace_bytes.argtypes = [_c_int] * 4 + [_c_sz, _c_sz, _c_int, _c_int]
    L.dcn_workspace_bytes_for.restype = _c_sz
    L.dcn_workspace_bytes_for.argtypes = [_c_int] * 4 + [_c_sz, _c_sz, _c_int, _c_int, _c_int]
    tail = [_c_vp, _c_sz, _c_vp]            # workspace, workspace_bytes, stream
    for nd in (2, 3):
        geom = [_c_int] * N_GEOM[nd]
        for suf in ("f32", "f64", "bf16", "f16"):
            f = getattr(L, "dcn%dd_forward_%s" % (nd, suf))
            f.restype, f.argtypes = _c_int, [_c_vp] * 5 + geom + tail
            f = getattr(L, "dcn%dd_backward_input_offset_%s" % (nd, suf))
            f.restype, f.argtypes = _c_int, [_c_vp] * 6 + geom + tail
            f = getattr(L, "dcn%dd_backward_weight_%s" % (nd, suf))
            f.restype, f.argtypes = _c_int, [_c_vp] * 4 + geom + tail
            if nd == 3 and suf in ("f32", "f64"):
                f = getattr(L, "dcn3d_backward_input_offset_flags_%s" % suf)
                f.restype, f.argtypes = _c_int, [_c_vp] * 6 + geom + tail + [ctypes.c_uint]
    L.conv2d_workspace_bytes.restype = _c_sz
    L.conv2d_workspace_bytes.argtypes = [_c_int] * 4 + [_c_sz, _c_sz, _c_int, _c_int]
    cgeom = [_c_int] * N_CONV2D_GEOM
    for suf in ("f32", "f64"):
        f = getattr(L, "conv2d_forward_" + suf)
        f.restype, f.argtypes = _c_int, [_c_vp] * 4 + cgeom + tail
        f = getattr(L, "conv2d_backward_input_" + suf)
        f.restype, f.argtypes = _c_int, [_c_vp] * 3 + cgeom + tail
        f = getattr(L, "conv2d_backward_weight_" + suf)
        f.restype, f.argtypes = _c_int, [_c_vp] * 3 + cgeom + tail
    L.dcn3d_forward_noalloc_f32.restype = _c_int
    L.dcn3d_forward_noalloc_f32.argtypes = [_c_vp] * 5 + [_c_int] * N_GEOM[3] + [_c_vp]
    if L.dcn_version() != 1:
        raise ImportError("libdcn_amd.so has ABI version %d, expected 1" % L.dcn_version())
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise DcnError(load().dcn_last_error().decode())


EXPORTS = ["dcn_version", "dcn_arch", "dcn_last_error", "dcn_workspace_bytes", "dcn_workspace_bytes_for"] + [
    "dcn%dd_%s_%s" % (nd, op, suf)
    for nd in (2, 3) for op in ("forward", "backward_input_offset", "backward_weight")
    for suf in ("f32", "f64", "bf16", "f16")] + [
    "dcn3d_backward_input_offset_flags_f32", "dcn3d_backward_input_offset_flags_f64",
    "dcn3d_forward_noalloc_f32", "conv2d_workspace_bytes"] + [
    "conv2d_%s_%s" % (op, suf) for op in ("forward", "backward_input", "backward_weight") for suf in ("f32", "f64")]
NOALLOC_SCRATCH_BYTES = 8 << 20
FLAG_OOB_OFFSET_GRAD_ZERO = 1
