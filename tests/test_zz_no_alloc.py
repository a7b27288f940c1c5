"""The allocation-free forward entry point (dcn3d_forward_noalloc_f32) against dcn3d_forward_f32,
both called through the C ABI with ctypes: two calls in a row, the second on a smaller layer, so
that the fixed scratch array inside the library still holds the first call's weights when the
second starts.  Both entry points run the same kernels, so the outputs must agree to the float32
forward tolerance (1e-4 relative; in practice bit for bit).  Oversized layers must be rejected.
"""
import pytest
import torch

from deform_conv3d_pytorch_op_amd import _lib
from deform_conv3d_pytorch_op_amd.functions import _geom, _workspace
from tests.cases import make_case

pytestmark = pytest.mark.gpu

#        N, Cin, Cout, in, k, stride, pad, dil, cpg, groups, off_scale
FIRST = (2, 24, 40, (6, 12, 12), 3, 1, 1, 1, 12, 1, 2.0)
SECOND = (1, 6, 5, (4, 7, 5), (2, 3, 1), (1, 2, 1), (1, 2, 0), 1, 2, 1, 2.0)     # smaller: fewer weights, other geometry


def _both(L, spec, seed, poison):
    dev = torch.device("cuda:0")
    c = make_case(3, *spec, dtype=torch.float32, seed=seed)
    x, off, w, b = (c[k].to(dev) for k in ("x", "off", "w", "b"))
    geom = _geom(3, x, w, c["outs"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    shape = (x.size(0), w.size(0)) + c["outs"]
    want = torch.full(shape, poison, dtype=torch.float32, device=dev)
    got = torch.full(shape, poison, dtype=torch.float32, device=dev)
    ws, ws_bytes = _workspace(x, w, c["groups"], c["outs"], c["cpg"])
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(L.dcn3d_forward_f32(x.data_ptr(), w.data_ptr(), off.data_ptr(), b.data_ptr(), want.data_ptr(), *geom,
                                   ws.data_ptr(), ws_bytes, stream))
    # a first call resolves the scratch array's device address (once per device); the call that is
    # checked for allocations comes after it
    _lib.check(L.dcn3d_forward_noalloc_f32(x.data_ptr(), w.data_ptr(), off.data_ptr(), b.data_ptr(), got.data_ptr(),
                                           *geom, stream))
    torch.cuda.synchronize()
    got.fill_(poison)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    free_before = torch.cuda.mem_get_info(dev)[0]       # the driver's free bytes: sees allocations made behind torch's back
    _lib.check(L.dcn3d_forward_noalloc_f32(x.data_ptr(), w.data_ptr(), off.data_ptr(), b.data_ptr(), got.data_ptr(),
                                           *geom, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    return got, want


def test_noalloc_forward_matches_forward_twice_in_a_row():
    L = _lib.load()
    for spec, seed in ((FIRST, 11), (SECOND, 12)):
        print("no-alloc forward", spec, flush=True)
        got, want = _both(L, spec, seed, poison=7.0)
        scale = want.abs().max().item()
        assert scale > 0
        err = (got - want).abs().max().item() / scale
        assert err <= 1e-4, "relative error %.3e" % err


def test_noalloc_forward_rejects_a_layer_beyond_the_scratch():
    L = _lib.load()
    dev = torch.device("cuda:0")
    # 3x3x3 taps * 512 output channels * (512 + 4) channels * 4 bytes = 28.5 MB of re-laid-out weight > 8 MiB
    x = torch.zeros(1, 512, 2, 4, 4, device=dev)
    w = torch.zeros(512, 512, 3, 3, 3, device=dev)
    off = torch.zeros(1, 81, 2, 4, 4, device=dev)
    out = torch.zeros(1, 512, 2, 4, 4, device=dev)
    geom = _geom(3, x, w, (2, 4, 4), (1, 1, 1), (1, 1, 1), (1, 1, 1), 512, 1)
    rc = L.dcn3d_forward_noalloc_f32(x.data_ptr(), w.data_ptr(), off.data_ptr(), None, out.data_ptr(), *geom,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == -2
    assert "allocation-free" in L.dcn_last_error().decode()
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0
