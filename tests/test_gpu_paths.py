"""Runs the small parity cases again with the library's tuning knobs forced to the corner
settings, each in a process of its own (the knobs are read once per process):

  DCN_HALO_MARGIN=0    almost every sample reaches past the LDS halo -> global fallback paths
  DCN_HALO_MARGIN=50   the halo never fits -> kernels that do not use LDS tiling at all
  DCN_SCATTER=global   grad-input through global atomics on the channels-last copy
  DCN_LDS_BUDGET_KB / DCN_SCATTER_BUDGET_KB small -> smallest channel chunks
  DCN_FORWARD_WG=1024  the 1024-thread forward variant also where the grid would be too small for it
  DCN_FORWARD_WG=512   ... and never
  DCN_COORD=separate   grad_offset from the channels-last kernel, grad_input from the scatter-only kernel
  DCN_CSPLIT=1 / 4     channel chunks of the fused backward kernel on one / four workgroups
  DCN_FUSED_WAVES=4    the fused backward kernel's four-wavefront shape (otherwise only strided full-size cases use it)
  DCN_FUSED_CHUNK=4    the fused backward kernel with 4-channel chunks also for 2-D layers (which otherwise take 16, or 8
                       where a deformable group has fewer than 16 channels); =8: 8-channel chunks where it would take 16
  DCN_FUSED_SLOTS=3    plans the fused backward launch for a device of three workgroups: unsplit items first, the
                       items of the last round split over several workgroups (otherwise only full-size layers get there)
  DCN_FUSED_TAIL=0     ... and the same without that split; DCN_FUSED_FIXED=0: runtime plane stride
  DCN_OVERLAP_BACKWARD=1  backward_weight on a second stream next to backward_input_offset
  DCN_FUSED_BREG2=0    the grad_output operand of 64 < M <= 128 output channels read from memory instead of a second register set
  DCN_FUSED_PAIR=0     float32 LDS cells of the fused backward kernel with one channel each (64-bit) instead of two
  DCN_FORWARD_SLOTS=3  plans the forward launch for a device of three workgroups: the units of the last, partly filled
                       round are split over workgroups whose partial sums a second kernel joins (otherwise only
                       full-size layers get there), all the same number of ways or, where that fills the rounds
                       better, some of them one way more (DCN_FORWARD_TAIL2=0: never); DCN_FORWARD_TAIL=2 forces a
                       two-way split, =0 none
  DCN_ADAPTIVE_MARGIN=0  one halo margin of 2 instead of the choice on the device among 2, 3, 4 (2, 4, 6 in 2-D): the
                       cases with wide offsets then take the paths through global memory (the default runs cover the
                       wider plans and the choice)
  DCN_FORWARD_SPLIT=0  the forward pass never splits the input channels of a position block over workgroups
                       (small layers otherwise do, so the default runs cover the split and its joining kernel)
"""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SETTINGS = [
    {"DCN_HALO_MARGIN": "0"},
    {"DCN_HALO_MARGIN": "50"},
    {"DCN_SCATTER": "global"},
    {"DCN_LDS_BUDGET_KB": "16", "DCN_SCATTER_BUDGET_KB": "72"},
    {"DCN_FORWARD_WG": "1024", "DCN_CSPLIT": "4"},
    {"DCN_FORWARD_WG": "512", "DCN_CSPLIT": "1"},
    {"DCN_COORD": "separate"},
    {"DCN_FUSED_WAVES": "4"},
    {"DCN_FUSED_CHUNK": "4"},
    {"DCN_FUSED_CHUNK": "8"},
    {"DCN_FUSED_SLOTS": "3"},
    {"DCN_FUSED_SLOTS": "3", "DCN_FUSED_TAIL": "0", "DCN_FUSED_FIXED": "0"},
    {"DCN_OVERLAP_BACKWARD": "1", "DCN_FORWARD_SPLIT": "0"},
    {"DCN_FUSED_PAIR": "0", "DCN_FUSED_BREG2": "0"},
    # the forward pass planned for a device of three workgroups: units of the last round split over several workgroups
    {"DCN_FORWARD_SLOTS": "3"},
    {"DCN_FORWARD_SLOTS": "7", "DCN_FORWARD_SPLIT": "0"},
    {"DCN_FORWARD_SLOTS": "3", "DCN_FORWARD_TAIL2": "0"},
    {"DCN_FORWARD_SLOTS": "5", "DCN_FORWARD_TAIL": "2", "DCN_FORWARD_SPLIT": "0"},
    {"DCN_FORWARD_TAIL": "0"},
    # one halo margin, as narrow as the default: the wide offsets of the cases then leave the halo
    # and take the paths through global memory, which the margin chosen on the device avoids
    {"DCN_ADAPTIVE_MARGIN": "0"},
    {"DCN_ADAPTIVE_MARGIN": "0", "DCN_FUSED_PAIR": "0", "DCN_FUSED_FIXED": "0"},
    {"DCN_ADAPTIVE_MARGIN": "0", "DCN_FUSED_WAVES": "4", "DCN_FORWARD_WG": "512"},
]
# the 16-bit forward through the float32 kernels: by request, and because the halo kernel declines the layer
MIXED_SETTINGS = [{"DCN_NATIVE16": "0"}, {"DCN_HALO_MARGIN": "50"}, {"DCN_ADAPTIVE_MARGIN": "0"},
                  # (the split last round of the 16-bit forward: float partial sums, rounded once when they are joined)
                  {"DCN_FORWARD_SLOTS": "3"}, {"DCN_FORWARD_SLOTS": "7"}, {"DCN_FORWARD_SLOTS": "5", "DCN_FORWARD_TAIL": "2"}]


@pytest.mark.parametrize("extra", MIXED_SETTINGS, ids=lambda e: ",".join("%s=%s" % kv for kv in e.items()))
def test_16bit_cases_under_knob(extra):
    print("knobs", extra, flush=True)
    env = dict(os.environ)
    env.update(extra)
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.join(ROOT, "tests", "test_gpu_mixed.py"), "-q", "-x",
                        "-m", "gpu", "--timeout", "120", "--timeout-method", "thread"],
                       cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]


@pytest.mark.parametrize("extra", SETTINGS, ids=lambda e: ",".join("%s=%s" % kv for kv in e.items()))
def test_small_cases_under_knob(extra):
    print("knobs", extra, flush=True)
    env = dict(os.environ)
    env.update(extra)
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.join(ROOT, "tests", "test_gpu_parity.py"), "-q", "-x",
                        "-m", "gpu", "-k", "small_cases or golden or non_finite or heavy_tailed or oob_offset_grad or random_geometries or random_medium", "--timeout", "120", "--timeout-method", "thread"],
                       cwd=ROOT, env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]


_TWO_RUNS_CASE = r"""
import sys, torch
sys.path.insert(0, %r)
from tests.cases import make_case
from oracle import dcn_oracle as orc
import deform_conv3d_pytorch_op_amd as dcn
for dtype, tol in ((torch.float32, 1e-4), (torch.float64, 1e-10)):
    c = make_case(2, 4, 32, 8, 64, 3, 1, 1, 1, 4, 1, 1.0, dtype=dtype, seed=11, bias=True)
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    want = orc.forward(c["x"], c["off"], c["w"], c["b"], *cfg)
    got = dcn.ConvOffset2dFunction.apply(c["x"].cuda(), c["off"].cuda(), c["w"].cuda(), c["b"].cuda(), *cfg)
    err = ((got.cpu().double() - want.double()).abs().max() / want.double().abs().max()).item()
    assert err <= tol, (dtype, err)
print("two-runs case ok")
"""


def test_forward_last_round_split_in_two_runs():
    """The units of the forward pass's last round split 3 ways and 4 ways side by side (so that the
    short rounds they make are full): eight deformable groups give a unit eight channel passes, and
    one of the planned device sizes leaves a last round that the two-run split fills better than a
    uniform one.  Every planned size must give the oracle's output; at least one must take two runs."""
    hits = 0
    for slots in ("14", "25", "41", "33"):
        print("DCN_FORWARD_SLOTS", slots, flush=True)
        env = dict(os.environ)
        env.update({"DCN_FORWARD_SLOTS": slots, "DCN_FORWARD_SPLIT": "0", "DCN_TRACE_PLANS": "1"})
        r = subprocess.run([sys.executable, "-u", "-c", _TWO_RUNS_CASE % ROOT], cwd=ROOT, env=env, stdout=subprocess.PIPE,
                           stderr=subprocess.PIPE, text=True, timeout=300)
        assert r.returncode == 0, (r.stdout[-1000:], r.stderr[-3000:])
        hits += "of the rest:" in r.stderr
    assert hits >= 1, "no planned device size took the two-run split"
