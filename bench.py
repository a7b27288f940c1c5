"""Benchmark of the deformable-convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1..c5|all] [--no-cpu] [--dtype f32|f64|bf16|f16]

A step is one forward + backward (grad input, grad offset, grad weight) of one layer through the
package's autograd Function on synthetic inputs already resident in HBM.  The default workload is
BASELINE.json's headline configuration c4: deform3d float32, N=4, 64->64 channels, 16x56x56,
kernel 3x3x3, stride 1, pad 1, one deformable group, offsets U[-1.5, 1.5].

Prints one JSON line (`--config all`: one line per configuration, c1 to c5).  `value` is effective
TFLOP/s = 3 * 2*N*C_out*(C_in/G)*kV*outV / step time (only the three dense contractions are counted
as work).  `roofline` describes the slowest kernel
of the step, timed on its own with HIP events on the stream it is launched on; `cpu_baseline` is
the CPU oracle (the reference algorithm restated: im2col + GEMM per sample and group) timed on a
bounded sample of the same workload on the host cores.
"""
import argparse
import ctypes
import hashlib
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"float32": 157.3, "float64": 78.6, "bfloat16": 2500.0, "float16": 2500.0}     # MI355X dense matrix peaks
DTYPES = {"f32": "float32", "f64": "float64", "bf16": "bfloat16", "f16": "float16"}
PEAK_HBM_GBS = 8000.0

# HBM bytes per C-ABI call measured with rocprofv3 (--pmc FETCH_SIZE, then --pmc WRITE_SIZE, each scaled by
# what the same counter reads for a plain 256 MiB device copy in the same run).  The figures live in a data
# file that is rewritten whenever the kernels are profiled again: {"c4": {"forward": bytes, ...}, ...} plus the
# SHA-256 of the kernel sources they were measured on.  `traffic` is null for a configuration or call that
# was not profiled, and for every call once the kernel sources differ from the profiled ones.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
CSRC = os.path.join(ROOT, "deform_conv3d_pytorch_op_amd", "csrc")


def csrc_sha256():
    h = hashlib.sha256()
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".h", ".hip")):
            with open(os.path.join(CSRC, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def measured_traffic(config, call):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
        if table.get("_csrc_sha256") != csrc_sha256():
            return None
        v = table.get(config, {}).get(call)
        return float(v) if v is not None else None
    except (OSError, ValueError):
        return None


# name: (nd, N, C_in, C_out, in, k, stride, pad, dil, cpg, groups, offset scale / dist, dtype)
CONFIGS = {
    "c1": (2, 2, 8, 8, 16, 3, 1, 1, 1, 8, 1, 1.5, "float64"),
    "c2": (2, 8, 256, 256, 56, 3, 1, 1, 1, 256, 1, 2.0, "float32"),
    "c3": (2, 4, 512, 512, 28, 3, 1, 2, 2, 128, 2, "normal_mix", "float32"),
    "c4": (3, 4, 64, 64, (16, 56, 56), 3, 1, 1, 1, 64, 1, 1.5, "float32"),
    "c5": (3, 2, 128, 128, (16, 112, 112), 3, (1, 2, 2), 1, 1, 32, 1, 2.0, "float32"),
}
DESCR = {
    "c1": "deform2d f64 N=2 8->8 16x16 k3 p1 (gradcheck shape)",
    "c2": "deform2d f32 N=8 256->256 56x56 k3 p1",
    "c3": "deform2d f32 N=4 512->512 28x28 k3 p2 d2 groups2 dg4",
    "c4": "deform3d f32 N=4 64->64 16x56x56 k3 s1 p1 dg1 offsets U[-1.5,1.5]",
    "c5": "deform3d f32 N=2 128->128 16x112x112 k3 s(1,2,2) p1 dg4",
}


def gemm_flops(c):
    N, C_out = c["x"].shape[0], c["w"].shape[0]
    return 2.0 * N * C_out * c["w"].shape[1] * math.prod(c["k"]) * math.prod(c["outs"])


def algorithmic_bytes(c):
    """Compulsory traffic: every distinct tensor read once, every result written once."""
    es = c["x"].element_size()
    nb = lambda t: t.numel() * es
    out_b = c["gout"].numel() * es
    fwd = nb(c["x"]) + nb(c["off"]) + nb(c["w"]) + out_b
    data = out_b + nb(c["x"]) + nb(c["off"]) + nb(c["w"]) + nb(c["x"]) + nb(c["off"])   # + grad_input, grad_offset
    wgt = out_b + nb(c["x"]) + nb(c["off"]) + nb(c["w"])                                # + grad_weight
    return dict(forward=fwd, backward_input_offset=data, backward_weight=wgt)


def run_config(name, a):
    import torch
    import deform_conv3d_pytorch_op_amd as dcn
    from deform_conv3d_pytorch_op_amd import _lib
    from deform_conv3d_pytorch_op_amd.functions import _geom
    from deform_conv3d_pytorch_op_amd.synthetic import make_case

    spec = CONFIGS[name]
    if a.dtype is not None:             # the configuration's shapes in the other precision
        spec = spec[:-1] + (DTYPES[a.dtype],)
    dtype = getattr(torch, spec[-1])
    kw = dict(dtype=dtype, seed=0, bias=False)
    if a.offset_scale is not None:      # not the configuration's own offsets: U[-s, s]
        c = make_case(*spec[:-2], a.offset_scale, **kw)
    elif spec[-2] == "normal_mix":
        c = make_case(*spec[:-2], 1.0, off_dist="normal_mix", **kw)
    else:
        c = make_case(*spec[:-1], **kw)
    nd = c["nd"]
    dev = torch.device("cuda:0")
    fn = dcn.ConvOffset3dFunction if nd == 3 else dcn.ConvOffset2dFunction
    x, off, w = (c[k].to(dev).requires_grad_(True) for k in ("x", "off", "w"))
    gout = c["gout"].to(dev)
    cfg = (c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])

    def step():
        x.grad = off.grad = w.grad = None
        out = fn.apply(x, off, w, None, *cfg)
        out.backward(gout)

    def fwd_only():
        with torch.no_grad():
            fn.apply(x, off, w, None, *cfg)

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) * 1e3 / a.steps

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        fwd_only()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) * 1e3 / a.steps

    # the same two quantities step by step between HIP events (median and minimum), outside the timed region above
    def event_times(fn_):
        evs = []
        for _ in range(a.steps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn_()
            e1.record()
            evs.append((e0, e1))
        torch.cuda.synchronize()
        ts = sorted(e0.elapsed_time(e1) for e0, e1 in evs)
        return {"median": round(ts[len(ts) // 2], 4), "min": round(ts[0], 4)}
    step_events, fwd_events = event_times(step), event_times(fwd_only)

    F = gemm_flops(c)
    value = 3 * F / (ms_step * 1e-3) / 1e12

    # ---- per-kernel durations: each C-ABI call between two HIP events on its own stream ------
    L = _lib.load()
    suf = {v: k for k, v in DTYPES.items()}[spec[-1]]
    geom = _geom(nd, x, w, c["outs"], c["stride"], c["pad"], c["dil"], c["cpg"], c["groups"])
    nbytes = L.dcn_workspace_bytes_for(x.element_size(), x.shape[0], x.shape[1], w.shape[0], math.prod(c["ins"]),
                                       math.prod(c["outs"]), math.prod(c["k"]), c["groups"], c["cpg"])
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    out = torch.empty((x.shape[0], w.shape[0]) + c["outs"], dtype=dtype, device=dev)
    gin, goff, gw = torch.zeros_like(x), torch.empty_like(off), torch.zeros_like(w)
    stream = torch.cuda.current_stream()
    sp = stream.cuda_stream
    xd, od, wd = x.detach(), off.detach(), w.detach()
    calls = {
        "forward": lambda: getattr(L, "dcn%dd_forward_%s" % (nd, suf))(
            xd.data_ptr(), wd.data_ptr(), od.data_ptr(), None, out.data_ptr(), *geom, ws.data_ptr(), nbytes, sp),
        "backward_input_offset": lambda: getattr(L, "dcn%dd_backward_input_offset_%s" % (nd, suf))(
            xd.data_ptr(), wd.data_ptr(), od.data_ptr(), gout.data_ptr(), gin.data_ptr(), goff.data_ptr(), *geom,
            ws.data_ptr(), nbytes, sp),
        "backward_weight": lambda: getattr(L, "dcn%dd_backward_weight_%s" % (nd, suf))(
            xd.data_ptr(), od.data_ptr(), gout.data_ptr(), gw.data_ptr(), *geom, ws.data_ptr(), nbytes, sp),
    }
    kernel_ms = {}
    for cname, call in calls.items():
        for _ in range(2):
            assert call() == 0, L.dcn_last_error()
        evs = []
        for _ in range(a.steps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            assert call() == 0, L.dcn_last_error()
            e1.record(stream)
            evs.append((e0, e1))
        torch.cuda.synchronize()
        kernel_ms[cname] = sum(e0.elapsed_time(e1) for e0, e1 in evs) / len(evs)
    dominant = max(kernel_ms, key=kernel_ms.get)
    ab = algorithmic_bytes(c)
    peak = PEAK_TFLOPS[spec[-1]]
    achieved = F / (kernel_ms[dominant] * 1e-3) / 1e12
    roofline = {"kernel": dominant, "bound": "mfma", "achieved": round(achieved, 3), "peak": peak,
                "unit": "TFLOP/s", "frac": round(achieved / peak, 4),
                "traffic": measured_traffic(name, dominant) if a.offset_scale is None and a.dtype is None else None,
                "ms": round(kernel_ms[dominant], 4),
                "algorithmic_flops": F, "algorithmic_bytes": ab[dominant],
                "hbm_frac_at_algorithmic_bytes": round(ab[dominant] / (kernel_ms[dominant] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)}
    kernels = {k: {"ms": round(v, 4), "tflops": round(F / (v * 1e-3) / 1e12, 3),
                   "mfma_frac": round(F / (v * 1e-3) / 1e12 / peak, 4),
                   "algorithmic_GBps": round(ab[k] / (v * 1e-3) / 1e9, 1)} for k, v in kernel_ms.items()}

    if a.calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)                      # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()

    # ---- CPU baseline: the oracle on a bounded sample of the same workload --------------------
    cpu = None
    if not a.no_cpu and a.dtype not in ("bf16", "f16"):      # (the oracle computes in float32 / float64)
        from oracle import dcn_oracle as orc
        ns = x.shape[0]
        xs, offs, gs = c["x"][:ns].contiguous(), c["off"][:ns].contiguous(), c["gout"][:ns].contiguous()
        def once():
            t0 = time.perf_counter()
            orc.forward(xs, offs, c["w"], None, *cfg, acc64=False)
            orc.backward(xs, offs, c["w"], gs, None, *cfg, acc64=False)
            return time.perf_counter() - t0
        def once_blas():                       # the same loop with the host BLAS (torch.mm) for the three GEMMs
            t0 = time.perf_counter()
            orc.step_blas(xs, offs, c["w"], gs, *cfg)
            return time.perf_counter() - t0
        threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
        results = {}
        for label, fn_ in (("loops", once), ("blas", once_blas)):
            first = fn_()                      # also warms the thread pool; not counted
            reps = max(3, min(25, int(6.0 / max(first, 1e-3))))       # about 6 s of host work per variant and configuration
            times = sorted(fn_() for _ in range(reps))
            results[label] = (times[len(times) // 2], reps)
        best = min(results, key=lambda k: results[k][0])
        dt, reps = results[best]
        cpu = {"value": round(3 * F * ns / x.shape[0] / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
               "kind": "port", "seconds": round(dt, 2),
               "gemm": "host BLAS through torch.mm" if best == "blas" else "plain OpenMP loops of the oracle",
               "variants_seconds": {k: round(v[0], 3) for k, v in results.items()},
               "sample": "%d of %d samples of %s, forward + backward, median of %d runs, float accumulate; the faster of "
                         "the oracle's own OpenMP GEMM loops and the same per-sample loop with torch.mm for the GEMMs" %
                         (ns, x.shape[0], name, reps)}

    return {
        "metric": "deform conv fwd+bwd effective TFLOP/s per layer (3 dense contractions counted)",
        "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_step, 4), "fwd_ms": round(ms_fwd, 4),
        "ms_per_step_events": step_events, "fwd_ms_events": fwd_events, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": suf, "data": "synthetic",
        "config": {"workload": name + ": " + DESCR[name] +
                               ("" if a.dtype is None else " -- %s instead of its own precision" %
                                ("stored as %s, float32 accumulation," % a.dtype if a.dtype in ("bf16", "f16") else "computed in %s" % a.dtype)) +
                               ("" if a.offset_scale is None else " -- with offsets U[-%g,%g] instead of its own" % (a.offset_scale, a.offset_scale))},
        "mfma_frac_whole_step": round(value / peak, 4),
        "roofline": roofline, "kernels": kernels, "cpu_baseline": cpu,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", default="c4", choices=sorted(CONFIGS) + ["all"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--offset-scale", type=float, default=None,
                    help="offsets uniform in [-s, s] instead of the configuration's own (how the rates depend on the reach of the offsets)")
    ap.add_argument("--dtype", choices=sorted(DTYPES), default=None,
                    help="run the configuration's shapes in this precision instead of its own (f64: against the fp64 matrix "
                         "peak; bf16 / f16: tensors stored in 16 bits, float32 accumulation, against the 16-bit matrix peak)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a kernel of known traffic for scaling rocprof's "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    for name in (sorted(CONFIGS) if a.config == "all" else [a.config]):
        print(json.dumps(run_config(name, a)), flush=True)


if __name__ == "__main__":
    main()
