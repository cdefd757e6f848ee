#!/usr/bin/env python3
"""Benchmark of the backward pass + SGD-momentum update on one MI355X.

Workload (the configuration the headline metric is quoted on): ResNet-18, N=64, 3x224x224, fp32,
BatchNorm in training mode, 1000-class softmax cross-entropy, SGD momentum 0.9 -- the graph of the
reference's examples/cnn/model/resnet.py.  One "step" = loss-gradient seed -> last parameter
updated (every backward kernel in tape order plus the update of all 62 parameter tensors), on
synthetic seeded inputs whose forward activations are already resident in HBM.

Prints ONE JSON line: the whole-job images/s plus
  roofline     -- the dominant kernel family (fp32 MFMA conv dgrad + wgrad kernels):
                  algorithmic FLOPs / measured kernel time (HIP events on the kernels' stream),
                  against the MI355X fp32 matrix peak;
  cpu_baseline -- the CPU oracle replaying the same tape on the host cores, on a bounded sample.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_16BIT_MFMA_TFLOPS = 2500.0   # dense fp16 / bf16 matrix peak
PEAK_HBM_GBS = 8000.0
# HBM bytes the 40 conv dgrad/wgrad MFMA launches of one default step move (fetched + written), from the
# rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this script, each scaled by what the same counter reads for
# a streaming kernel of known size (ReLU forward: 1.998 and 1.000).  Valid for the default workload only.
CONV_HBM_BYTES_PER_STEP = 6.71e9


def collect_prof(lib):
    n = C.c_int()
    lib.sgh_prof_count(C.byref(n))
    out = {}
    buf = C.create_string_buffer(32)
    for i in range(n.value):
        ms, work = C.c_float(), C.c_double()
        rc = lib.sgh_prof_get(i, buf, 32, C.byref(ms), C.byref(work))
        if rc != 0:
            raise RuntimeError("sgh_prof_get rc=%d" % rc)
        d = out.setdefault(buf.value.decode(), {"launches": 0, "ms": 0.0, "flop": 0.0})
        d["launches"] += 1
        d["ms"] += ms.value
        d["flop"] += work.value
    return out


def cpu_baseline(config, sample_batch, budget_s):
    """The CPU oracle (a restatement of SINGA's CppCPU algorithms) replaying the same tape on the
    host cores: whole steps at `sample_batch` until about `budget_s` seconds have been spent."""
    from oracle import cpu_oracle as O
    from oracle.ops import OracleOps
    from singa_amd import workloads as wl
    ops = OracleOps()
    net = wl.build(config, ops)
    x, labels = wl.make_inputs(config, sample_batch)
    net.forward(ops.from_numpy(x), ops.from_numpy(labels))
    steps, t0 = 0, time.perf_counter()
    while True:
        net.backward_and_update()
        steps += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or steps >= 50:
            break
    return {"value": round(sample_batch * steps / dt, 3), "unit": "imgs/s", "cores": O.get_threads(), "kind": "port",
            "sample": "%d %s backward+update step(s) at batch %d on the same seeded inputs, %.1f s of CPU time "
                      "(OpenMP over the SGEMM rows / channels; the per-image loop is serial like the reference's)"
                      % (steps, config, sample_batch, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--config", default="resnet18")
    ap.add_argument("--cpu-sample-batch", type=int, default=32)
    ap.add_argument("--cpu-budget-s", type=float, default=10.0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--storage", default="f32", choices=["f32", "f16", "bf16"],
                    help="f16 / bf16: the mixed-precision tape (16-bit activations, gradients and conv weights, "
                         "fp32 BatchNorm statistics and master weights), e.g. --config resnet50 --batch 128")
    ap.add_argument("--graph", action="store_true",
                    help="record one step and replay it (graph mode, Device::EnableGraph / RunGraph) instead of "
                         "enqueueing every launch of every step from the host; the step is GPU-bound, so this "
                         "frees the host (0.94 -> 0.09 ms/step) without changing the throughput")
    ap.add_argument("--no-fusion", action="store_true",
                    help="one call per op of the reference's tape (no ReLU+BatchNorm backward fusion, residual += as its own kernel)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="every kernel on the one device stream (weight gradients otherwise run on a second stream); "
                         "the setting for kernel traces whose durations should be those of kernels running alone")
    ap.add_argument("--per-parameter-update", action="store_true",
                    help="update each parameter right after its gradient (one launch each) instead of one fused launch")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch  # device synchronisation only; no torch op is on the measured path
    from singa_amd import _lib
    from singa_amd import singa_wrap as singa
    from singa_amd import workloads as wl

    lib = _lib.lib()
    dev = singa.create_hip_gpu_on(0)
    half = args.storage != "f32"
    hip = wl.HalfHipOps(dev, singa.kFloat16 if args.storage == "f16" else singa.kBFloat16) if half else wl.HipOps(dev)
    hip.set_fusion(not args.no_fusion)
    if args.no_overlap:
        hip.overlap_wgrad = False
    net = wl.build(args.config, hip, lr=0.05, momentum=0.9)
    x, labels = wl.make_inputs(args.config, args.batch)
    net.forward(hip.from_numpy(x), hip.from_numpy(labels))
    fused = not args.per_parameter_update

    def sync():
        dev.Sync()
        torch.cuda.synchronize()

    graph = args.graph
    if graph:
        # graph mode as the reference runs a compiled model (python/singa/model.py:70-90): the first
        # iterations run eagerly, one is recorded, every later one replays the recording
        for _ in range(2):
            net.backward_and_update(fused_update=fused)
        sync()
        dev.EnableGraph(True)
        net.backward_and_update(fused_update=fused)
        dev.EnableGraph(False)
        step = dev.RunGraph
    else:
        def step():
            net.backward_and_update(fused_update=fused)
    for _ in range(args.warmup):
        step()
    sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    t_enqueued = time.perf_counter() - t0   # host time to enqueue every launch of the timed steps
    sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    imgs_per_s = args.batch * args.steps / elapsed

    if graph:
        dev.ResetGraph()
    # kernel-level pass (eager): every conv / GEMM launch bracketed by HIP events on the device stream
    prof_steps = max(1, min(args.steps, 5))
    hip.overlap_wgrad = False   # one kernel at a time on the device, so that an event pair brackets that kernel alone
    lib.sgh_prof_enable(1)
    for _ in range(prof_steps):
        net.backward_and_update(fused_update=fused)
    sync()
    prof = collect_prof(lib)
    lib.sgh_prof_enable(0)
    conv = {k: prof[k] for k in ("conv_dgrad", "conv_wgrad", "conv_dgrad16", "conv_wgrad16") if k in prof}
    flop = sum(v["flop"] for v in conv.values())
    ms = sum(v["ms"] for v in conv.values())
    launches = sum(v["launches"] for v in conv.values())
    achieved = flop / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
    peak = PEAK_16BIT_MFMA_TFLOPS if half else PEAK_FP32_MFMA_TFLOPS
    roofline = {
        "bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
        "frac": round(achieved / peak, 4),
        "traffic": CONV_HBM_BYTES_PER_STEP if (args.config == "resnet18" and args.batch == 64 and not half
                                               and not args.no_fusion) else None,
        "traffic_unit": "HBM bytes per step over the same launches (PMC, calibrated)",
        "kernel": ("16-bit MFMA conv dgrad + wgrad kernels (k_dgrad16, k_wgrad16; fp32 kernels for the stem dgrad; %d launches/step)"
                   if half else
                   "fp32 MFMA conv dgrad + wgrad kernels (k_dgrad3x3, k_wgrad3x3, k_dgrad_fewc, k_wgrad_fewc, k_igemm; %d launches/step)")
                  % (launches // prof_steps),
        "flop_per_step": flop / prof_steps, "kernel_ms_per_step": round(ms / prof_steps, 4),
        "timing": "HIP event pair around every launch in %d extra steps with all kernels on one stream "
                  "(the timed steps run the weight gradients on a second stream)" % prof_steps,
    }
    for k, v in conv.items():
        roofline[k + "_tflops"] = round(v["flop"] / (v["ms"] * 1e-3) / 1e12, 3) if v["ms"] > 0 else 0.0
    # whole entry points (weight re-layout, split-K reduction and column gather kernels included)
    ops_ms = sum(prof[k]["ms"] for k in ("conv_dgrad_op", "conv_wgrad_op") if k in prof)
    roofline["entry_points_ms_per_step"] = round(ops_ms / prof_steps, 4)

    out = {
        "metric": "backward+update imgs/sec, ResNet-18 N=64 fp32" if (args.config == "resnet18" and not half and args.batch == 64)
                  else "backward+update imgs/sec, %s N=%d %s" % (args.config, args.batch, args.storage),
        "value": round(imgs_per_s, 2), "unit": "imgs/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.storage, "data": "synthetic",
        "config": {"workload": "%s backward+update, N=%d, 3x224x224, %s, SGD momentum 0.9" % (
                       args.config, args.batch, "fp32" if not half else args.storage + " storage / fp32 accumulate, statistics and master weights"),
                   "update": "fused multi-tensor" if fused else "per parameter",
                   "launch": "one recorded step replayed (graph mode)" if graph else "eager, one launch per kernel",
                   "tape": "ReLU backward folded into BatchNorm backward (conv-BN-ReLU), residual += folded into the "
                           + ("data gradient" if hip.fuse_dgrad_add else "ReLU backward that reads the sum")
                           + ", weight re-layouts in one launch"
                           + (", weight gradients on a second stream" if not (args.no_overlap or graph) else "")
                           if hip.fuse_bn_relu
                           else "one call per reference op"},
        "roofline": roofline,
        "host_enqueue_ms_per_step": round(t_enqueued / args.steps * 1e3, 4),
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.config, args.cpu_sample_batch, args.cpu_budget_s)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
