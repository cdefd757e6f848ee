#!/usr/bin/env python3
"""Benchmark of the backward pass + SGD-momentum update on one MI355X.

Workload (the configuration the headline metric is quoted on): ResNet-18, N=64, 3x224x224, fp32,
BatchNorm in training mode, 1000-class softmax cross-entropy, SGD momentum 0.9 -- the graph of the
reference's examples/cnn/model/resnet.py.  One "step" = loss-gradient seed -> last parameter
updated (every backward kernel in tape order plus the update of all 62 parameter tensors), on
synthetic seeded inputs whose forward activations are already resident in HBM.

Prints ONE JSON line: the whole-job images/s (mean over the timed steps; median and minimum of the
per-step HIP event times as extra keys) plus
  roofline     -- the dominant kernel family (fp32 MFMA conv dgrad + wgrad kernels):
                  algorithmic FLOPs / measured kernel time (HIP events on the kernels' stream),
                  against the MI355X fp32 matrix peak; `traffic` = HBM bytes per step of the same
                  launches, read from the rocprofv3 counter summary under profiles/ when that
                  summary was taken on the kernels this run launched (null otherwise);
  hbm_kernels  -- the bandwidth-bound kernel families: algorithmic bytes / measured time against
                  the HBM3E peak;
  cpu_baseline -- the CPU oracle replaying the same tape on the host cores, on a bounded sample
                  (all host threads at the benchmark's batch, and one thread on a few images).
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
# HBM bytes the conv dgrad/wgrad MFMA launches of one step move (fetched + written) come from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE), summarised in this file together with the
# workload and the kernels the figure covers; it is quoted only for a run that launched exactly those kernels.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "conv_grad_kernels_hbm_traffic_pmc.txt")


def collect_prof(lib):
    """{class: {"launches", "ms", "work", "kernels": set}} from the library's per-launch event pairs;
    a record's tag is "class" or "class/kernel"."""
    n = C.c_int()
    lib.sgh_prof_count(C.byref(n))
    out = {}
    buf = C.create_string_buffer(64)
    for i in range(n.value):
        ms, work = C.c_float(), C.c_double()
        rc = lib.sgh_prof_get(i, buf, 64, C.byref(ms), C.byref(work))
        if rc != 0:
            raise RuntimeError("sgh_prof_get rc=%d" % rc)
        cls, _, kern = buf.value.decode().partition("/")
        d = out.setdefault(cls, {"launches": 0, "ms": 0.0, "work": 0.0, "kernels": set()})
        d["launches"] += 1
        d["ms"] += ms.value
        d["work"] += work.value
        if kern:
            d["kernels"].add(kern)
    return out


def traffic_from_profile(workload, kernels):
    """HBM bytes per step from the committed counter summary, or None when the summary is missing, was
    taken on another workload, or covers a different set of kernels than this run launched."""
    try:
        fields = {}
        for line in open(TRAFFIC_PROFILE):
            if line.startswith("#@ "):
                k, _, v = line[3:].partition(":")
                fields[k.strip()] = v.strip()
        if fields.get("workload") != workload:
            return None
        if set(fields.get("kernels", "").split()) != set(kernels):
            return None
        return float(fields["traffic_bytes_per_step"])
    except (OSError, KeyError, ValueError):
        return None


def cpu_baseline(config, sample_batch, budget_s, single_thread_batch):
    """The CPU oracle (a restatement of SINGA's CppCPU algorithms) replaying the same tape on the
    host cores: whole steps at `sample_batch` until about `budget_s` seconds have been spent, then
    one step on `single_thread_batch` images with one thread (the reference's per-image loop is
    serial, and so is its tensor math without a threaded BLAS)."""
    from oracle import cpu_oracle as O
    from oracle.ops import OracleOps
    from singa_amd import workloads as wl

    def run(batch, budget, max_steps):
        ops = OracleOps()
        net = wl.build(config, ops)
        x, labels = wl.make_inputs(config, batch)
        net.forward(ops.from_numpy(x), ops.from_numpy(labels))
        steps, t0 = 0, time.perf_counter()
        while True:
            net.backward_and_update()
            steps += 1
            dt = time.perf_counter() - t0
            if dt >= budget or steps >= max_steps:
                return steps, dt

    threads = O.get_threads()
    steps, dt = run(sample_batch, budget_s, 50)
    out = {"value": round(sample_batch * steps / dt, 3), "unit": "imgs/s", "cores": threads, "kind": "port",
           "sgemm": "the oracle's own blocked SGEMM loops (no BLAS library in this image)",
           "sample": "%d %s backward+update step(s) at batch %d on the same seeded inputs, %.1f s of CPU time "
                     "(OpenMP over the SGEMM rows / channels; the per-image loop is serial like the reference's)"
                     % (steps, config, sample_batch, dt)}
    if single_thread_batch > 0:
        O.set_threads(1)
        try:
            s1, d1 = run(single_thread_batch, 0.0, 1)
        finally:
            O.set_threads(threads)
        out["single_thread"] = {"value": round(single_thread_batch * s1 / d1, 3), "unit": "imgs/s", "cores": 1,
                                "sample": "1 step at batch %d, %.1f s" % (single_thread_batch, d1)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--config", default="resnet18")
    ap.add_argument("--cpu-sample-batch", type=int, default=0, help="0: the benchmark's batch")
    ap.add_argument("--cpu-budget-s", type=float, default=10.0)
    ap.add_argument("--cpu-single-thread-batch", type=int, default=4, help="images of the one-thread CPU sample (0: skip)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--storage", default="f32", choices=["f32", "f16", "bf16"],
                    help="f16 / bf16: the mixed-precision tape (16-bit activations, gradients and conv weights, "
                         "fp32 BatchNorm statistics and master weights), e.g. --config resnet50 --batch 128")
    ap.add_argument("--graph", action="store_true",
                    help="record one step and replay it (graph mode, Device::EnableGraph / RunGraph) instead of "
                         "enqueueing every launch of every step from the host; the recording holds the weight "
                         "gradients as a branch on the second stream, in groups of layers behind one fork each; it "
                         "frees the host (1.7 -> 0.3 ms/step) and replays a few per cent below the eager two-stream tape")
    ap.add_argument("--no-fusion", action="store_true",
                    help="one call per op of the reference's tape (no ReLU+BatchNorm backward fusion, residual += as its own kernel)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="every kernel on the one device stream (weight gradients otherwise run on a second stream); "
                         "the setting for kernel traces whose durations should be those of kernels running alone")
    ap.add_argument("--with-forward", action="store_true",
                    help="time whole training steps -- forward pass, backward pass and update, inputs resident on the "
                         "device -- instead of the backward pass and update alone (the metric's name says so)")
    ap.add_argument("--no-reference-tape", action="store_true",
                    help="skip the second measurement of the unfused one-stream tape (profiler runs: keeps its "
                         "kernels out of the trace)")
    ap.add_argument("--per-parameter-update", action="store_true",
                    help="update each parameter right after its gradient (one launch each) instead of one fused launch")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

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
    x_dev, labels_dev = hip.from_numpy(x), hip.from_numpy(labels)
    net.forward(x_dev, labels_dev)
    fused = not args.per_parameter_update
    if args.with_forward and args.graph:
        print("bench.py: --with-forward times the eager tape (drop --graph)", file=sys.stderr)
        sys.exit(2)

    sync = dev.Sync   # waits for both streams of the device

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
            if args.with_forward:
                net.forward(x_dev, labels_dev)
            net.backward_and_update(fused_update=fused)
    for _ in range(args.warmup):
        step()
    # one event on the main stream at every step boundary (a step ends with the join and the update there)
    evs = []
    for _ in range(args.steps + 1):
        e = C.c_void_p()
        _lib.check(lib.sgh_event_create(C.byref(e)), "sgh_event_create")
        evs.append(e)
    sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        _lib.check(lib.sgh_event_record(evs[i], dev.stream))
        step()
    _lib.check(lib.sgh_event_record(evs[args.steps], dev.stream))
    t_enqueued = time.perf_counter() - t0   # host time to enqueue every launch of the timed steps
    sync()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    imgs_per_s = args.batch * args.steps / elapsed
    step_ms = []
    for i in range(args.steps):
        ms = C.c_float()
        _lib.check(lib.sgh_event_elapsed_ms(evs[i], evs[i + 1], C.byref(ms)))
        step_ms.append(ms.value)
    for e in evs:
        lib.sgh_event_destroy(e)
    # one more step enqueued into empty queues: what the host needs when nothing makes it wait
    t1 = time.perf_counter()
    step()
    t_idle_enqueue = time.perf_counter() - t1
    sync()
    step_ms.sort()
    median_ms = step_ms[len(step_ms) // 2] if len(step_ms) % 2 else 0.5 * (step_ms[len(step_ms) // 2 - 1] + step_ms[len(step_ms) // 2])

    if graph:
        dev.ResetGraph()
    # What a SINGA tree with unchanged python/singa/autograd.py and opt.py would see through this library: one call
    # per reference op (ReLU.backward and _BatchNorm2d.backward separately, `+=` as its own kernel, a weight
    # re-layout inside every data gradient), everything on the one device stream, and SGD.apply parameter by
    # parameter (python/singa/autograd.py:128-224, python/singa/opt.py:269-310).  A short second measurement
    # after the timed region, reported beside the headline figure.
    reference_tape = None
    if not (args.no_fusion or args.with_forward or args.no_reference_tape):
        saved = {f: getattr(hip, f) for f in ("fuse_bn_relu", "fuse_dgrad_add", "fuse_add_relu", "fuse_wgrad_bias",
                                              "batch_relayout", "overlap_wgrad", "fuse_forward")}
        hip.set_fusion(False)
        net.sgd.op_by_op = True     # SGD.apply's own tensor ops, three launches per parameter
        ref_steps = max(3, min(args.steps, 10))
        for _ in range(2):
            net.backward_and_update(fused_update=False)
        sync()
        t2 = time.perf_counter()
        for _ in range(ref_steps):
            net.backward_and_update(fused_update=False)
        sync()
        ref_ms = (time.perf_counter() - t2) / ref_steps * 1e3
        reference_tape = {"value": round(args.batch / ref_ms * 1e3, 2), "unit": "imgs/s", "ms_per_step": round(ref_ms, 4),
                          "steps": ref_steps,
                          "tape": "one call per reference op on one stream, SGD.apply parameter by parameter through its own "
                                  "Axpy / EltwiseMult ops (what unchanged autograd.py / opt.py issue)"}
        for f, v in saved.items():
            setattr(hip, f, v)
        net.sgd.op_by_op = False
    # kernel-level pass (eager): every conv / GEMM launch bracketed by HIP events on the device stream
    prof_steps = max(1, min(args.steps, 5))
    hip.overlap_wgrad = False   # one kernel at a time on the device, so that an event pair brackets that kernel alone
    lib.sgh_prof_enable(1)
    for _ in range(prof_steps):
        net.backward_and_update(fused_update=fused)
    sync()
    prof = collect_prof(lib)
    lib.sgh_prof_enable(0)
    lib.sgh_prof_clear()
    conv = {k: prof[k] for k in ("conv_dgrad", "conv_wgrad", "conv_dgrad16", "conv_wgrad16") if k in prof}
    flop = sum(v["work"] for v in conv.values())
    ms = sum(v["ms"] for v in conv.values())
    launches = sum(v["launches"] for v in conv.values())
    kernels = sorted(set().union(*[v["kernels"] for v in conv.values()])) if conv else []
    achieved = flop / (ms * 1e-3) / 1e12 if ms > 0 else 0.0
    peak = PEAK_16BIT_MFMA_TFLOPS if half else PEAK_FP32_MFMA_TFLOPS
    workload_key = "%s N=%d %s%s" % (args.config, args.batch, args.storage, " no-fusion" if args.no_fusion else "")
    roofline = {
        "bound": "mfma", "achieved": round(achieved, 3), "peak": peak, "unit": "TFLOP/s",
        "frac": round(achieved / peak, 4),
        "traffic": traffic_from_profile(workload_key, kernels),
        "traffic_unit": "HBM bytes per step over the same launches (rocprofv3 FETCH_SIZE + WRITE_SIZE, calibrated on a "
                        "streaming kernel; from profiles/%s, null when that summary covers other kernels or another workload)"
                        % os.path.basename(TRAFFIC_PROFILE),
        "kernel": "%s MFMA conv dgrad + wgrad kernels (%s; %d launches/step)"
                  % ("16-bit" if half else "fp32", ", ".join(kernels), launches // prof_steps),
        "flop_per_step": flop / prof_steps, "kernel_ms_per_step": round(ms / prof_steps, 4),
        "timing": "HIP events attached to each dispatch (the kernel's own start and end) in %d extra steps with all "
                  "kernels on one stream (the timed steps run the weight gradients on a second stream)" % prof_steps,
    }
    for k, v in conv.items():
        roofline[k + "_tflops"] = round(v["work"] / (v["ms"] * 1e-3) / 1e12, 3) if v["ms"] > 0 else 0.0
    # whole entry points (weight re-layout, split-K reduction and column gather kernels included)
    ops_ms = sum(prof[k]["ms"] for k in ("conv_dgrad_op", "conv_wgrad_op") if k in prof)
    roofline["entry_points_ms_per_step"] = round(ops_ms / prof_steps, 4)

    # the bandwidth-bound families: algorithmic bytes (minimal tensor traffic) / time between the two events
    hbm = {}
    for k in ("bn_relu_bwd", "bn_bwd", "relu_bwd", "relu_bwd_add", "add", "pool_bwd", "sgd"):
        if k in prof and prof[k]["ms"] > 0:
            v = prof[k]
            gbs = v["work"] / (v["ms"] * 1e-3) / 1e9
            hbm[k] = {"launches_per_step": v["launches"] // prof_steps, "bytes_per_step": v["work"] / prof_steps,
                      "ms_per_step": round(v["ms"] / prof_steps, 4), "GB/s": round(gbs, 1),
                      "frac": round(gbs / PEAK_HBM_GBS, 4)}

    out = {
        "metric": "forward+backward+update imgs/sec, %s N=%d %s" % (args.config, args.batch, args.storage) if args.with_forward
                  else "backward+update imgs/sec, ResNet-18 N=64 fp32" if (args.config == "resnet18" and not half and args.batch == 64)
                  else "backward+update imgs/sec, %s N=%d %s" % (args.config, args.batch, args.storage),
        "value": round(imgs_per_s, 2), "unit": "imgs/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_median": round(median_ms, 4), "ms_per_step_min": round(step_ms[0], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.storage, "data": "synthetic",
        "config": {"workload": "%s %sbackward+update, N=%d, 3x224x224, %s, SGD momentum 0.9" % (
                       args.config, "forward+" if args.with_forward else "", args.batch, "fp32" if not half else args.storage + " storage / fp32 accumulate, statistics and master weights"),
                   "update": "fused multi-tensor" if fused else "per parameter",
                   "launch": "one recorded step replayed (graph mode)" if graph else "eager, one launch per kernel",
                   "tape": "ReLU backward folded into BatchNorm backward (conv-BN-ReLU), residual += folded into the "
                           + ("data gradient" if hip.fuse_dgrad_add else "ReLU backward that reads the sum")
                           + ", weight re-layouts in one launch"
                           + (", weight gradients on a second stream" if not args.no_overlap else "")
                           if hip.fuse_bn_relu
                           else "one call per reference op"},
        "roofline": roofline,
        "hbm_kernels": {"peak_GB/s": PEAK_HBM_GBS, "bytes": "algorithmic (every tensor of the op once)",
                        "timing": "HIP events attached to the dispatch where the entry point is one kernel, a pair of markers "
                                  "around it otherwise; same extra steps as the roofline", **hbm},
        "host_enqueue_ms_per_step": round(t_enqueued / args.steps * 1e3, 4),
        "host_enqueue_ms_idle_queue": round(t_idle_enqueue * 1e3, 4),
    }
    if reference_tape is not None:
        out["reference_tape"] = reference_tape
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.config, args.cpu_sample_batch or args.batch, args.cpu_budget_s,
                                           args.cpu_single_thread_batch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
