#!/usr/bin/env python3
"""Benchmark of the tiny-dnn training hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others]

Prints ONE JSON line. The default workload is the CIFAR-10-shape CNN train step at batch
128 (fwd + bwd + update, Adam), the configuration the samples/s target is quoted on; inputs
are synthetic and resident in HBM before the timed region. Other workloads:
vgg_stack_b64, lenet5_b16 (train steps), conv2d_bwd_b64 and fc_bwd_adam_b256 (single-op
backward passes). Their results are appended under "others" in compact form (ms/step,
samples/s, step TFLOP/s, the slowest kernels with their roofline fraction, a bounded CPU
baseline), so that one run times all five configurations; ``--no-others`` leaves them out.
Every timed region (whole steps and the per-kernel pass, of every workload) follows untimed
steps that keep the device busy for 100 ms, the other workloads run at least 50 timed steps,
and all CPU legs come after the last GPU measurement.

"roofline" describes the kernel with the largest total time in the workload: its average
launch duration is measured with HIP events on the library's stream in a second, separately
timed pass (per-launch events slow the step down, so they are kept out of ``value``).
"cpu_baseline" times the reference's OpenMP+AVX build (oracle/_ref, kind "reference") or,
where that library is absent, the scalar restatement (kind "port") on this host's cores.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
PER_KERNEL_PASSES = 2
STEPS_PER_CALL = 8   # train steps a call of the network workloads' timed region


def load_pkg():
    T = importlib.import_module("tiny-cnn_amd")
    W = importlib.import_module("tiny-cnn_amd.workloads")
    return T, W


class NetWorkload:
    def __init__(self, T, W, name, extra_flags=0):
        self.T, self.W, self.name = T, W, name
        (self.spec, self.params, x, t, self.batch, self.loss, self.opt_kind,
         self.opt_kw) = W.make_batch(name)
        self.net = T.Net(W.build_layers(T, self.spec), self.batch,
                         T.NET_FUSE_ACT_GRAD | T.NET_GRAPH | T.NET_SAMPLE_STEP | extra_flags)
        for (i, which, a) in self.params:
            self.net.set_param(i, which, a)
        self.opt = T.opt_desc(self.opt_kind, **self.opt_kw)
        self.x, self.t = T.to_device(x), T.to_device(t)
        self.samples = self.batch
        self.config = {"workload": name, "batch": self.batch, "loss": self.loss,
                       "optimizer": self.opt_kind, "step": "fwd+bwd+update",
                       "launch": f"captured HIP graphs of {STEPS_PER_CALL} steps each (tdh_net_train_steps; the "
                                 "per-kernel pass runs the same kernels eagerly, step by step)",
                       "flop_per_step": 3 * self.batch * W.flops_per_sample(self.spec)}

        self.host_x, self.host_t = x, t
        self.feeder = None

    def step(self):
        self.net.train_step(self.opt, self.loss, self.batch, self.x, self.t)

    def run(self, n):
        """n steps, STEPS_PER_CALL at a time (tdh_net_train_steps: one captured graph holds them, so
        a replay starts once for all of them), the rest one by one."""
        k = STEPS_PER_CALL
        xs, ts = [self.x] * k, [self.t] * k
        for _ in range(n // k):
            self.net.train_steps(self.opt, self.loss, self.batch, xs, ts)
        for _ in range(n % k):
            self.step()

    def step_from_host(self):
        """The same step when the caller hands over host buffers: inputs and targets cross PCIe,
        two batches ahead (a batch is copied and uploaded while the step before it runs)."""
        if self.feeder is None:
            self.feeder = self.T.Feeder(self.host_x.shape[1], self.host_t.shape[1], self.batch)
            self.feeder.stage(self.host_x, self.host_t)
            self.feeder.stage(self.host_x, self.host_t)
        xd, td, n = self.feeder.acquire()
        self.feeder.stage(self.host_x, self.host_t)  # the worker copies and uploads while this thread launches
        self.net.train_step(self.opt, self.loss, n, xd, td)


class ConvBwdWorkload:
    """configs[1]: conv2d backward, batch 64, 32x64x64 -> 64 channels, 3x3, pad same."""

    def __init__(self, T, W, name="conv2d_bwd_b64", batch=64):
        self.T = T
        (hw, _, c, k, oc), x, w, dy = W.conv_bwd_case(batch=batch)
        self.d = T.conv_desc(hw, hw, c, k, k, oc, pad_same=True)
        self.batch = self.samples = batch
        self.x, self.w, self.dy = T.to_device(x), T.to_device(w), T.to_device(dy)
        self.dx, self.dw, self.db = T.DevBuf(x.shape), T.DevBuf(w.shape), T.DevBuf((oc,))
        gemm_flop = 2 * batch * hw * hw * oc * c * k * k
        self.config = {"workload": name, "batch": batch, "step": "conv2d backward (dX, dW, db)",
                       "flop_per_step": 2 * gemm_flop}

    def step(self):
        self.T.conv2d_bwd(self.d, self.batch, self.x, self.w, self.dy, self.dx, self.dw, self.db)


class FcBwdWorkload:
    """configs[2]: tanh-grad -> FC backward (dX, dW, db) -> Adam on W and b, batch 256."""

    def __init__(self, T, W, name="fc_bwd_adam_b256", batch=256, n=4096):
        self.T = T
        x, w, b, dy = W.fc_bwd_case(batch, n, n)
        self.n, self.batch, self.samples = n, batch, batch
        self.x, self.w, self.b = T.to_device(x), T.to_device(w), T.to_device(b)
        self.y, self.dy, self.dz = T.DevBuf((batch, n)), T.to_device(dy), T.DevBuf((batch, n))
        T.fc_fwd(n, n, True, batch, self.x, self.w, self.b, self.dz)
        T.act_fwd("tanh", batch, n, self.dz, self.y)
        self.dx, self.dw, self.db = T.DevBuf((batch, n)), T.DevBuf((n * n,)), T.DevBuf((n,))
        self.s = [T.DevBuf((n * n,), zero=True), T.DevBuf((n * n,), zero=True),
                  T.DevBuf((n,), zero=True), T.DevBuf((n,), zero=True)]
        self.opt = T.opt_desc("adam")
        self.config = {"workload": name, "batch": batch, "step": "tanh-grad + fc backward + adam",
                       "flop_per_step": 4 * batch * n * n}

    def step(self):
        T, n, bs = self.T, self.n, self.batch
        T.act_bwd("tanh", bs, n, self.y, self.dy, self.dz)
        T.fc_bwd(n, n, True, bs, self.x, self.w, self.dz, self.dx, self.dw, self.db)
        T.opt_update(self.opt, n * n, self.dw, self.w, self.s[0], self.s[1])
        T.opt_update(self.opt, n, self.db, self.b, self.s[2], self.s[3])


def make_workload(T, W, name):
    if name in W.WORKLOADS:
        return NetWorkload(T, W, name)
    if name == "conv2d_bwd_b64":
        return ConvBwdWorkload(T, W)
    if name == "fc_bwd_adam_b256":
        return FcBwdWorkload(T, W)
    raise SystemExit(f"unknown workload {name}")


def roofline_of(entry):
    per_s = entry["work"] / (entry["avg_us"] * 1e-6) if entry["avg_us"] > 0 else 0.0
    if entry["unit"] == "flop":
        achieved, peak, unit, bound = per_s / 1e12, PEAK_FP32_MFMA_TFLOPS, "TFLOP/s", "mfma"
    else:
        achieved, peak, unit, bound = per_s / 1e9, PEAK_HBM_GBS, "GB/s", "hbm"
    return {"kernel": entry["tag"], "bound": bound, "achieved": round(achieved, 3), "peak": peak,
            "unit": unit, "frac": round(achieved / peak, 4), "traffic": None,
            "avg_launch_us": round(entry["avg_us"], 2), "launches": entry["launches"],
            "algorithmic_work_per_launch": entry["work"]}


WARM_MS = 100.0


def run_steps(wl, n):
    if hasattr(wl, "run"):
        wl.run(n)
    else:
        for _ in range(n):
            wl.step()


def warm_by_time(T, wl, min_ms=WARM_MS):
    """Runs untimed steps until the device has been busy for `min_ms`: a GPU that has idled (a
    CPU leg, a fresh process) clocks down, and a timed region of a few milliseconds would
    otherwise be measured on the ramp. Returns the number of steps run."""
    done, spent, chunk = 0, 0.0, 4
    while spent < min_ms and done < 100000:
        t0 = time.perf_counter()
        run_steps(wl, chunk)
        T.sync()
        spent += (time.perf_counter() - t0) * 1e3
        done += chunk
        chunk = min(chunk * 2, 256)
    return done


def run_workload(T, wl, steps, warmup, profile_steps, sequence=None):
    run_steps(wl, warmup)
    T.sync()
    warm_by_time(T, wl)
    e0, e1 = T.Event(), T.Event()
    t0 = time.perf_counter()
    e0.record()
    run_steps(wl, steps)
    e1.record()
    T.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    single_ms = None
    if hasattr(wl, "run"):   # the same steps one call each, for comparison
        t0 = time.perf_counter()
        for _ in range(steps):
            wl.step()
        T.sync()
        single_ms = (time.perf_counter() - t0) * 1e3 / steps
    gpu_ms = e1.elapsed_ms_since(e0)
    ms_per_step = wall_ms / steps
    # second pass: per-kernel durations, stamped by the dispatches themselves. A network workload
    # launches eagerly here (the timed steps replayed a graph): one eager step first, so that
    # one-time costs of that path (code loading, scratch growth) do not sit between the launches
    # of a scope
    T.profile_begin()
    wl.step()
    T.profile_end()
    warm_by_time(T, wl)
    marker = T.DevBuf((4400,), zero=True)
    prof = None
    for _ in range(PER_KERNEL_PASSES):
        # (two passes, the one with less kernel time in total is reported: a single launch that
        # something outside the workload held up by a few hundred microseconds would otherwise
        # move a ten-launch average by tens of percent)
        T.profile_begin()
        for _ in range(profile_steps):
            T.profile_mark(marker)   # three fill launches under a tag of their own
            wl.step()
        T.profile_mark(marker)
        p = T.profile_end()
        if prof is None or sum(e["total_ms"] for e in p) < sum(e["total_ms"] for e in prof):
            prof = p
    # the marks are not part of the workload
    prof = [e for e in prof if e["tag"] != "profile_mark"]
    if sequence is not None:  # the tags of one step's launches, in dispatch order
        tags = T.profile_launches()
        per = (len(tags) - 3) // profile_steps
        chunks = [tags[i * per:(i + 1) * per] for i in range(profile_steps)]
        assert per * profile_steps + 3 == len(tags) and all(c == chunks[0] for c in chunks) \
            and chunks[0][:3] == ["profile_mark"] * 3, "the steps of the per-kernel pass differ"
        sequence.extend(chunks[0][3:])
    kernels = [roofline_of(e) for e in prof]
    for k, e in zip(kernels, prof):
        k["ms_per_step"] = round(e["total_ms"] / profile_steps, 4)
    return {"ms_per_step": ms_per_step, "gpu_ms_per_step": gpu_ms / steps, "single_step_calls_ms": single_ms,
            "samples_per_s": wl.samples / (ms_per_step * 1e-3), "kernels": kernels,
            "profile_steps": profile_steps}


def copy_yardstick(T, mib=256, reps=5):
    """Achieved bandwidth of the library's plain copy kernel (reads and writes `mib` MiB each):
    what a bandwidth-bound kernel can reach on this device, and the dispatch of known size
    that hardware byte counters are scaled by."""
    n = mib << 20
    a, b = T.DevBuf((n // 4,), zero=True), T.DevBuf((n // 4,))
    T.copy_d2d(b, a)
    T.sync()
    e0, e1 = T.Event(), T.Event()
    e0.record()
    for _ in range(reps):
        T.copy_d2d(b, a)
    e1.record()
    T.sync()
    us = e1.elapsed_ms_since(e0) * 1e3 / reps
    return {"kernel": "copy_kernel", "read_bytes": n, "write_bytes": n, "avg_launch_us": round(us, 2),
            "GB/s": round(2 * n / (us * 1e-6) / 1e9, 1)}


def measured_traffic(tag, workload=None):
    """HBM bytes per launch of kernel `tag` from hardware counters, when a counter run of this
    workload has been recorded in profiles/hbm_traffic.json (null otherwise)."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            js = json.load(f)
        rec = js.get("workloads", {}).get(workload, {}).get(tag)
        return rec and rec["hbm_bytes_per_launch"]
    except (OSError, ValueError, KeyError):
        return None


def cpu_baseline(W, name, budget_s=20.0, max_steps=20):
    """Reference CPU figure on a bounded sample of the same workload."""
    from oracle import oracle as O
    try:
        if not os.path.exists(O.ORACLE_SO):
            O.build()
    except Exception:
        pass
    kind = "reference" if O.ref_lib("avx") is not None else "port"
    cores = os.cpu_count() or 1
    if kind == "reference":
        cores = O.ref_lib("avx").tdr_num_threads()
    if name in W.WORKLOADS:
        full_batch = W.WORKLOADS[name][1]
        batch = {"vgg_stack_b64": 2}.get(name, full_batch)
        spec, params, x, t, batch, loss, opt_kind, opt_kw = W.make_batch(name, batch=batch)
        opt = O.opt_desc(opt_kind, **opt_kw)
        if kind == "reference":
            net = O.RefNet(W.build_layers(O, spec), "avx", 1)
            for (i, which, a) in params:
                net.set_param(i, which, a)
            net.fit(opt, loss, x, t, 1)  # warm-up step (allocates the per-sample buffers)
            steps, spent, per = 0, 0.0, []
            while spent < budget_s and steps < max_steps:
                sec = net.fit(opt, loss, x, t, 1)
                per.append(sec); spent += sec; steps += 1
        else:
            net = O.OracleNet(W.build_layers(O, spec), batch)
            for (i, which, a) in params:
                (net.weight(i) if which == 0 else net.bias(i))[:] = a
            steps, spent, per = 0, 0.0, []
            while spent < budget_s and steps < max_steps:
                t0 = time.perf_counter(); net.train_step(opt, loss, x, t)
                sec = time.perf_counter() - t0
                per.append(sec); spent += sec; steps += 1
        med = float(np.median(per))
        return {"value": round(batch / med, 2), "unit": "samples/s", "cores": cores, "kind": kind,
                "sample": f"{steps} train steps at batch {batch} (full workload batch {full_batch}), "
                          f"median {med * 1e3:.1f} ms/step"}
    if name == "conv2d_bwd_b64":
        batch = 8
        (hw, _, c, k, oc), x, w, dy = W.conv_bwd_case(batch=batch)
        d = O.conv_desc(hw, hw, c, k, k, oc, pad_same=True)
        if kind == "reference":
            *_, sec = O.ref_conv2d_bwd(d, x, w, dy, kind="avx", engine=1, repeat=3, want_time=True)
        else:
            t0 = time.perf_counter(); O.conv2d_bwd(d, x, w, dy); sec = time.perf_counter() - t0
        return {"value": round(batch / sec, 2), "unit": "samples/s", "cores": cores, "kind": kind,
                "sample": f"layer.backward at batch {batch} (full workload batch 64), best of 3: "
                          f"{sec * 1e3:.1f} ms"}
    if name == "fc_bwd_adam_b256":
        batch = 16
        x, w, b, dy = W.fc_bwd_case(batch)
        if kind == "reference":
            *_, sec = O.ref_fc_bwd(x, w, dy, kind="avx", engine=1, repeat=3, want_time=True)
        else:
            t0 = time.perf_counter(); O.fc_bwd(x, w, dy); sec = time.perf_counter() - t0
        return {"value": round(batch / sec, 2), "unit": "samples/s", "cores": cores, "kind": kind,
                "sample": f"fc layer.backward only (no tanh-grad/adam) at batch {batch} (full "
                          f"workload batch 256; per-sample gradient storage needs 67 MB/sample), "
                          f"best of 3: {sec * 1e3:.1f} ms"}
    return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cifar10_cnn_b128")
    ap.add_argument("--others", action="store_true", help="(default) also run the other workloads")
    ap.add_argument("--no-others", action="store_true", help="only the named workload")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-host-inputs", action="store_true",
                    help="leave out the legs beside the headline: host batches handed over every step, the step "
                         "without the input gradient (profiler runs: rocprofv3 7.2 dies in the first of the two "
                         "for the VGG workload, in a host copy below hipGraphInstantiate)")
    ap.add_argument("--sequence-out", default=None,
                    help="write the kernel tags of one step in dispatch order to this JSON file "
                         "(tiny-cnn_amd.profsum reads a rocprofv3 trace of the same run tag by tag with it)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no multi-GPU part); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)

    T, W = load_pkg()
    T.init(0)
    dev_name, cus, mem = T.device_info()

    wl = make_workload(T, W, args.workload)
    prof_steps = max(1, min(args.steps, 10))
    sequence = [] if args.sequence_out else None
    res = run_workload(T, wl, args.steps, args.warmup, prof_steps, sequence)
    if args.sequence_out:
        with open(args.sequence_out, "w") as f:
            json.dump({"workload": args.workload, "sequence": sequence}, f, indent=1)
    out = {
        "metric": "train samples/sec (fwd+bwd+update)",
        "value": round(res["samples_per_s"], 2),
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 4),
        "gpu_ms_per_step": round(res["gpu_ms_per_step"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": wl.config,
        "device": {"name": dev_name, "compute_units": cus},
        "one_step_per_call": None if res["single_step_calls_ms"] is None else
        {"ms_per_step": round(res["single_step_calls_ms"], 4),
         "samples_per_s": round(wl.samples / (res["single_step_calls_ms"] * 1e-3), 2),
         "note": "the same steps through tdh_net_train_step, one captured graph replayed per step"},
        "roofline": dict(res["kernels"][0]) if res["kernels"] else None,
        "kernels": res["kernels"],
    }
    if out["roofline"]:
        out["roofline"]["traffic"] = measured_traffic(out["roofline"]["kernel"], args.workload)
    flop_k = [k for k in res["kernels"] if k["unit"] == "TFLOP/s"]
    if flop_k:  # all MFMA-bound kernels of the step together
        tot_flop = sum(k["algorithmic_work_per_launch"] * k["launches"] for k in flop_k)
        tot_s = sum(k["avg_launch_us"] * k["launches"] for k in flop_k) * 1e-6
        out["mfma_kernels_together"] = {"TFLOP/s": round(tot_flop / tot_s / 1e12, 2),
                                        "frac": round(tot_flop / tot_s / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
    out["copy_yardstick"] = copy_yardstick(T)
    if hasattr(wl, "step_from_host") and not args.no_host_inputs:  # never `value`: reported for callers that own host buffers
        for _ in range(12):  # every device slot gets its captured steps (three slots, two Adam buffers)
            wl.step_from_host()
        T.sync()
        host_steps = max(args.steps, 200)
        t0 = time.perf_counter()
        for _ in range(host_steps):
            wl.step_from_host()
        T.sync()
        ms = (time.perf_counter() - t0) * 1e3 / host_steps
        out["host_inputs"] = {"ms_per_step": round(ms, 4), "samples_per_s": round(wl.samples / (ms * 1e-3), 2),
                              "steps": host_steps,
                              "note": "inputs and targets handed over in pageable host memory every step "
                                      "and uploaded through pinned slots on a copy stream (tdh_feeder)"}
    if isinstance(wl, NetWorkload) and not args.no_host_inputs:
        # never `value` either: the same step without the gradient of the net's input, which the
        # reference computes and training never reads (the caller's choice: TDH_NET_NO_INPUT_GRAD)
        w3 = NetWorkload(T, W, args.workload, T.NET_NO_INPUT_GRAD)
        run_steps(w3, max(2, args.warmup))
        T.sync()
        warm_by_time(T, w3)
        t0 = time.perf_counter()
        run_steps(w3, args.steps)
        T.sync()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        out["no_input_grad"] = {"ms_per_step": round(ms, 4), "samples_per_s": round(w3.samples / (ms * 1e-3), 2),
                                "steps": args.steps,
                                "note": "TDH_NET_NO_INPUT_GRAD: the first layer's input gradient is left out; "
                                        "weights after the step are the same"}
        del w3
    if wl.config.get("flop_per_step"):
        out["step_tflops"] = round(wl.config["flop_per_step"] / (res["ms_per_step"] * 1e-3) / 1e12, 3)
    out["timing"] = {"warm_ms_before_each_timed_region": WARM_MS,
                     "per_kernel_pass_steps": res["profile_steps"],
                     "per_kernel_passes": f"{PER_KERNEL_PASSES}, the one with the lower total kernel time is reported",
                     "order": "all GPU timing first, every CPU baseline afterwards"}
    del wl
    others = {}
    if not args.no_others:
        # the other four configurations, compact: the six slowest kernels each. Every GPU
        # measurement of the run comes before the first CPU leg, so no timed region follows
        # seconds of an idle device.
        other_steps = max(50, args.steps)
        for name in ("conv2d_bwd_b64", "fc_bwd_adam_b256", "vgg_stack_b64", "lenet5_b16",
                     "cifar10_cnn_b128"):
            if name == args.workload:
                continue
            w2 = make_workload(T, W, name)
            r = run_workload(T, w2, other_steps, max(2, args.warmup), 10)
            ks = r["kernels"]
            flop_k = [k for k in ks if k["bound"] == "mfma"]
            rec = {"samples_per_s": round(r["samples_per_s"], 2),
                   "ms_per_step": round(r["ms_per_step"], 4), "steps": other_steps,
                   "one_step_per_call_ms": None if r["single_step_calls_ms"] is None else round(r["single_step_calls_ms"], 4),
                   "config": w2.config,
                   "step_tflops": round(w2.config["flop_per_step"] / (r["ms_per_step"] * 1e-3) / 1e12, 3),
                   "roofline": {k: ks[0][k] for k in ("kernel", "bound", "achieved", "peak", "unit", "frac",
                                                      "avg_launch_us")} if ks else None,
                   "kernels": [{k: e[k] for k in ("kernel", "achieved", "unit", "frac", "avg_launch_us",
                                                  "launches", "ms_per_step")} for e in ks[:6]]}
            if rec["roofline"]:
                rec["roofline"]["traffic"] = measured_traffic(rec["roofline"]["kernel"], name)
            if flop_k:   # all MFMA-bound kernels of the step together
                tot_flop = sum(k["algorithmic_work_per_launch"] * k["launches"] for k in flop_k)
                tot_s = sum(k["avg_launch_us"] * k["launches"] for k in flop_k) * 1e-6
                rec["mfma_kernels_together"] = {"TFLOP/s": round(tot_flop / tot_s / 1e12, 2),
                                                "frac": round(tot_flop / tot_s / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4)}
            del w2
            others[name] = rec
    if not args.no_cpu_baseline:
        try:
            out["cpu_baseline"] = cpu_baseline(W, args.workload)
            if out["cpu_baseline"]:
                out["gpu_over_cpu"] = round(out["value"] / out["cpu_baseline"]["value"], 1)
        except Exception as e:  # the baseline is reported, never required
            out["cpu_baseline"] = {"error": repr(e)}
        for name, rec in others.items():  # capped at a few seconds each
            try:
                rec["cpu_baseline"] = cpu_baseline(W, name, budget_s=4.0, max_steps=3)
                if rec["cpu_baseline"]:
                    rec["gpu_over_cpu"] = round(rec["samples_per_s"] / rec["cpu_baseline"]["value"], 1)
            except Exception as e:
                rec["cpu_baseline"] = {"error": repr(e)}
    if others:
        out["others"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
