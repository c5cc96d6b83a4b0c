#!/usr/bin/env python3
"""Benchmark of the MI355X VJP/JVP path.  Prints ONE JSON line.

Workload (N=1): BASELINE.json configs[1], "Broadcast and reduction VJPs":
    L(A, b, c) = sum(logsumexp(A * b[None, :] + c[:, None], axis=1)),  float32,
    A (8192, 4096) ~ N(0,1), b (4096,) ~ U(.5, 1.5), c (8192,) ~ N(0,1), RandomState(0);
    one step = one grad(L, (0, 1, 2))(A, b, c) call (forward trace + backward replay), inputs
    resident in HBM before the timed region.
metric = grad evals/sec.  `roofline` describes the kernel that takes most of the step, timed
with HIP events on the launch stream, once during the timed steps (`avg_launch_ms_in_timed_region`:
the eager tracer leaves the GPU waiting for the host, so the event pair also holds the host's
dispatch latency) and once over the same number of steps with the stream kept busy ahead of each
step (`avg_launch_ms`, the figure `achieved` uses: the events then bracket GPU execution only, which
is what a rocprofv3 kernel trace reports); `cpu_baseline` is the CPU oracle
(the NumPy restatement of reference autograd) timed on this machine's host cores on a
bounded sample of the same workload.  `extras` holds the other four workloads and the MLP
contraction rate, measured after the timed region (never part of `value`).
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_F32_PEAK_TFLOPS = 157.3


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument("--no-extras", action="store_true", help="skip the other workloads")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget for the CPU baseline sample")
    ap.add_argument("--workload", default="bcast", choices=["bcast", "tanh", "mlp", "rnn", "rosen", "convnet", "arrayfuncs"],
                    help="bcast (default) is the headline workload, BASELINE configs[1]; the others are the "
                         "remaining BASELINE configs and the convnet example, selectable for profiling")
    ap.add_argument("--graph", action="store_true",
                    help="time the workload replayed from a HIP graph (autograd_amd.capture) instead of the eager "
                         "tracer; no per-kernel events in this mode")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch plain copies of a (8192,4096) f32 array (134.2 MB read + 134.2 MB written "
                         "each): the reference dispatch that hardware traffic counters are scaled by")
    return ap.parse_args()


def end_to_end(compulsory_bytes, evals_per_sec):
    """The secondary roofline figure of a whole evaluation: the bytes it cannot avoid (its inputs read once, its
    results written once) over the time one evaluation takes, against the HBM peak."""
    gbps = compulsory_bytes * evals_per_sec / 1e9
    return {"compulsory_bytes": compulsory_bytes, "achieved_GBps": gbps, "frac": gbps / HBM_PEAK_GBS}


def time_steps(fn, sync, steps, warmup):
    # at least three untimed runs: an elementwise program handed over for the third time is compiled into a kernel
    # of its own (a few tenths of a second, once), which belongs to the warm-up like the first run's allocations
    for _ in range(max(warmup, 3)):
        fn()
    sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    sync()
    return (time.perf_counter() - t0) / steps


class HeadStart:
    """Keeps the launch stream busy for about ``ms`` milliseconds, so that the launches the host enqueues
    meanwhile run back to back on the GPU and HIP events around one of them measure its execution, not the
    host's dispatch latency.  The filler only READS (minima of a 256 MiB array, a reduction no workload here
    launches, so a kernel trace tells it apart by its `AccMin` kernels): what it leaves in the caches is
    clean, as after the reads that end a real evaluation; a filler that writes leaves 256 MiB of dirty lines
    whose write-back is then charged to the first kernels of the measured step (measured: +10 us on the
    134 MB forward reduction)."""

    def __init__(self):
        import numpy as onp

        from autograd_amd import _lib
        from autograd_amd._lib import Op, Red
        from autograd_amd.numpy import devarray as D

        self._lib = _lib
        self.buf = D.empty((64 << 20,), onp.float32)
        _lib.fill(_lib.DTYPE_CODE[self.buf.dtype], self.buf._t, 0.0)
        self.read = lambda: D.map_reduce(Op.COPY, Red.MIN, self.buf.dtype, (self.buf,), (0,), False)
        self.read()
        _lib.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            self.read()
        _lib.synchronize()
        self.ms_per_pass = (time.perf_counter() - t0) / 20 * 1e3

    def __call__(self, ms):
        with self._lib.untimed():
            for _ in range(max(1, int(ms / self.ms_per_pass) + 1)):
                self.read()


def event_pair_overhead_ms(ahead, pairs=40):
    """What a HIP event pair adds to the kernel it brackets, measured live: pairs around ONE launch of a probe
    kernel give overhead + k, pairs around TWO of them overhead + 2k, so overhead = 2 * t1 - t2.  The probe
    is a 64 MiB fill (about 10 us, the scale of the kernels being timed): around a tiny launch the same
    arithmetic gives 4.5 us instead of about 2, because a tiny kernel hides none of the pair's cost, and
    subtracting that from a 20-50 us kernel would flatter it.  Taken behind a busy stream, like the kernel
    timings it corrects."""
    import numpy as onp
    import torch

    from autograd_amd import _lib
    from autograd_amd.numpy import devarray as D

    cell = D.empty((16 << 20,), onp.float32)
    code = _lib.DTYPE_CODE[cell.dtype]
    stream = torch.cuda.current_stream(_lib.device())
    events = [torch.cuda.Event(enable_timing=True) for _ in range(4 * pairs)]
    for ev in events:
        ev.record(stream)
    _lib.synchronize()
    with _lib.untimed():
        ahead(1.0)
        for i in range(pairs):
            events[4 * i].record(stream)
            _lib.fill(code, cell._t, 0.0)
            events[4 * i + 1].record(stream)
            events[4 * i + 2].record(stream)
            _lib.fill(code, cell._t, 0.0)
            _lib.fill(code, cell._t, 0.0)
            events[4 * i + 3].record(stream)
    _lib.synchronize()
    one = sorted(events[4 * i].elapsed_time(events[4 * i + 1]) for i in range(pairs))[pairs // 2]
    two = sorted(events[4 * i + 2].elapsed_time(events[4 * i + 3]) for i in range(pairs))[pairs // 2]
    return max(0.0, 2.0 * one - two)


def cpu_baseline(seconds):
    """Time the CPU oracle on the same full-size workload; bounded by ``seconds``."""
    import numpy as onp

    import autograd_amd as ag
    import oracle.anp as anp
    from autograd_amd import configs

    be = configs.Backend("oracle", anp, anp.logsumexp, ag.grad, ag.elementwise_grad, ag.make_hvp, ag.make_jvp,
                         lambda a: a, onp.asarray, lambda: None)
    inp = configs.bcast_inputs()
    g = configs.bcast_program(be)["grad"]
    t0 = time.perf_counter()
    g(inp["A"], inp["b"], inp["c"])  # warm-up (page faults, BLAS/thread pools)
    first = time.perf_counter() - t0
    times = []
    deadline = time.perf_counter() + max(0.0, seconds - first)
    while len(times) < 50 and (not times or time.perf_counter() + min(times) < deadline):
        t0 = time.perf_counter()
        g(inp["A"], inp["b"], inp["c"])
        times.append(time.perf_counter() - t0)
    best = min(times)
    return {
        "value": 1.0 / best,
        "unit": "grad evals/sec",
        "cores": 1,
        "kind": "port",
        "sample": f"{len(times)} full-size grad evals (8192x4096 f32) after 1 warm-up, best of them; "
                  f"NumPy {onp.__version__} ufunc loops and scipy logsumexp are single-threaded; "
                  f"host has {os.cpu_count()} logical cores",
        "ms_per_eval_min": best * 1e3,
        "ms_per_eval_median": float(onp.median(times)) * 1e3,
    }


def cpu_baseline_contractions(seconds):
    """The CPU oracle on the two workloads whose time goes into BLAS (MLP and RNN gradients, full size): NumPy's
    BLAS uses every host core it is given, so these are all-core figures; each is bounded by ``seconds`` / 2."""
    import numpy as onp

    import autograd_amd as ag
    import oracle.anp as anp
    from autograd_amd import configs

    try:
        from threadpoolctl import threadpool_info

        blas = [f"{d.get('internal_api')} x{d.get('num_threads')}" for d in threadpool_info() if d.get("user_api") == "blas"]
    except Exception:  # threadpoolctl is optional
        blas = []
    be = configs.Backend("oracle", anp, anp.logsumexp, ag.grad, ag.elementwise_grad, ag.make_hvp, ag.make_jvp,
                         lambda a: a, onp.asarray, lambda: None)
    out = {}
    for name, inputs, program in (("mlp", configs.mlp_inputs, configs.mlp_program),
                                  ("rnn", configs.rnn_inputs, configs.rnn_program)):
        inp = inputs()
        g = program(be)["grad"]
        call_args = (inp["params"], inp["X"], inp["T"]) if name == "mlp" else (inp["params"], inp["inputs"], inp["targets"])
        t0 = time.perf_counter()
        g(*call_args)
        first = time.perf_counter() - t0
        times = []
        deadline = time.perf_counter() + max(0.0, seconds / 2 - first)
        while len(times) < 20 and (not times or time.perf_counter() + min(times) < deadline):
            t0 = time.perf_counter()
            g(*call_args)
            times.append(time.perf_counter() - t0)
        out[name] = {"value": 1.0 / min(times), "unit": "grad evals/sec", "cores": os.cpu_count(), "kind": "port",
                     "blas_threads": blas,
                     "sample": f"{len(times)} full-size grad evals after 1 warm-up, best of them",
                     "ms_per_eval_min": min(times) * 1e3}
    return out


def make_workload(name, be):
    """(function, device arguments, config description, arithmetic dtype) for one BASELINE workload;
    inputs are uploaded here, before any timing."""
    from autograd_amd import configs

    if name == "bcast":
        inp = configs.bcast_inputs()
        A, b, c = be.put(inp["A"]), be.put(inp["b"]), be.put(inp["c"])
        g = configs.bcast_program(be)["grad"]
        cfg = {"workload": "configs[1] broadcast+reduction VJPs: grad wrt (A,b,c) of "
                           "sum(logsumexp(A*b[None,:]+c[:,None],axis=1))",
               "A": [8192, 4096], "b": [4096], "c": [8192], "seed": 0}
        return g, (A, b, c), cfg, "f32"
    if name == "tanh":
        x = be.put(configs.tanh_inputs()["x"])
        prog = configs.tanh_program(be)
        cfg = {"workload": "configs[0] elementwise tanh: egrad, egrad^2 and egrad^3 of (1-exp(-2x))/(1+exp(-2x)); "
                           "one step = the three calls", "x": [4194304]}
        return (lambda x: (prog["d1"](x), prog["d2"](x), prog["d3"](x))), (x,), cfg, "f64"
    if name == "mlp":
        inp = configs.mlp_inputs()
        params = configs.tree_map(be.put, inp["params"])
        X, T = be.put(inp["X"]), be.put(inp["T"])
        g = configs.mlp_program(be)["grad"]
        cfg = {"workload": "configs[2] MLP 784-1024-1024-10 tanh, log-softmax loss, grad wrt [(W,b)]",
               "batch": 1024, "seed": 0}
        return g, (params, X, T), cfg, "f32"
    if name == "rnn":
        inp = configs.rnn_inputs()
        params = configs.tree_map(be.put, inp["params"])
        xs, ts = be.put(inp["inputs"]), be.put(inp["targets"])
        g = configs.rnn_program(be)["grad"]
        cfg = {"workload": "configs[3] tanh RNN T=64 B=256 H=512, grad wrt params dict", "seed": 0}
        return g, (params, xs, ts), cfg, "f32"
    if name == "convnet":
        from autograd_amd.scipy.signal import convolve

        inp = configs.convnet_inputs()  # float64, as the example's npr.randn weights and /255.0 images are
        params = configs.tree_map(be.put, inp["params"])
        X, T = be.put(inp["X"]), be.put(inp["T"])
        g = configs.convnet_program(be, convolve)["grad"]
        cfg = {"workload": "examples/convnet.py LeNet stack (conv5x5x6, pool, conv5x5x16, pool, 120, 84, 10) on 28x28, "
                           "grad wrt params dict", "batch": 256, "seed": 0}
        return g, (params, X, T), cfg, "f64"
    if name == "arrayfuncs":
        # not a BASELINE config: the index-shaped kernels of the array-function table (running sums, reversal,
        # triangle, roll, sort) on one 4096 x 4096 matrix and one 16384-vector, forward and cotangent
        import numpy as onp

        np = be.np
        rs = onp.random.RandomState(0)
        x = be.put(rs.randn(4096, 4096).astype(onp.float32))
        v, w = be.put(rs.randn(16384).astype(onp.float32)), be.put(rs.randn(16384).astype(onp.float32))

        def f(x, v):
            y = np.cumsum(x, axis=1) * 1e-3 + np.cumsum(x, axis=0) * 1e-3
            y = y + np.tril(x) - x[::-1] + np.roll(x, 3, axis=1) + np.fliplr(x)
            return np.sum(y * y) + np.sum(np.sort(v) * w)

        cfg = {"workload": "array functions: grad wrt (x, v) of cumsum (both axes), tril, reversed rows and columns, "
                           "roll on x (4096,4096) and sort on v (16384,)", "seed": 0}
        return be.grad(f, (0, 1)), (x, v), cfg, "f32"
    inp = configs.rosen_inputs()
    x, v = be.put(inp["x"]), be.put(inp["v"])
    prog = configs.rosen_program(be)
    cfg = {"workload": "configs[4] Rosenbrock HVP n=2^24: one step = make_hvp(f)(x)[0](v) and make_jvp(grad(f))(x)(v)",
           "seed": 0}
    return (lambda x, v: (prog["hvp_rev"](x, v), prog["hvp_fwd"](x, v))), (x, v), cfg, "f64"


def priced(r, steps, overhead_ms):
    """One row of `kernels_per_step`: launches per step, average duration, algorithmic MB (and GFLOP) per launch and
    the rates they give against the published peaks."""
    ms = max(r["avg_ms"] - overhead_ms, 1e-6)
    row = {"launches": r["launches"] / steps, "avg_ms": round(ms, 5), "MB": round(r["avg_bytes"] / 1e6, 3),
           "GB/s": round(r["avg_bytes"] / (ms * 1e-3) / 1e9, 1),
           "frac_hbm": round(r["avg_bytes"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if r.get("avg_flops"):
        row["GFLOP"] = round(r["avg_flops"] / 1e9, 4)
        row["TFLOP/s"] = round(r["avg_flops"] / (ms * 1e-3) / 1e12, 2)
        row["frac_mfma"] = round(r["avg_flops"] / (ms * 1e-3) / 1e12 / MFMA_F32_PEAK_TFLOPS, 4)
    return row


def measured_traffic(kernel):
    """HBM bytes per launch of ``kernel`` from the committed rocprofv3 counter summary
    (profiles/bcast_grad_hbm_traffic.md: FETCH_SIZE + WRITE_SIZE scaled by a plain copy) and where the figure
    comes from (the file and a hash of its contents, which also identifies it where there is no git history);
    (None, None) when the file has no row for this kernel."""
    import hashlib

    rel = os.path.join("profiles", "bcast_grad_hbm_traffic.md")
    family, _, functor = kernel.partition("<")
    functor = functor.split(">")[0].split(",")[0]
    try:
        text = open(os.path.join(ROOT, rel)).read()
        for line in text.splitlines():
            cells = [c.strip() for c in line.split("|")]
            # (a functor name, `F...`, tells rows of one kernel family apart; other template arguments do not matter)
            if len(cells) > 8 and family in cells[1] and (not functor.startswith("F") or functor in cells[1]):
                digest = hashlib.sha256(text.encode()).hexdigest()[:12]
                return float(cells[7]) * 1e6, f"{rel} sha256:{digest} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)"
    except (OSError, ValueError):
        pass
    return None, None


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); "
              "run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    from autograd_amd import _lib, configs

    be = configs.device_backend()
    fun, fun_args, config, dtype = make_workload(args.workload, be)
    from autograd_amd import _compiled

    # whether the tracer / rule tables / launch marshalling ran as compiled extension modules or interpreted
    config = dict(config, host_modules=_compiled.status()["mode"])
    if args.graph:
        return main_graph(args, be, fun, fun_args, config, dtype)

    def step():
        return fun(*fun_args)

    # warm-up, then PROBE_STEPS steps with every launch timed (stream kept busy ahead of each step) to find
    # the kernel that dominates the step and to report every kernel's average duration
    PROBE_STEPS = 5
    for _ in range(max(3, args.warmup)):  # (three: a recurring elementwise program is compiled at its third sighting)
        step()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(2):
        step()
    be.sync()
    host_ms = (time.perf_counter() - t0) / 2 * 1e3
    ahead = HeadStart()
    with _lib.KernelTimer() as probe:
        for _ in range(PROBE_STEPS):
            be.sync()
            ahead(1.5 * host_ms + 0.2)
            step()
    per_kernel = probe.summary()
    dominant = max(per_kernel, key=lambda k: per_kernel[k]["ms"])
    dom_key = per_kernel[dominant]["key"]
    dom_launches = max(1, per_kernel[dominant]["launches"] // PROBE_STEPS)

    # timed region: K steps bracketed by synchronise; only the dominant kernel carries events, and only on every
    # fourth of its launches (a pair costs the host about 7 us and delays the launch behind it: on the 140 us step
    # of the headline workload, events on every launch took 15-20 us per step)
    be.sync()
    every = max(4, dom_launches // 4)  # (a kernel launched hundreds of times per step carries about four pairs per step)
    with _lib.KernelTimer(only={dom_key}, events=2 * args.steps * dom_launches, every=every) as kt:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        be.sync()
        elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    # (kernels that share a launch key carry events in turn: a label launched once per step may have had none)
    dom_eager = kt.summary().get(dominant, {"avg_ms": None, "launches": 0})
    # the same K steps again, each behind a busy stream: the events bracket GPU execution only
    with _lib.KernelTimer(only={dom_key}, events=2 * args.steps * dom_launches) as kt:
        for _ in range(args.steps):
            be.sync()
            ahead(1.5 * ms_per_step + 0.2)
            step()
        be.sync()
    dom = kt.summary()[dominant]
    overhead_ms = event_pair_overhead_ms(ahead)
    dom["avg_ms"] = max(dom["avg_ms"] - overhead_ms, 1e-6)
    if dominant.startswith(("gemm_", "correlate")):
        achieved = dom["avg_flops"] / (dom["avg_ms"] * 1e-3) / 1e12
        # the window contraction runs on the vector ALUs, whose published fp32 peak equals the MFMA one
        roofline = {"bound": "mfma" if dominant.startswith("gemm") else "valu", "kernel": dominant, "achieved": achieved, "peak": MFMA_F32_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": achieved / MFMA_F32_PEAK_TFLOPS, "traffic": None,
                    "algorithmic_flops_per_launch": dom["avg_flops"]}
    else:
        achieved = dom["avg_bytes"] / (dom["avg_ms"] * 1e-3) / 1e9
        traffic, source = measured_traffic(dominant) if args.workload == "bcast" else (None, None)
        roofline = {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": source,
                    "algorithmic_bytes_per_launch": dom["avg_bytes"]}
    roofline["avg_launch_ms"] = dom["avg_ms"]
    if dom.get("avg_call_ms", 0.0) > dom["avg_ms"] + overhead_ms + 1e-4:
        # the entry point launches this kernel and then a small one that adds up its partial results; events around the
        # call would bracket both (48 us here, of which the finishing kernel is 4), so the library records the pair itself,
        # around the first kernel (agmi_probe_arm)
        roofline["event_pair"] = ("recorded by the library around this kernel alone (agmi_probe_arm): the entry point launches "
                                  "a second, small kernel that adds up partial sums, which a pair around the call would include")
    roofline["avg_launch_ms_event_pair"] = dom["avg_ms"] + overhead_ms
    roofline["event_pair_overhead_ms"] = overhead_ms
    roofline["avg_launch_ms_in_timed_region"] = dom_eager["avg_ms"]
    roofline["launches_timed"] = dom["launches"]
    roofline["launches_timed_in_timed_region"] = dom_eager["launches"]
    roofline["timing"] = ("HIP events on the launch stream around every launch of this kernel over `steps` steps, the stream "
                          "kept busy ahead of each step so that the pair brackets GPU execution only; the pair's own cost "
                          "(measured live: 2 x pair around one 64 MiB fill - pair around two) is subtracted; "
                          "avg_launch_ms_in_timed_region comes from events around every fourth launch (of a kernel launched many times per step: about four launches per step) inside the timed region, "
                          "where the host sets the pace and the figure includes what the pair itself adds")

    result = {
        "metric": "grad evals/sec",
        "value": args.steps / elapsed,
        "unit": "grad evals/sec",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": config,
        "roofline": roofline,
        # (averages over the probe steps, the event pair's own cost subtracted; one row per kernel AND shape, with
        # the algorithmic bytes / flops of one launch, so that every rate can be recomputed from the row)
        "kernels_per_step": {name: priced(r, PROBE_STEPS, overhead_ms)
                             for name, r in sorted(per_kernel.items(), key=lambda kv: -kv[1]["ms"])},
    }

    if args.calibrate_copy:
        import numpy as onp

        from autograd_amd._lib import Op
        from autograd_amd.numpy import devarray as D

        ref = D.zeros((8192, 4096), onp.float32)
        for _ in range(5):
            D.map_op(Op.COPY, ref.dtype, ref)
        be.sync()
    # the same evaluation recorded once and replayed as a HIP graph (autograd_amd.capture): same kernels,
    # no per-step Python tracing; reported beside the eager figure, never as `value`
    rate = graph_rate(fun, fun_args, be.sync, args.steps)
    result["graph_replay"] = {"value": rate, "unit": "grad evals/sec", "ms_per_step": 1e3 / rate}
    if args.workload == "bcast":
        # the whole evaluation against its compulsory traffic: A read once, dA written once, the vectors
        compulsory = 2 * 8192 * 4096 * 4 + 2 * (8192 + 4096) * 4
        roofline["end_to_end"] = dict(end_to_end(compulsory, result["value"]),
                                      graph_replay=end_to_end(compulsory, rate),
                                      what="inputs read once + results written once per evaluation, over the time of one "
                                           "evaluation (eager: `value`; graph_replay: the recorded evaluation replayed)")
    if not args.no_extras and args.workload == "bcast":
        result["extras"] = extras(be)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.cpu_seconds)
        if "extras" in result:
            result["extras"]["cpu_baselines"] = cpu_baseline_contractions(args.cpu_seconds)
    print(json.dumps(result))


def main_graph(args, be, fun, fun_args, config, dtype):
    """--graph: the step is one replay of the workload recorded as a HIP graph (no per-kernel events:
    nothing is launched from the host but the graph)."""
    import autograd_amd as ag

    graphed = ag.capture(fun, *fun_args)
    sec = time_steps(lambda: graphed(*fun_args), be.sync, args.steps, max(1, args.warmup))
    config = dict(config, execution="HIP graph replay of the recorded evaluation")
    print(json.dumps({
        "metric": "grad evals/sec", "value": 1.0 / sec, "unit": "grad evals/sec", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": sec * 1e3, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": config, "roofline": None,
        "cpu_baseline": None,
    }))


def graph_rate(fun, args, sync, steps):
    """grad evals/sec of ``fun(*args)`` replayed from a HIP graph; the graph is dropped afterwards."""
    import autograd_amd as ag

    graphed = ag.capture(fun, *args)
    sec = time_steps(lambda: graphed(*args), sync, steps, 2)
    del graphed
    return 1.0 / sec


def extras(be):
    """The other workloads (grad evals/sec each) and the MLP contraction rate; short runs."""
    from autograd_amd import _lib, configs

    out = {}
    # config 1: elementwise tanh derivatives, f64
    x = be.put(configs.tanh_inputs()["x"])
    prog = configs.tanh_program(be)
    for k in ("d1", "d2", "d3"):
        ms = time_steps(lambda: prog[k](x), be.sync, 40, 5) * 1e3
        out[f"tanh_{k}_evals_per_sec"] = 1e3 / ms
        out[f"tanh_{k}_graph_evals_per_sec"] = graph_rate(prog[k], (x,), be.sync, 40)
    # config 3: MLP gradient, f32; MFMA rate over the GEMMs whose dimensions are all >= 784
    inp = configs.mlp_inputs()
    params3 = configs.tree_map(be.put, inp["params"])
    X3, T3 = be.put(inp["X"]), be.put(inp["T"])
    g3 = configs.mlp_program(be)["grad"]
    ms = time_steps(lambda: g3(params3, X3, T3), be.sync, 20, 3) * 1e3
    out["mlp_grad_evals_per_sec"] = 1e3 / ms
    out["mlp_grad_graph_evals_per_sec"] = graph_rate(g3, (params3, X3, T3), be.sync, 20)
    ahead = HeadStart()
    with _lib.KernelTimer(only={("gemm",)}) as kt:
        for _ in range(5):
            be.sync()
            ahead(1.5 * ms + 0.2)  # the five big contractions then run back to back with their neighbours
            g3(params3, X3, T3)
    be.sync()
    pair_ms = event_pair_overhead_ms(ahead)
    gemm_ms, gemm_flops, worst = 0.0, 0.0, None
    for name, key, ev0, ev1, nbytes, flops, _probe in kt.records:
        if flops >= 2.0 * 784 * 1024 * 1024:  # skip the three GEMMs with a 10-wide dimension (memory-bound)
            t = max(ev0.elapsed_time(ev1) - pair_ms, 1e-6)
            gemm_flops += flops
            gemm_ms += t
            rate = flops / (t * 1e-3) / 1e12
            worst = rate if worst is None else min(worst, rate)
    tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12 if gemm_ms else 0.0
    out["mlp_gemm"] = {"bound": "mfma", "achieved": tflops, "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s",
                       "frac": tflops / MFMA_F32_PEAK_TFLOPS, "gemms_timed": 5 * 5, "slowest_single_launch_TFLOPs": worst,
                       "event_pair_overhead_ms": pair_ms,
                       "timing": "HIP events around each contraction, stream kept busy ahead of each evaluation, the event "
                                 "pair's own cost (measured live) subtracted"}
    del ahead
    # config 4: RNN, f32
    inp = configs.rnn_inputs()
    params = configs.tree_map(be.put, inp["params"])
    xs, ts = be.put(inp["inputs"]), be.put(inp["targets"])
    g4 = configs.rnn_program(be)["grad"]
    ms = time_steps(lambda: g4(params, xs, ts), be.sync, 20, 3) * 1e3
    out["rnn_grad_evals_per_sec"] = 1e3 / ms
    out["rnn_grad_graph_evals_per_sec"] = graph_rate(g4, (params, xs, ts), be.sync, 5)
    # config 5: Rosenbrock HVP, f64
    inp = configs.rosen_inputs()
    x5, v5 = be.put(inp["x"]), be.put(inp["v"])
    p5 = configs.rosen_program(be)
    ms = time_steps(lambda: p5["hvp_rev"](x5, v5), be.sync, 30, 5) * 1e3
    out["rosen_hvp_rev_evals_per_sec"] = 1e3 / ms
    out["rosen_hvp_rev_graph_evals_per_sec"] = graph_rate(p5["hvp_rev"], (x5, v5), be.sync, 30)
    ms = time_steps(lambda: p5["hvp_fwd"](x5, v5), be.sync, 30, 5) * 1e3
    out["rosen_hvp_fwd_evals_per_sec"] = 1e3 / ms
    out["rosen_hvp_fwd_graph_evals_per_sec"] = graph_rate(p5["hvp_fwd"], (x5, v5), be.sync, 30)
    # training-loop residency: one fused Adam update of a flat 2^24-element float64 parameter vector
    # (reads x, g, m, v; writes m, v, x: 56 bytes per element), and whole MLP training steps
    # (gradient + flatten + update, nothing leaves HBM)
    import numpy as onp

    from autograd_amd._lib import OPT_ADAM
    from autograd_amd.misc.optimizers import adam
    from autograd_amd.numpy import devarray as D

    # what this part streams on cold data: (8192,4096) f32 buffers in rotation (1 GiB of sources, far more than the
    # 256 MB last-level cache holds), a plain copy (read + write), a row sum (read only) and a fill (write only)
    from autograd_amd._lib import Op

    src = [D.zeros((8192, 4096), onp.float32) for _ in range(8)]
    dst = [D.empty((8192, 4096), onp.float32) for _ in range(8)]
    nbytes = 8192 * 4096 * 4
    turn = [0]

    def rotate(fn):
        def step():
            turn[0] += 1
            fn(turn[0] % 8)
        return step

    sec = time_steps(rotate(lambda i: D.map_op(Op.COPY, src[0].dtype, src[i], out=dst[i])), be.sync, 40, 8)
    ceil_copy = 2 * nbytes / sec / 1e9
    sec = time_steps(rotate(lambda i: be.np.sum(src[i], axis=1)), be.sync, 40, 8)
    ceil_read = nbytes / sec / 1e9
    sec = time_steps(rotate(lambda i: _lib.fill(_lib.DTYPE_CODE[dst[0].dtype], dst[i]._t, 1.0)), be.sync, 40, 8)
    out["stream_ceiling_GBps"] = {"copy": ceil_copy, "read": ceil_read, "write": nbytes / sec / 1e9}
    del src, dst
    n = 1 << 24
    xs = [D.zeros((n,), onp.float64) for _ in range(5)]
    hyper = (0.1, 0.9, 0.001, 0.999, 0.5, 0.5, 0.001, 1e-8)
    sec = time_steps(lambda: _lib.optimizer_step(OPT_ADAM, xs[0]._t, xs[1]._t, xs[2]._t, xs[3]._t, xs[4]._t, hyper),
                     be.sync, 20, 3)
    out["adam_update_GBps"] = 56.0 * n / sec / 1e9
    del xs
    steps = 20
    t0 = time.perf_counter()
    adam(lambda p, i: g3(p, X3, T3), params3, num_iters=steps)
    be.sync()
    out["mlp_adam_training_steps_per_sec"] = steps / (time.perf_counter() - t0)
    # the same loop with the gradient replayed from a HIP graph (parameters are copied into the recorded
    # input buffers every step, the update stays a separate kernel)
    import autograd_amd as ag

    graphed = ag.capture(g3, params3, X3, T3)
    adam(lambda p, i: graphed(p, X3, T3), params3, num_iters=3)
    be.sync()
    t0 = time.perf_counter()
    adam(lambda p, i: graphed(p, X3, T3), params3, num_iters=steps)
    be.sync()
    out["mlp_adam_training_graph_steps_per_sec"] = steps / (time.perf_counter() - t0)
    del graphed
    # every workload against its compulsory bytes (inputs read once + results written once): what the per-kernel
    # figures do not show is how many passes an evaluation makes
    n1, n5 = 4194304, 1 << 24
    out["end_to_end"] = {
        **{f"tanh_{k}": {"eager": end_to_end(16 * n1, out[f"tanh_{k}_evals_per_sec"]),
                         "graph_replay": end_to_end(16 * n1, out[f"tanh_{k}_graph_evals_per_sec"])} for k in ("d1", "d2", "d3")},
        **{f"rosen_{k}": {"eager": end_to_end(24 * n5, out[f"rosen_{k}_evals_per_sec"]),
                          "graph_replay": end_to_end(24 * n5, out[f"rosen_{k}_graph_evals_per_sec"])} for k in ("hvp_rev", "hvp_fwd")},
        "mlp": {"flops_per_eval": 9.794e9,
                "eager_frac_of_mfma_peak": 9.794e9 * out["mlp_grad_evals_per_sec"] / 1e12 / MFMA_F32_PEAK_TFLOPS,
                "graph_replay_frac_of_mfma_peak": 9.794e9 * out["mlp_grad_graph_evals_per_sec"] / 1e12 / MFMA_F32_PEAK_TFLOPS},
        "rnn": {"flops_per_eval": 38.8e9,
                "eager_frac_of_mfma_peak": 38.8e9 * out["rnn_grad_evals_per_sec"] / 1e12 / MFMA_F32_PEAK_TFLOPS,
                "graph_replay_frac_of_mfma_peak": 38.8e9 * out["rnn_grad_graph_evals_per_sec"] / 1e12 / MFMA_F32_PEAK_TFLOPS},
    }
    return out


if __name__ == "__main__":
    main()
