#!/usr/bin/env python3
"""Gradient throughput of the gfx950 backend on the synthetic configs.

One "step" = one full forward + reverse gradient of a config's objective on one
batch of synthetic input that is already resident in HBM (uploads happen before
the timed region).  `ms_per_step` is throughput: the K timed steps are queued
back to back and the host waits once after the last; `ms_per_step_synced` has
the host wait for every step and read the loss back, the equivalent of the
reference forcing every gradient leaf, bench/ConvVjpBench.hs:174-175.  As the
reference builds its gradient artifact once and times its evaluation
(bench/ConvVjpBench.hs:254-257), the gradient program is recorded once into a
device graph and a step launches that graph; `ms_per_step_eager` is the same
program submitted operation by operation from Python, and --eager times that.

Prints ONE JSON line.  `value` is gradient samples/s of the headline config
(the CNN); the other configs ride along under "configs".  "roofline" prices the
dominant kernel of the headline config: its ALGORITHMIC bytes (or flops) per
launch divided by its average launch duration, measured here with HIP events
on the library's stream.  "cpu_baseline" is the CPU checker (a single-threaded
dense restatement of the reference's array semantics) timed on a bounded
sample of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f64": 78.6, "f32": 157.3}
MFMA_KERNELS = ("gemm_f64", "gemm_f32")   # kernel families priced against the matrix-core peak
DTYPE_NAME = {0: "f64", 1: "f32"}
# CPU-baseline sample sizes (batch) chosen so the checker runs ~10-30 s in total
CPU_SAMPLE = {"c0": dict(n=1024, m=1024), "c1": dict(batch=250), "c2": dict(batch=64),
              "c3": dict(batch=12), "c4": dict(batch=64)}


def array_ctx(capi, host):
    """The array-library context behind a host-layer context, as a capi.Ctx."""
    ctx = capi.Ctx.__new__(capi.Ctx)
    ctx.lib = capi.Lib()
    ctx.h = C.c_void_p(host.dll.hh_array_ctx(host.h))
    return ctx


def time_steps(host, wl, ps, ds, steps, warmup):
    for _ in range(warmup):
        wl.gradient(host, ps, ds)
        host.sync()
    host.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss, grads = wl.gradient(host, ps, ds)
    host.sync()
    dt = time.perf_counter() - t0
    return dt / steps, float(loss.numpy())


def time_graph(host, wl, ps, ds, steps, warmup):
    """The same gradient recorded once (the reference builds its gradient
    artifact once, outside the timed region) and launched per step."""
    graph, (loss, grads) = host.capture(lambda: wl.gradient(host, ps, ds))
    try:
        for _ in range(warmup):
            graph.launch()
            host.sync()
        host.sync()
        t0 = time.perf_counter()
        for _ in range(steps):       # the steps queue up on the one stream; the host waits once, after the last
            graph.launch()
        host.sync()
        dt = time.perf_counter() - t0
        # the same with the host waiting for every step and reading the loss back, the way the reference's
        # benchmark forces every gradient before the next one starts (bench/ConvVjpBench.hs:174-175)
        t1 = time.perf_counter()
        for _ in range(steps):
            graph.launch()
            last = float(loss.numpy())
        dt_synced = time.perf_counter() - t1
        return dt / steps, last, dt_synced / steps
    finally:
        graph.free()


def time_train_graph(pkg, host, wl, steps, warmup):
    """One training step -- gradient, Adam update of every parameter array, new
    parameters and moments written back where the next launch reads them --
    recorded once and launched per step: the parameters never leave the device."""
    import numpy as np
    OPT = pkg.optimizer
    ps, ds = wl.upload(host)
    args = OPT.defaultArgsAdam
    ms = [host.concrete(np.zeros_like(x)) for x in wl.params]
    vs = [host.concrete(np.zeros_like(x)) for x in wl.params]
    alphat = OPT.adamStepSize(host, ps[0].dtype, args, 1)

    def step():
        loss, grads = wl.gradient(host, ps, ds)
        mn, vn, pn = OPT.adamApply(args, alphat, ms, vs, ps, grads)
        for dst, src in zip(ms + vs + ps, mn + vn + pn):
            dst.assign(src)
        return loss

    step()
    host.sync()
    graph, loss = host.capture(step)
    try:
        t = 1
        for _ in range(warmup):
            t += 1
            alphat.overwrite(OPT.adamStepSize(host, ps[0].dtype, args, t).numpy())
            graph.launch()
            host.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            t += 1
            alphat.overwrite(OPT.adamStepSize(host, ps[0].dtype, args, t).numpy())
            graph.launch()
            host.sync()
        dt = time.perf_counter() - t0
        return dt / steps
    finally:
        graph.free()


def profile(capi, host, wl, ps, ds, reps=10):
    """Per-launch HIP-event timing by the library, one label per kernel and
    problem shape: {label: (launches, ms, bytes, flops)} per gradient.  The
    gradients are submitted one after another without waiting in between, as
    in the timed region (a device left idle between steps clocks down, and its
    kernels then take a few per cent longer)."""
    actx = array_ctx(capi, host)
    for _ in range(2):
        wl.gradient(host, ps, ds)
    actx.check(actx.lib.profile_enable(actx.h, 2))
    for _ in range(reps):
        wl.gradient(host, ps, ds)
    host.sync()
    rep = actx.profile_report()
    actx.check(actx.lib.profile_enable(actx.h, 0))
    return {k: (v[0] / reps, v[1] / reps, v[2] / reps, v[3] / reps) for k, v in rep.items()}


def family(label):
    return label.split("[", 1)[0]


def measured_traffic(label):
    """HBM bytes per launch of a kernel, where a counter run has measured them
    (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain copy; the
    figures and the commands are in profiles/)."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if not os.path.exists(path):
        return None
    table = json.load(open(path))
    val = table.get(label)      # the exact label only: a changed kernel or shape has no figure until it is measured again
    return None if label.startswith("_") else val


def roofline_of(rep, dtype_name):
    """Prices the kernel (one label = one kernel at one problem shape) with the
    largest share of device time."""
    if not rep:
        return None, {}
    name = max(rep, key=lambda k: rep[k][1])
    launches, ms, by, fl = rep[name]
    if launches == 0 or ms <= 0:
        return None, {}
    avg_ms = ms / launches
    if family(name) in MFMA_KERNELS:
        ach = fl / launches / (avg_ms * 1e-3) / 1e12
        peak = MFMA_PEAK_TFLOPS[dtype_name]
        roof = {"bound": "mfma", "achieved": ach, "peak": peak, "unit": "TFLOP/s", "frac": ach / peak,
                "algorithmic_gflop_per_launch": fl / launches / 1e9}
    else:
        ach = by / launches / (avg_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": ach / HBM_PEAK_GBS,
                "algorithmic_mb_per_launch": by / launches / 1e6}
    roof.update({"kernel": name, "launches_per_step": launches, "avg_launch_ms": avg_ms,
                 "share_of_device_time": ms / sum(v[1] for v in rep.values()), "traffic": measured_traffic(name),
                 "traffic_source": "profiles/hbm_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this kernel, committed with the build (not measured in this run)"})
    fams = {}
    for k, v in rep.items():
        fams[family(k)] = fams.get(family(k), 0.0) + v[1]
    shares = {k: round(v, 4) for k, v in sorted(fams.items(), key=lambda kv: -kv[1])}
    return roof, shares


def kernel_table(rep, dtype_name, top=14):
    """The launches of one gradient by label (one label = one kernel at one problem shape), largest share first:
    launches, average microseconds, and the rate on the label's own algorithmic flops / bytes."""
    rows = []
    for name, (launches, ms, by, fl) in sorted(rep.items(), key=lambda kv: -kv[1][1])[:top]:
        if launches <= 0 or ms <= 0:
            continue
        row = {"kernel": name, "launches": launches, "avg_us": ms / launches * 1e3}
        if family(name) in MFMA_KERNELS:
            row["tflops"] = fl / ms / 1e9
            row["frac_of_mfma_peak"] = row["tflops"] / MFMA_PEAK_TFLOPS[dtype_name]
        elif by > 0:
            row["gbs"] = by / ms / 1e6
            row["frac_of_hbm_peak"] = row["gbs"] / HBM_PEAK_GBS
        rows.append(row)
    return rows


def cpu_baseline(pkg, key, mk):
    capi, H = pkg.capi, pkg.hostapi
    if not os.path.exists(entry.ORACLE_LIB):
        return None
    host = H.Host(capi.Lib(entry.ORACLE_LIB, "horc_"))
    wl = mk(**CPU_SAMPLE[key])
    ps, ds = wl.upload(host)
    t0 = time.perf_counter()
    n = 0
    while True:
        wl.gradient(host, ps, ds)
        n += 1
        if time.perf_counter() - t0 > 8.0 or n >= 3:
            break
    dt = (time.perf_counter() - t0) / n
    return {"value": wl.batch / dt, "unit": "samples/s", "cores": 1, "host_cores": os.cpu_count(), "kind": "port",
            "sample": f"{wl.name} at {CPU_SAMPLE[key]} ({wl.batch} samples per gradient, {n} gradients, {dt:.3f} s each)"}


def index_micro(capi, which, steps, warmup):
    """One index kernel at a stated size, through the array-level entry points.

    gather_units: 100 MB of 1 KiB slices picked by a data-dependent index vector (the general gather, 16-byte units).
    scatter_sorted: 12.5 M single elements added into 3.1 M cells, four to a cell as in the adjoint of 2 x 2 pooling
    over [1000, 16, 28, 28], the cells given as data (the general path: sort by destination, add each run in order).
    Algorithmic bytes: what is read plus what is written, the index vector included."""
    import numpy as np
    ctx = capi.Lib().context(0)
    rng = np.random.default_rng(3)
    if which == "gather_units":
        rows, width = 100_000, 128                    # 1 KiB slices of doubles
        src = ctx.upload(rng.standard_normal((rows, width)))
        ix = [ctx.upload(rng.integers(0, rows, rows).astype(np.int64))]
        call = lambda: ctx.gather(src, ix, [rows])
        alg = 2.0 * rows * width * 8 + 8.0 * rows
        what = "gather of 100000 slices of 1 KiB from [100000, 128] f64 by an index vector"
    else:
        b, c, h, w = 1000, 16, 28, 28
        m = b * c * h * w
        pos = np.arange(m, dtype=np.int64).reshape(b, c, h // 2, 2, w // 2, 2)
        cells_np = np.broadcast_to(np.arange(m // 4, dtype=np.int64).reshape(b, c, h // 2, 1, w // 2, 1), pos.shape).reshape(-1).copy()
        src = ctx.upload(rng.standard_normal(m))
        ix = [ctx.upload(cells_np)]
        call = lambda: ctx.scatter_add(src, ix, 1, [m // 4])
        alg = 8.0 * m + 8.0 * m + 8.0 * (m // 4)
        what = "scatter-add of 12544000 f64 into 3136000 cells (four to a cell), cells given as an index vector"
    for _ in range(max(1, warmup)):
        o = call()
        del o
    ctx.sync()
    ctx.profile(2)
    t0 = time.perf_counter()
    for _ in range(steps):
        o = call()
        del o
    ctx.sync()
    sec = (time.perf_counter() - t0) / steps
    rep = ctx.profile_report()
    ctx.profile(0)
    kernels = {k: {"launches_per_call": v[0] / steps, "avg_us": v[1] / v[0] * 1e3} for k, v in rep.items() if v[0]}
    return {"micro": which, "what": what, "ms_per_call": sec * 1e3, "algorithmic_mb": alg / 1e6, "achieved_gbs": alg / sec / 1e9,
            "frac_of_hbm_peak": alg / sec / 1e9 / HBM_PEAK_GBS, "kernels": kernels}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="c3", help="headline config: c0..c4")
    ap.add_argument("--only", action="store_true", help="measure the headline config only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--eager", action="store_true", help="time op-by-op submission instead of the recorded graph")
    ap.add_argument("--train", action="store_true",
                    help="also time a recorded training step (gradient + Adam + write-back) of the headline config")
    ap.add_argument("--calibrate-mfma", action="store_true",
                    help="time loops of single matrix-core instructions (the ceiling of the product kernels) and exit")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run plain dense copies of 1 GiB (for scaling hardware traffic counters) and exit")
    ap.add_argument("--micro", choices=["gather_units", "scatter_sorted", "riders"],
                    help="time one index kernel at a stated size (its algorithmic bytes over its launch time) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, no sharding)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    pkg = entry.load_package()
    capi, H, W = pkg.capi, pkg.hostapi, pkg.workloads
    if args.calibrate_mfma:
        ctx = capi.Lib().context(0)
        out = {}
        names = ["v_mfma_f64_16x16x4_f64", "v_mfma_f64_4x4x4_4b_f64", "v_mfma_f32_16x16x4_f32", "v_mfma_f32_32x32x2_f32",
                 "v_mfma_f64_16x16x4_f64 fed from LDS, 1 wavefront per SIMD", "v_mfma_f64_16x16x4_f64 fed from LDS, 2 wavefronts per SIMD",
                 "v_mfma_f64_16x16x4_f64 fed from LDS, 4 wavefronts per SIMD"]
        for variant, name in enumerate(names):
            best = 0.0
            for _ in range(3):
                t = C.c_double()
                ctx.check(ctx.lib.mfma_probe(ctx.h, variant, 20000, C.byref(t)))
                best = max(best, t.value)
            out[name] = {"sustained_tflops": best, "nominal_peak_tflops": MFMA_PEAK_TFLOPS["f64" if "f64_" in name[:12] else "f32"],
                         "fraction_of_nominal": best / MFMA_PEAK_TFLOPS["f64" if "f64_" in name[:12] else "f32"]}
        print(json.dumps({"calibration": "loops of one MFMA instruction, 20000 iterations: operands in registers, 16 wavefronts per CU, 4 (8, 2) independent accumulators; and fed from LDS as a 64 x 64 tile of four wavefronts (2 x 2 blocks each, a barrier per 16 k)", "instructions": out}))
        return
    if args.calibrate_copy:
        import numpy as np
        ctx = capi.Lib().context(0)
        src = ctx.upload(np.zeros(1 << 27, np.float64))       # 1 GiB
        for _ in range(5):
            dst = src.materialize()                            # k_copy: reads 1 GiB, writes 1 GiB
            del dst
        ctx.sync()
        print(json.dumps({"calibration": "5 dense copies", "bytes_read_per_copy": 1 << 30, "bytes_written_per_copy": 1 << 30}))
        return
    if args.micro in ("gather_units", "scatter_sorted"):
        print(json.dumps(index_micro(capi, args.micro, args.steps, args.warmup)))
        return
    host = H.Host()      # raises when the HIP library is missing or no device is usable
    if args.micro == "riders":
        out = {}
        for key, make in W.RIDERS.items():
            if key == "c3_artifact_form":
                continue
            wl = make()
            ps, ds = wl.upload(host)
            eager_sec, loss = time_steps(host, wl, ps, ds, args.steps, args.warmup)
            rep = profile(capi, host, wl, ps, ds)
            out[key] = {"workload": wl.name, "ms_per_call_eager": eager_sec * 1e3, "algorithmic_mb": wl.bytes / 1e6, "kernels": kernel_table(rep, DTYPE_NAME[wl.dtype])}
        print(json.dumps({"micro": "riders", "results": out}))
        return

    keys = [args.workload] if args.only else [args.workload] + [k for k in W.CONFIGS if k != args.workload]
    results = {}
    for key in keys:
        wl = W.CONFIGS[key]()
        ps, ds = wl.upload(host)
        host.sync()
        eager_sec, loss = time_steps(host, wl, ps, ds, args.steps, args.warmup)
        sec, graph_loss, synced_sec = (eager_sec, loss, None) if args.eager else time_graph(host, wl, ps, ds, args.steps, args.warmup)
        if graph_loss != loss:
            raise SystemExit(f"bench.py: {key}: the recorded program computed {graph_loss!r}, the eager one {loss!r}")
        rep = profile(capi, host, wl, ps, ds)
        dn = DTYPE_NAME[wl.dtype]
        roof, shares = roofline_of(rep, dn)
        dev_ms = sum(v[1] for v in rep.values())
        gemm_ms = sum(v[1] for k, v in rep.items() if family(k) in MFMA_KERNELS)
        gemm_fl = sum(v[3] for k, v in rep.items() if family(k) in MFMA_KERNELS)
        results[key] = {"workload": wl.name, "dtype": dn, "batch": wl.batch, "ms_per_step": sec * 1e3,
                        "samples_per_s": wl.batch / sec, "gradients_per_s": 1.0 / sec, "loss": loss,
                        "ms_per_step_synced": None if synced_sec is None else synced_sec * 1e3,
                        "ms_per_step_eager": eager_sec * 1e3, "execution": "eager" if args.eager else "recorded graph, one launch per step",
                        "launches_per_step": sum(v[0] for v in rep.values()),
                        "device_ms_per_step": dev_ms, "algorithmic_gflop": wl.flops / 1e9,
                        "achieved_tflops": wl.flops / sec / 1e12, "roofline": roof, "kernel_ms": shares,
                        "kernels": kernel_table(rep, dn),
                        "all_matrix_products": {"ms": gemm_ms, "tflops": gemm_fl / gemm_ms / 1e9 if gemm_ms > 0 else None,
                                                "frac_of_peak": gemm_fl / gemm_ms / 1e9 / MFMA_PEAK_TFLOPS[dn] if gemm_ms > 0 else None}}
        if wl.bytes:
            results[key]["algorithmic_gb"] = wl.bytes / 1e9
            results[key]["achieved_gbs_whole_step"] = wl.bytes / sec / 1e9
        del ps, ds

    # the same work written another way (the reference's derived form of relu and pooling): timed beside the configs
    riders = {}
    if not args.only:
        for key, make in getattr(W, "RIDERS", {}).items():
            wl = make()
            ps, ds = wl.upload(host)
            host.sync()
            eager_sec, loss = time_steps(host, wl, ps, ds, args.steps, args.warmup)
            sec, graph_loss, _ = (eager_sec, loss, None) if args.eager else time_graph(host, wl, ps, ds, args.steps, args.warmup)
            if graph_loss != loss:
                raise SystemExit(f"bench.py: {key}: the recorded program computed {graph_loss!r}, the eager one {loss!r}")
            riders[key] = {"workload": wl.name, "batch": wl.batch, "ms_per_step": sec * 1e3, "ms_per_step_eager": eager_sec * 1e3, "loss": loss}
            if wl.bytes:      # a chain of a few microseconds, timed by itself: launching a recorded graph costs more than its one or two kernels
                best = min(sec, eager_sec)
                riders[key]["us_per_call"] = best * 1e6
                riders[key]["algorithmic_mb"] = wl.bytes / 1e6
                riders[key]["achieved_gbs"] = wl.bytes / best / 1e9
            if "c3" in results and key.startswith("c3"):
                riders[key]["ms_per_step_over_c3"] = sec * 1e3 / results["c3"]["ms_per_step"]
                riders[key]["loss_equals_c3"] = loss == results["c3"]["loss"]
            del ps, ds

    head = results[args.workload]
    train = None
    if args.train:
        wl = W.CONFIGS[args.workload]()
        sec = time_train_graph(pkg, host, wl, args.steps, args.warmup)
        train = {"ms_per_step": sec * 1e3, "samples_per_s": wl.batch / sec, "optimizer": "Adam, reference defaults",
                 "execution": "recorded graph: gradient, update and write-back in one launch"}
    cpu = None if args.no_cpu else cpu_baseline(pkg, args.workload, W.CONFIGS[args.workload])
    line = {
        "metric": "gradient samples/sec at 1 GPU", "value": head["samples_per_s"], "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "ms_per_step_synced": head["ms_per_step_synced"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": head["dtype"],
        "data": "synthetic",
        "config": {"workload": f"{head['workload']}: forward + reverse gradient, batch {head['batch']}, {head['dtype']}"},
        "roofline": head["roofline"], "cpu_baseline": cpu,
        "configs": {k: v for k, v in results.items() if k != args.workload},
        "headline_detail": {k: v for k, v in head.items() if k != "roofline"},
    }
    if riders:
        line["riders"] = riders
    if train:
        line["training_step"] = train
    print(json.dumps(line))


if __name__ == "__main__":
    main()
