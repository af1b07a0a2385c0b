#!/usr/bin/env python3
"""Benchmark of the weight-only-quantised GEMV hot path on one MI355X.

A step is one GEMV call (one pass of the hot path over one activation batch).  Operands are
synthetic, seeded, and already resident in HBM when the timed region starts; weight / scale /
zero buffers are rotated between calls so that more than the 256 MB Infinity Cache is
touched between two uses of the same buffer (cold-cache timing).

Prints ONE JSON line:
  value            whole-job algorithmic GB/s over the K timed steps (wall clock, launch gaps included)
  roofline         achieved = algorithmic bytes per launch / average kernel duration, measured with a
                   HIP event pair on the launch stream around the back-to-back launches of the timed
                   region (gaps between kernels count as kernel time); peak = 8000 GB/s
  cpu_baseline     the CPU oracle (a port of the reference's HOST_CHECK loop) timed on this host
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBS = 8000.0
MALL_BYTES = 256 << 20

# name -> (n_out, k, weight_bits, quant_op, group_size, m_batch, bias, x distribution, scale range, description)
WORKLOADS = {
    "ns": (4096, 4096, 4, 3, 128, 1, False, "uniform", (0.001, 0.02),
           "int4 group-128 scale+zero GEMV, M=1, N=K=4096"),
    "c1": (4096, 4096, 8, 1, 4096, 1, True, "uniform", (0.001, 0.01),
           "int8 per-column scale GEMV + bias, M=1, N=K=4096"),
    "c2": (4096, 4096, 4, 2, 128, 1, True, "uniform", (0.001, 0.02),
           "int4 group-128 scale-only GEMV + bias, M=1, N=K=4096"),
    "c3a": (11008, 4096, 4, 3, 128, 1, False, "normal", (0.001, 0.02),
            "int4 group-128 scale+zero GEMV, M=1, K=4096, N=11008"),
    "c3b": (4096, 11008, 4, 3, 128, 1, False, "normal", (0.001, 0.02),
            "int4 group-128 scale+zero GEMV, M=1, K=11008, N=4096"),
    "c4": (8192, 8192, 4, 3, 64, 1, True, "uniform", (0.001, 0.02),
           "int4 group-64 scale+zero GEMV + bias, N=K=8192"),
    "c5": (28672, 8192, 4, 3, 128, 1, False, "normal", (0.001, 0.02),
           "int4 group-128 scale+zero GEMV, M=1, K=8192, N=28672"),
    # not one of the benchmark configurations: a vocabulary projection, the longest launch a decoder step has
    "vocab": (128256, 4096, 4, 3, 128, 1, False, "normal", (0.001, 0.02),
              "int4 group-128 scale+zero GEMV, M=1, K=4096, N=128256 (vocabulary projection)"),
}


# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch,
# averaged over the launches of `bench.py --workload <name> --launch stream`), scaled by what the same
# counters read for a plain 512 MiB device copy on the same box: FETCH_SIZE reads 262155.5 for 524288 KiB
# (factor 2.0), WRITE_SIZE reads 524288 (factor 1.0).  See profiles/.  name -> (fetch KiB raw, write KiB raw)
MEASURED_TRAFFIC_KIB = {"ns": (4472.0, 8.0), "c5": (61089.5, 56.0)}
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def measured_traffic_bytes(name, m_batch):
    if name not in MEASURED_TRAFFIC_KIB or m_batch != 1:
        return None
    fetch, write = MEASURED_TRAFFIC_KIB[name]
    return int((fetch * FETCH_SCALE + write * WRITE_SCALE) * 1024)


def algorithmic_bytes(n_out, k, bits, quant_op, group, m_batch, bias):
    groups = 1 if quant_op == 1 else k // group
    return (n_out * k * bits // 8 + groups * n_out * 2 * (2 if quant_op == 3 else 1) + (n_out * 2 if bias else 0)
            + m_batch * k * 2 + m_batch * n_out * 2)


class Workload:
    """Builds the rotating operand sets of one workload directly in HBM (torch is the allocator)."""

    def __init__(self, name, device, m_batch=None, seed=1234, min_sets=None, element="f16"):
        import numpy as np
        import torch
        import mixed_gemv_amd as mg

        self.element = element
        dt = torch.bfloat16 if element == "bf16" else torch.half   # activations, scales, zeros, bias, outputs

        (self.n_out, self.k, self.bits, self.quant_op, self.group, mb, self.has_bias, xdist, srange,
         self.description) = WORKLOADS[name]
        self.name = name
        self.m_batch = m_batch or mb
        self.bytes = algorithmic_bytes(self.n_out, self.k, self.bits, self.quant_op, self.group, self.m_batch,
                                       self.has_bias)
        groups = 1 if self.quant_op == 1 else self.k // self.group
        per_set = self.n_out * self.k * self.bits // 8 + 2 * groups * self.n_out * 2
        # enough sets that (sets - 1) * per_set exceeds the Infinity Cache plus the 8 x 4 MB L2s
        self.sets = max(8, -(-(MALL_BYTES + (32 << 20)) // per_set) + 1)
        if min_sets:
            self.sets = max(self.sets, min_sets)
        gen = torch.Generator(device="cpu").manual_seed(seed)
        qt = mg.QuantType.W4_A16 if self.bits == 4 else mg.QuantType.W8_A16
        self.raw0 = None
        self.w, self.s, self.z = [], [], []
        # All rotating sets live in ONE device allocation (256-byte aligned slices): large
        # contiguous mappings keep address-translation misses on cold buffers low.
        w_bytes = mg.preprocessed_size((self.k, self.n_out), qt)
        s_bytes = groups * self.n_out * 2
        align = lambda v: (v + 255) // 256 * 256  # noqa: E731
        set_bytes = align(w_bytes) + 2 * align(s_bytes)
        self.arena = torch.empty(set_bytes * self.sets, dtype=torch.uint8, device=device)

        def carve(offset, nbytes, dtype, shape):
            return self.arena[offset:offset + nbytes].view(dtype).view(shape)

        for i in range(self.sets):
            base = i * set_bytes
            # uniform random bytes == uniform int4 pairs in [-8, 7] (or int8 in [-128, 127])
            raw = torch.randint(0, 256, (self.n_out * self.k * self.bits // 8,), dtype=torch.uint8, generator=gen)
            if i == 0:
                self.raw0 = raw.numpy().copy()
            pre = mg.MixedGemvWeightPreprocessor.run(raw.numpy(), (self.k, self.n_out), mg.LayoutType.kColumnMajor, qt)
            w = carve(base, w_bytes, torch.uint8, (w_bytes,))
            w.copy_(torch.from_numpy(pre))
            self.w.append(w)
            sc = (torch.rand((groups, self.n_out), generator=gen) * (srange[1] - srange[0]) + srange[0]).to(dt)
            sdev = carve(base + align(w_bytes), s_bytes, dt, (groups, self.n_out))
            sdev.copy_(sc)
            self.s.append(sdev)
            if self.quant_op == 3:
                zz = (torch.rand((groups, self.n_out), generator=gen) * 0.1 - 0.05).to(dt)
                zdev = carve(base + align(w_bytes) + align(s_bytes), s_bytes, dt, (groups, self.n_out))
                zdev.copy_(zz)
                self.z.append(zdev)
            else:
                self.z.append(None)
        if xdist == "uniform":
            x = torch.rand((self.m_batch, self.k), generator=gen) * 2 - 1
        else:
            x = torch.randn((self.m_batch, self.k), generator=gen).clamp_(-4, 4)
        self.x = x.to(dt).to(device)
        self.bias = (torch.rand((self.n_out,), generator=gen) * 0.2 - 0.1).to(dt).to(device) if self.has_bias else None
        self.y = torch.zeros((self.m_batch, self.n_out), dtype=dt, device=device)
        self.np = np
        self.mg = mg

    def launch(self, i):
        if getattr(self, "batch", 0):
            return self.launch_batched(i)
        j = i % self.sets
        self.mg.device_gemv(self.w[j], self.x, self.s[j], self.z[j], self.bias, self.y, 1, self.n_out, self.m_batch,
                            self.k, self.group, self.quant_op, self.bits, element=self.element)

    def enable_batched(self, batch):
        """Later launches run `batch` consecutive buffer sets as ONE batched launch (the reference's
        batch_count / batch strides, gemv/device/gemv_adaptor.h:129-135): independent problems that
        share the activations."""
        import torch
        self.batch = batch
        self.set_stride = (self.w[1].data_ptr() - self.w[0].data_ptr()) if self.sets > 1 else 0
        self.y_batched = torch.zeros((batch, self.m_batch, self.n_out), dtype=self.y.dtype, device=self.y.device)

    def launch_batched(self, i):
        b = self.batch
        j = (i % (self.sets // b)) * b
        self.mg.device_gemv(self.w[j], self.x, self.s[j], self.z[j], self.bias, self.y_batched, b, self.n_out,
                            self.m_batch, self.k, self.group, self.quant_op, self.bits,
                            batch_strides=(self.set_stride, 0, self.set_stride // 2, 0, self.m_batch * self.n_out),
                            element=self.element)

    def host_operands(self, j=0):
        np = self.np
        return dict(
            w_raw=self.raw0 if j == 0 else None,
            x=self.x.cpu().numpy(), scale=self.s[j].cpu().numpy(),
            zero=self.z[j].cpu().numpy() if self.z[j] is not None else None,
            bias=self.bias.cpu().numpy() if self.bias is not None else None)


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


SPIN_UP_SECONDS = 0.06  # the clocks of an idle MI355X take ~20 ms of load to settle (measured: 30.7 -> 25.5 us)


def _capture(wl, first, count):
    """A HIP graph of `count` launches (steps first .. first+count-1): kernel nodes only."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(first, first + count):
                wl.launch(i)
    torch.cuda.current_stream().wait_stream(side)
    return graph


def time_workload(wl, steps, warmup, use_graph=False):
    """Runs at least `warmup` untimed steps (more if needed to bring an idle device up to its
    steady clocks), then times EXACTLY `steps` steps.  Returns (wall seconds, average kernel
    microseconds by a HIP event pair on the launch stream, steps, warm-up steps actually run)."""
    import torch
    main = rest = None
    if use_graph:
        # whole rotations of the buffer sets, at least 32 kernel nodes per replay so that the cost
        # of starting a replay is spread thin; a second graph holds the remainder so that the
        # timed region is exactly `steps` launches
        nodes = min(steps, wl.sets * max(1, -(-32 // wl.sets)))
        main = _capture(wl, 0, nodes)
        if steps % nodes:
            rest = _capture(wl, 0, steps % nodes)
    done = 0
    for i in range(warmup):
        wl.launch(i)
    done += warmup
    torch.cuda.synchronize()
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < SPIN_UP_SECONDS:
        if main is not None:
            main.replay()
            done += nodes
        else:
            for i in range(32):
                wl.launch(i)
            done += 32
        torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    if main is not None:
        for _ in range(steps // nodes):
            main.replay()
        if rest is not None:
            rest.replay()
    else:
        for i in range(steps):
            wl.launch(i)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e3 / steps, steps, done


def launch_floor_us(device):
    """Cadence of the smallest possible kernel (a one-element fill) replayed from a HIP graph like the
    timed steps: what one launch costs on this machine before it reads a single byte."""
    import torch
    cell = torch.zeros(1, dtype=torch.int32, device=device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(64):
                cell.fill_(1)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(20):
        graph.replay()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(100):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / 6400


def check_against_oracle(wl, rows=None):
    """GPU result of buffer set 0 against the CPU oracle on the first `rows` rows; also times
    the oracle single-threaded (the reference's HOST_CHECK loop has no threading)."""
    import numpy as np
    import torch
    import oracle as orc  # cpu_baseline leg: the checker, never the thing measured

    ops = wl.host_operands(0)
    rows = wl.n_out if rows is None else min(rows, wl.n_out)
    row_bytes = wl.k * wl.bits // 8
    w_rows = np.ascontiguousarray(ops["w_raw"][: rows * row_bytes])
    if wl.bits == 8:
        w_rows = w_rows.view(np.int8)
    scale = np.ascontiguousarray(ops["scale"][:, :rows])
    zero = np.ascontiguousarray(ops["zero"][:, :rows]) if ops["zero"] is not None else None
    bias = np.ascontiguousarray(ops["bias"][:rows]) if ops["bias"] is not None else None
    reps, elapsed, ref = 0, 0.0, None
    while reps < 2 or (elapsed < 8.0 and reps < 64):
        t0 = time.perf_counter()
        ref = orc.gemv(w_rows, ops["x"], scale, zero, bias, rows, wl.m_batch, wl.k, wl.group, wl.quant_op, wl.bits,
                       threads=1)
        elapsed += time.perf_counter() - t0
        reps += 1
    cpu_s = elapsed / reps
    wl.launch(0)
    torch.cuda.synchronize()
    got = wl.y.cpu().numpy()[:, :rows].astype(np.float64)
    r = ref.astype(np.float64)
    rms = float(np.sqrt(np.mean(r * r)))
    floor = max(rms * 2.0 ** -7, 2.0 ** -24)  # see tests/helpers.py:error_report for why 2^-7 * rms
    abs_err = np.abs(got - r)
    rel_err = abs_err / np.maximum(np.abs(r), floor)
    sample_bytes = algorithmic_bytes(rows, wl.k, wl.bits, wl.quant_op, wl.group, wl.m_batch, wl.has_bias)
    # the same loop with OpenMP over the rows, on every core the process may use
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, orc.max_threads()))
    t_all, r_all = 0.0, 0
    while r_all < 3 or (t_all < 2.0 and r_all < 200):
        t0 = time.perf_counter()
        orc.gemv(w_rows, ops["x"], scale, zero, bias, rows, wl.m_batch, wl.k, wl.group, wl.quant_op, wl.bits,
                 threads=cores)
        t_all += time.perf_counter() - t0
        r_all += 1
    # dequantised weights of buffer set 0, kernels' own dequantiser against the oracle's: must be identical
    dq_ref = orc.dequantize(w_rows, scale, zero, rows, wl.k, wl.group, wl.quant_op, wl.bits)
    dq_gpu = torch.empty((wl.n_out, wl.k), dtype=torch.half, device=wl.y.device)
    wl.mg.dequantize(wl.w[0], wl.s[0], wl.z[0], dq_gpu, wl.n_out, wl.k, wl.group, wl.quant_op, wl.bits)
    torch.cuda.synchronize()
    dq_bad = int((dq_gpu[:rows].cpu().numpy().view(np.uint16) != np.asarray(dq_ref).reshape(rows, wl.k).view(np.uint16)).sum())
    return dict(cpu_seconds=cpu_s, cpu_reps=reps, sample_bytes=sample_bytes, rows=rows,
                cpu_all_seconds=t_all / r_all, cpu_all_reps=r_all, cpu_all_cores=cores,
                max_abs_err=float(abs_err.max()), max_rel_err=float(rel_err.max()), rel_floor=floor,
                dequant_mismatches=dq_bad)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20000)
    ap.add_argument("--warmup", type=int, default=2000)
    ap.add_argument("--workload", default="ns", choices=sorted(WORKLOADS))
    ap.add_argument("--m-batch", type=int, default=None)
    ap.add_argument("--launch", default="graph", choices=["graph", "stream"],
                    help="graph: the steps are replayed from a captured HIP graph (one kernel node per step, one "
                         "rotation of the buffer sets per replay); stream: one host launch per step")
    ap.add_argument("--extra", default="c5,vocab,nsx8,nsx16,ns:bf16,c5:bf16",
                    help="comma list of further workloads reported under 'other_workloads' ('' = none); "
                         "'<name>x<B>' runs B problems per launch through the batched entry point, "
                         "'<name>:bf16' runs the bfloat16 entry point")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / oracle check")
    ap.add_argument("--no-warm-cache", action="store_true",
                    help="skip the warm-cache and launch-floor side measurements (keeps a kernel trace to the cold launches)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only copy 512 MiB device to device four times and exit: the known-size kernel against which "
                         "the FETCH_SIZE / WRITE_SIZE counters of `rocprofv3 --pmc` are scaled")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (a GEMV over one weight matrix held by one MI355X); "
              "--gpus above 1 is not supported", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    import mixed_gemv_amd as mg
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.copy_calibration:
        n = 512 << 20
        src = torch.full((n,), 3, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copied_bytes_per_kernel": n, "kernels": 4}))
        return

    wl = Workload(args.workload, device, m_batch=args.m_batch)
    wall, ev_us, steps, warm_done = time_workload(wl, args.steps, args.warmup, use_graph=(args.launch == "graph"))
    us_per_step = wall * 1e6 / steps
    value = wl.bytes / (wall / steps) / 1e9
    kernel_us = ev_us
    achieved = wl.bytes / (kernel_us * 1e-6) / 1e9
    plan = mg.query_launch(wl.n_out, wl.m_batch, wl.k, wl.bits, wl.k if wl.quant_op == 1 else wl.group)

    out = {
        "metric": "HBM GB/s & % of peak, us/call; int4-g128 GEMV M=1, N=K=4096",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": args.warmup,
        "warmup_steps_run": warm_done,
        "ms_per_step": round(us_per_step / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": wl.description, "name": wl.name, "n_out": wl.n_out, "k": wl.k, "m_batch": wl.m_batch,
                   "weight_bits": wl.bits, "quant_op": wl.quant_op, "group_size": wl.group, "bias": wl.has_bias,
                   "buffer_sets_rotated": wl.sets, "launch": "hip_graph" if args.launch == "graph" else "stream", "plan": plan},
        "us_per_call": round(us_per_step, 3),
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
        "algorithmic_bytes_per_call": wl.bytes,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": measured_traffic_bytes(wl.name, wl.m_batch),
                     "kernel_us_avg_events": round(kernel_us, 3)},
    }
    # the same launches on ONE buffer set, i.e. out of the Infinity Cache: reported beside the cold
    # figure, never as `value`
    if not args.no_warm_cache:
        all_sets, wl.sets = wl.sets, 1
        wall_w, ev_w, st_w, _ = time_workload(wl, max(200, args.steps // 4), 20, use_graph=(args.launch == "graph"))
        wl.sets = all_sets
        out["warm_cache"] = {"us_per_call": round(wall_w * 1e6 / st_w, 3),
                             "GBps": round(wl.bytes / (wall_w / st_w) / 1e9, 1),
                             "note": "one buffer set re-read from the 256 MB Infinity Cache; not an HBM figure"}
    if args.launch == "graph" and not args.no_warm_cache:
        floor = launch_floor_us(device)
        out["launch_floor"] = {"us_per_launch": round(floor, 3),
                               "kernel_us_above_floor": round(kernel_us - floor, 3),
                               "note": "graph replay of a one-element fill kernel: the cadence of an empty launch"}
    if not args.no_cpu:
        chk = check_against_oracle(wl)
        out["cpu_baseline"] = {
            "value": round(chk["sample_bytes"] / chk["cpu_seconds"] / 1e9, 4), "unit": "GB/s", "cores": 1,
            "kind": "port",
            "sample": f"the whole workload ({chk['rows']} rows x {wl.k}), single-threaded HOST_CHECK loop, "
                      f"mean of {chk['cpu_reps']} runs, {chk['cpu_seconds']:.3f} s each",
            "us_per_call": round(chk["cpu_seconds"] * 1e6, 1)}
        out["cpu_baseline_all_cores"] = {
            "value": round(chk["sample_bytes"] / chk["cpu_all_seconds"] / 1e9, 4), "unit": "GB/s",
            "cores": chk["cpu_all_cores"], "kind": "port", "cpu_model": cpu_model(),
            "sample": f"the same loop with OpenMP over the rows, mean of {chk['cpu_all_reps']} runs",
            "us_per_call": round(chk["cpu_all_seconds"] * 1e6, 1)}
        out["parity"] = {"max_abs_err": chk["max_abs_err"], "max_rel_err": chk["max_rel_err"],
                         "rel_floor": chk["rel_floor"], "tolerance_rel": 2e-3,
                         "dequantized_weight_mismatches": chk["dequant_mismatches"],
                         "ok": bool(chk["max_rel_err"] <= 2e-3 and chk["dequant_mismatches"] == 0)}
    others = {}
    for name in [n for n in args.extra.split(",") if n and n != args.workload]:
        # "<workload>x<B>": B problems per launch through the batched entry point
        base, _, element = name.partition(":")
        base, _, batch = base.partition("x")
        batch = int(batch) if batch else 1
        w2 = Workload(base, device, min_sets=5 * batch if batch > 1 else None, element=element or "f16")
        if batch > 1:
            w2.enable_batched(batch)
        wall2, ev2, st2, _ = time_workload(w2, max(200, args.steps // (8 * batch)), max(20, args.warmup // 4),
                                           use_graph=(args.launch == "graph"))
        others[name] = {"workload": w2.description + (f", {batch} independent problems per launch" if batch > 1 else "")
                        + (", bfloat16 activations / scales / outputs" if element == "bf16" else ""),
                        "us_per_call": round(wall2 * 1e6 / st2, 3),
                        "us_per_problem": round(wall2 * 1e6 / st2 / batch, 3),
                        "value_GBps": round(batch * w2.bytes / (wall2 / st2) / 1e9, 1),
                        "kernel_us_avg_events": round(ev2, 3),
                        "roofline_frac": round(batch * w2.bytes / (ev2 * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                        "buffer_sets_rotated": w2.sets, "steps": st2}
        del w2
        torch.cuda.empty_cache()
    if others:
        out["other_workloads"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
