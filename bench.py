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
MEASURED_TRAFFIC_KIB = {"ns": (4466.5, 8.0), "c5": (61110.0, 56.0)}
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0


def measured_traffic_bytes(name, m_batch):
    if name not in MEASURED_TRAFFIC_KIB or m_batch != 1:
        return None
    fetch, write = MEASURED_TRAFFIC_KIB[name]
    return int((fetch * FETCH_SCALE + write * WRITE_SCALE) * 1024)


def measure_traffic_live(name, log=None):
    """HBM bytes per launch of workload `name`, measured now: four short child runs of this file under
    `rocprofv3 --pmc` (FETCH_SIZE and WRITE_SIZE of the workload's kernel, then of a 512 MiB device copy
    that calibrates the two counters).  Returns (bytes, description) or (None, reason)."""
    import csv
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    tool = shutil.which("rocprofv3")
    if tool is None:
        return None, "rocprofv3 not found"
    if any(k.startswith("ROCPROF") or k.startswith("ROCP_") for k in os.environ):
        return None, "this run is itself being profiled"
    here = os.path.abspath(__file__)
    steps = {"ns": 140}.get(name, 64)
    work = ["--workload", name, "--no-cpu", "--no-ceilings", "--no-warm-cache", "--no-traffic", "--extra", "",
            "--steps", str(steps), "--warmup", "8", "--launch", "stream"]
    runs = (("FETCH_SIZE", work, ("gemv_dpp_kernel", "gemv_mfma")), ("WRITE_SIZE", work, ("gemv_dpp_kernel", "gemv_mfma")),
            ("FETCH_SIZE", ["--copy-calibration"], ("copyBuffer",)), ("WRITE_SIZE", ["--copy-calibration"], ("copyBuffer",)))
    values = []
    tmp = tempfile.mkdtemp(prefix="mgemv_pmc_", dir="/tmp")
    try:
        env = dict(os.environ, TMPDIR="/tmp")
        for i, (counter, args, kernels) in enumerate(runs):
            out_dir = os.path.join(tmp, f"run{i}")
            cmd = [tool, "--pmc", counter, "--output-format", "csv", "-d", out_dir, "--", sys.executable, here] + args
            # The profiler starts the python child itself: the pass runs in a session of its own, so that
            # whatever happens every process of it -- the profiler, its child, their helpers -- can be ended
            # as one group and is waited for before this function returns.
            proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                                    start_new_session=True)
            try:
                status = proc.wait(timeout=150)
            except subprocess.TimeoutExpired:
                status = None
            finally:
                try:
                    os.killpg(proc.pid, signal.SIGKILL)     # stragglers of a pass that has ended, or the whole pass after a time-out
                except (ProcessLookupError, PermissionError):
                    pass
                proc.wait()
            if status is None:
                return None, f"the {counter} pass did not finish in 150 s"
            if status != 0:
                return None, f"the {counter} pass ended with status {status}"
            got = []
            for f in glob.glob(os.path.join(out_dir, "**", "*counter_collection.csv"), recursive=True):
                with open(f) as fh:
                    for row in csv.DictReader(fh):
                        if row.get("Counter_Name") == counter and any(k in row.get("Kernel_Name", "") for k in kernels):
                            got.append(float(row["Counter_Value"]))
            if not got:
                return None, f"the {counter} pass recorded no dispatch of the kernel"
            got = got[len(got) // 4:] or got
            values.append((sum(got) / len(got), len(got)))
            if log:
                log(f"traffic pass {i}: {counter} = {values[-1][0]:.1f} KiB per dispatch over {values[-1][1]} dispatches")
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    (fetch, n_f), (write, _), (copy_fetch, _), (copy_write, _) = values
    copied_kib = (512 << 20) / 1024.0
    fetch_scale, write_scale = copied_kib / copy_fetch, copied_kib / copy_write
    total = int((fetch * fetch_scale + write * write_scale) * 1024)
    return total, (f"measured by this run: rocprofv3 --pmc FETCH_SIZE {fetch:.1f} and WRITE_SIZE {write:.1f} KiB per dispatch "
                   f"(child runs of this file, --workload {name} --launch stream, {n_f} dispatches), scaled by what the same "
                   f"counters read for a 512 MiB device copy (x {fetch_scale:.3f}, x {write_scale:.3f})")


def algorithmic_bytes(n_out, k, bits, quant_op, group, m_batch, bias):
    groups = 1 if quant_op == 1 else k // group
    return (n_out * k * bits // 8 + groups * n_out * 2 * (2 if quant_op == 3 else 1) + (n_out * 2 if bias else 0)
            + m_batch * k * 2 + m_batch * n_out * 2)


class Workload:
    """Builds the rotating operand sets of one workload directly in HBM (torch is the allocator)."""

    def __init__(self, name, device, m_batch=None, seed=1234, min_sets=None, element="f16", keep_raw=(0,)):
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
        self.raw = {}   # buffer set -> un-preprocessed weights (host), for the sets the oracle is asked about
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
            if keep_raw == "all" or i in keep_raw:
                self.raw[i] = raw.numpy().copy()
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

    def set_m_batch(self, m_batch, seed=4321):
        """Another number of activation rows on the same weight sets."""
        import torch
        gen = torch.Generator(device="cpu").manual_seed(seed + m_batch)
        dt = self.y.dtype
        x = torch.rand((m_batch, self.k), generator=gen) * 2 - 1
        self.m_batch = m_batch
        self.x = x.to(dt).to(self.y.device)
        self.y = torch.zeros((m_batch, self.n_out), dtype=dt, device=self.y.device)
        self.bytes = algorithmic_bytes(self.n_out, self.k, self.bits, self.quant_op, self.group, m_batch, self.has_bias)

    def rotation(self):
        """Launches after which the sequence of buffer sets repeats."""
        b = getattr(self, "batch", 0)
        return self.sets // b if b else self.sets

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
            w_raw=self.raw.get(j),
            x=self.x.cpu().numpy(), scale=self.s[j].cpu().numpy(),
            zero=self.z[j].cpu().numpy() if self.z[j] is not None else None,
            bias=self.bias.cpu().numpy() if self.bias is not None else None)


class RoutedWorkload:
    """A decode step's expert GEMVs: one token, `top` of `experts` matrices of one shape (int4 group-128
    scale+zero, fp16), chosen per launch by a device-side index array -- one mgemv_gemv_routed launch, or
    `top` ordinary launches.  The stack is larger than the Infinity Cache and launch i takes experts
    i*top .. i*top+top-1, so every launch reads weights that have long left the caches."""

    def __init__(self, device, n_out=1408, k=2048, group=128, experts=256, top=8, seed=99):
        import numpy as np
        import torch
        import mixed_gemv_amd as mg
        self.mg, self.np = mg, np
        self.n_out, self.k, self.group, self.experts, self.top = n_out, k, group, experts, top
        self.bits, self.quant_op, self.m_batch, self.element = 4, 3, 1, "f16"
        gen = torch.Generator(device="cpu").manual_seed(seed)
        groups = k // group
        self.one = mg.preprocessed_size((k, n_out), mg.QuantType.W4_A16)
        self.raw = torch.randint(0, 256, (experts, n_out * k // 2), dtype=torch.uint8, generator=gen).numpy()
        pre = mg.MixedGemvWeightPreprocessor.run(self.raw.reshape(-1), (experts, k, n_out), mg.LayoutType.kColumnMajor,
                                                 mg.QuantType.W4_A16)
        self.w = torch.from_numpy(pre).to(device)
        self.s = (torch.rand((experts, groups, n_out), generator=gen) * 0.019 + 0.001).half().to(device)
        self.z = (torch.rand((experts, groups, n_out), generator=gen) * 0.1 - 0.05).half().to(device)
        self.x = (torch.rand((1, k), generator=gen) * 2 - 1).half().to(device)
        self.y = torch.zeros((top, n_out), dtype=torch.half, device=device)
        self.sets = experts // top            # distinct launches before the rotation repeats
        self.host_routes = [[(i * top + j) % experts for j in range(top)] for i in range(self.sets)]
        self.routes = [torch.tensor(r, dtype=torch.int32, device=device) for r in self.host_routes]
        self.strides = (self.one, 0, groups * n_out, 0, n_out)
        self.bytes = top * (algorithmic_bytes(n_out, k, 4, 3, group, 1, False) - k * 2) + k * 2
        self.routed = True
        self.description = (f"one token, {top} of {experts} experts of {n_out}x{k} (int4 group-{group} scale+zero), "
                            f"stack of {experts * self.one >> 20} MiB")

    def rotation(self):
        return self.sets

    def launch(self, i):
        j = i % self.sets
        if self.routed:
            self.mg.device_gemv_routed(self.w, self.x, self.s, self.z, None, self.y, self.routes[j], self.experts,
                                       self.top, self.n_out, 1, self.k, self.group, self.strides)
        else:
            for slot, e in enumerate(self.host_routes[j]):
                self.mg.device_gemv(self.w[e * self.one:(e + 1) * self.one], self.x, self.s[e], self.z[e], None,
                                    self.y[slot], 1, self.n_out, 1, self.k, self.group)

    def parity(self, threads):
        """Launch 0 both ways: the same bits; and its first and last problem against the oracle."""
        import oracle as orc
        import torch
        np = self.np
        got = {}
        for routed in (True, False):
            self.routed = routed
            self.y.fill_(float("nan"))
            self.launch(0)
            torch.cuda.synchronize()
            got[routed] = self.y.cpu().numpy().copy()
        self.routed = True
        worst = 0.0
        for slot in (0, self.top - 1):
            e = self.host_routes[0][slot]
            ref = orc.gemv(self.raw[e], self.x.cpu().numpy(), self.s[e].cpu().numpy(), self.z[e].cpu().numpy(), None,
                           self.n_out, 1, self.k, self.group, 3, 4, threads=threads).reshape(-1).astype(np.float64)
            y = got[True][slot].astype(np.float64)
            floor = max(float(np.sqrt(np.mean(ref * ref))) * 2.0 ** -7, 2.0 ** -24)
            worst = max(worst, float((np.abs(y - ref) / np.maximum(np.abs(ref), floor)).max()))
        same = bool(np.array_equal(got[True].view(np.uint16), got[False].view(np.uint16)))
        return {"tolerance_rel": 2e-3, "max_rel_err": worst, "problems_checked_against_the_oracle": 2,
                "routed_launch_equals_separate_launches_bit_for_bit": same, "ok": bool(same and worst <= 2e-3)}


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
MAX_GRAPH_NODES = 4096   # launches per captured graph; longer timed regions replay it several times
TIMED_BUDGET_SECONDS = 0.6


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


class _Region:
    """EXACTLY `steps` launches, starting at buffer set `first`: replayed HIP graphs (or plain
    stream launches).  Regions that start at different sets continue the rotation, so that the
    repetitions of a short region (20 steps over 35 sets) never re-read a set that is still in
    the Infinity Cache."""

    def __init__(self, wl, steps, first, use_graph):
        self.wl, self.steps, self.first, self.graphs = wl, steps, first, None
        if use_graph:
            self.graphs, done = [], 0
            while done < steps:
                n = min(MAX_GRAPH_NODES, steps - done)
                # replays of one graph must themselves keep rotating: whole rotations per graph
                if steps - done > MAX_GRAPH_NODES:
                    n -= n % wl.rotation()
                self.graphs.append((_capture(wl, first + done, n), n))
                done += n

    def run(self):
        if self.graphs is None:
            for i in range(self.first, self.first + self.steps):
                self.wl.launch(i)
        else:
            for g, _ in self.graphs:
                g.replay()


def time_workload(wl, steps, warmup, use_graph=False, repetitions=None):
    """Runs at least `warmup` untimed steps (more if needed to bring an idle device up to its
    steady clocks), then times a region of EXACTLY `steps` steps, bracketed by a device
    synchronisation on both sides; the region is repeated (each repetition continues the buffer
    rotation where the last one stopped) and the MEDIAN repetition is reported.  Returns (median
    wall seconds of one region, median kernel microseconds per step by a HIP event pair on the
    launch stream, steps, warm-up steps actually run, repetitions, min wall seconds)."""
    import math
    import statistics
    import torch
    rot = wl.rotation()
    distinct = rot // math.gcd(steps, rot)          # distinct starting sets that repetitions cycle through
    regions = [_Region(wl, steps, (r * steps) % rot, use_graph) for r in range(min(distinct, 12))]
    done = 0
    for i in range(warmup):
        wl.launch(i)
    done += warmup
    torch.cuda.synchronize()
    t_spin = time.perf_counter()
    k = 0
    while time.perf_counter() - t_spin < SPIN_UP_SECONDS:
        regions[k % len(regions)].run()
        k += 1
        done += steps
        torch.cuda.synchronize()
    # one untimed pass for an estimate, then as many repetitions as fit the budget (5 .. 64)
    t0 = time.perf_counter()
    regions[k % len(regions)].run()
    torch.cuda.synchronize()
    est = max(time.perf_counter() - t0, 1e-6)
    k += 1
    done += steps
    reps = repetitions or max(5, min(64, int(TIMED_BUDGET_SECONDS / est)))
    walls, events = [], []
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    # Wall-clock repetitions hold nothing but the `steps` launches between the two synchronisations; the
    # kernel time comes from repetitions of their own, with an event pair on the launch stream round the
    # same launches (the two event records cost a 20-step region about 7 us of wall time).
    for r in range(2 * reps):
        region = regions[(k + r) % len(regions)]
        torch.cuda.synchronize()
        if r % 2 == 0:
            t0 = time.perf_counter()
            region.run()
            torch.cuda.synchronize()
            walls.append(time.perf_counter() - t0)
        else:
            e0.record()
            region.run()
            e1.record()
            torch.cuda.synchronize()
            events.append(e0.elapsed_time(e1) * 1e3 / steps)
    return statistics.median(walls), statistics.median(events), steps, done, reps, min(walls)


class _Launches:
    """Anything with launch(i) and rotation(): lets time_workload time a probe like a workload."""

    def __init__(self, fn, rotation):
        self.fn, self.rot = fn, rotation

    def launch(self, i):
        self.fn(i)

    def rotation(self):
        return self.rot


def launch_floor_us(use_graph=True):
    """Cadence of an EMPTY kernel launched like the timed steps: what one launch costs on this
    machine before it reads a single byte."""
    import mixed_gemv_amd as mg
    probe = _Launches(lambda i: mg.probe_empty_launch(), 1)
    _, ev_us, *_ = time_workload(probe, 2000, 100, use_graph=use_graph, repetitions=7)
    return ev_us


def ceilings_of(wl, use_graph, timeline=False):
    """ceilings_of_valu_kernel; where the product launch of the workload is a matrix-core kernel (which has no
    measurement builds), the VALU kernel is put in its place for the probes, and the result says so."""
    import mixed_gemv_amd as mg
    if wl.bits != 4 or wl.quant_op != 3 or wl.m_batch != 1:
        return None
    product = mg.query_launch(wl.n_out, 1, wl.k, 4, wl.group)
    if product["matrix_core"] == 0:
        return ceilings_of_valu_kernel(wl, use_graph, timeline)
    mg.set_matrix_core_threshold(17)
    try:
        out = ceilings_of_valu_kernel(wl, use_graph, timeline)
        valu = mg.query_launch(wl.n_out, 1, wl.k, 4, wl.group)
        _, ev_us, *_ = time_workload(_Launches(lambda i: wl.launch(i), wl.sets), 400, 20, use_graph=use_graph, repetitions=5)
    finally:
        mg.set_matrix_core_threshold(0)
    out["probed_kernel"] = {
        "kernel": "VALU", "workgroups": valu["workgroups"], "waves_per_workgroup": valu["threads"] // 64,
        "tiles_in_sequence": valu["tiles_in_sequence"], "us_per_launch": round(ev_us, 3),
        "note": "the product launch of this workload is the k-stationary matrix-core kernel "
                f"({product['workgroups']} workgroups of {product['threads'] // 64} waves, walks of {product['tiles_in_sequence']} tiles), "
                "which has no measurement builds: loads_only, compute_only and the timeline are those of the VALU kernel "
                "that the same workload runs on when the matrix cores are switched off (mgemv_set_matrix_core_threshold(17))"}
    return out


def ceilings_of_valu_kernel(wl, use_graph, timeline=False):
    """What bounds the workload's kernel from above, measured with the probes of the library on
    the workload's own (rotated, cold) buffers:
      stream_read   a plain streaming read of exactly the workload's weight bytes, for the launch
                    shape of the GEMV and for the best of a few others (no scales, no activations,
                    no arithmetic): us per launch and GB/s of the bytes read;
      loads_only    the GEMV kernel itself with every load kept and the arithmetic removed;
      compute_only  the GEMV kernel itself with the arithmetic kept and only each wave's first unit loaded;
      timeline      when the phases of one launch happen, and how long its waves wait for their loads."""
    import statistics
    import numpy as np
    import torch
    import mixed_gemv_amd as mg
    if wl.bits != 4 or wl.quant_op != 3 or wl.m_batch != 1:
        return None
    plan = mg.query_launch(wl.n_out, 1, wl.k, 4, wl.group)
    w_bytes = wl.w[0].numel()
    sink = torch.zeros(1, dtype=torch.int32, device=wl.y.device)
    out = {"weight_bytes": w_bytes, "algorithmic_bytes": wl.bytes, "stream_read": []}
    waves = plan["threads"] // 64
    probe = _Launches(lambda i: mg.probe_empty_grid(plan["workgroups"], waves), 1)
    _, ev_us, *_ = time_workload(probe, 2000, 100, use_graph=use_graph, repetitions=7)
    out["empty_grid"] = {"workgroups": plan["workgroups"], "waves_per_workgroup": waves, "us_per_launch": round(ev_us, 3),
                         "note": "an empty kernel with the GEMV's grid: launch cadence plus the dispatch of its waves"}
    shapes = [("the GEMV's launch shape", plan["workgroups"], waves, 2)]
    shapes += [("", 128, 8, 2), ("", 256, 8, 2), ("", 512, 4, 4), ("", 1024, 4, 4), ("", 512, 8, 8)]
    for label, wgs, wv, depth in shapes:
        if w_bytes // 4096 < wgs * wv * depth:
            continue
        probe = _Launches(lambda i, a=(wgs, wv, depth): mg.probe_stream_read(wl.w[i % wl.sets], w_bytes, *a, sink), wl.sets)
        _, ev_us, *_ = time_workload(probe, 400, 20, use_graph=use_graph, repetitions=5)
        read = (w_bytes // 4096 // (wgs * wv)) * (wgs * wv) * 4096
        out["stream_read"].append({"workgroups": wgs, "waves_per_workgroup": wv, "units_in_flight": depth,
                                   "us_per_launch": round(ev_us, 3), "GBps": round(read / ev_us / 1e3, 1),
                                   "frac_of_hbm_peak": round(read / ev_us / 1e3 / HBM_PEAK_GBS, 4), "note": label})
    best = min(out["stream_read"], key=lambda e: e["us_per_launch"])
    out["stream_read_best_us"] = best["us_per_launch"]
    # the whole workload at the best plain-read rate: the time below which no kernel of this kind gets
    out["algorithmic_bytes_at_best_stream_rate_us"] = round(wl.bytes / (best["GBps"] * 1e3), 3)
    probe = _Launches(lambda i: mg.probe_gemv(mg.PROBE_LOADS_ONLY, None, wl.w[i % wl.sets], wl.x, wl.s[i % wl.sets],
                                              wl.z[i % wl.sets], wl.y, wl.n_out, wl.k, wl.group), wl.sets)
    _, ev_us, *_ = time_workload(probe, 400, 20, use_graph=use_graph, repetitions=5)
    out["loads_only"] = {"us_per_launch": round(ev_us, 3), "GBps": round(wl.bytes / ev_us / 1e3, 1),
                         "frac_of_hbm_peak": round(wl.bytes / ev_us / 1e3 / HBM_PEAK_GBS, 4),
                         "note": "the GEMV kernel with its weight, activation, scale and zero loads and no arithmetic"}
    probe = _Launches(lambda i: mg.probe_gemv(mg.PROBE_COMPUTE_ONLY, None, wl.w[i % wl.sets], wl.x, wl.s[i % wl.sets],
                                              wl.z[i % wl.sets], wl.y, wl.n_out, wl.k, wl.group), wl.sets)
    _, ev_us, *_ = time_workload(probe, 400, 20, use_graph=use_graph, repetitions=5)
    units_per_wave = plan["steps_per_wave"] * plan["tiles_in_sequence"]
    out["compute_only"] = {"us_per_launch": round(ev_us, 3), "units_per_wave": units_per_wave,
                           "note": "the GEMV kernel with its arithmetic kept (dequantise + dot of every unit, combine, store) "
                                   "and only the first unit of each wave loaded"}
    if timeline:
        cus = torch.cuda.get_device_properties(wl.y.device).multi_processor_count
        plan_dev = mg.query_launch(wl.n_out, 1, wl.k, 4, wl.group, num_compute_units=cus)
        n_waves = -(-plan_dev["workgroups"] // 8) * 8 * (plan_dev["threads"] // 64)   # the grid is a multiple of 8 workgroups
        words = mg.PROBE_TIMELINE_WORDS
        trace = torch.zeros((n_waves, words), dtype=torch.int64, device=wl.y.device)
        waves = plan_dev["threads"] // 64
        light, heavy = [], []
        med = lambda v: float(np.median(v))  # noqa: E731
        for i in range(48):
            trace.zero_()
            torch.cuda.synchronize()
            # behind a few ordinary launches, so that the probe launch meets the queue as a timed step does
            for w in range(3):
                wl.launch(i + w)
            j = (i + 3) % wl.sets
            # odd passes time the wait in front of every unit as well (two more clock readings per unit, a few per cent slower)
            mg.probe_gemv(mg.PROBE_TIMELINE_WAITS if i % 2 else mg.PROBE_TIMELINE, trace, wl.w[j], wl.x, wl.s[j], wl.z[j],
                          wl.y, wl.n_out, wl.k, wl.group)
            torch.cuda.synchronize()
            t = trace.cpu().numpy().astype("float64")
            if i < 8 or not np.all((t[:, 0] > 0) & (t[:, 11] > 0)):   # (a workgroup without a tile leaves no stamps)
                continue
            t0 = t[:, 0].min()
            if i % 2 == 0:
                end = t[:, 4] - t0
                loop_end = (t[:, 3] - t0).reshape(-1, waves)          # by position in the workgroup
                light.append([med(t[:, 0] - t0), float((t[:, 0] - t0).max()), med(t[:, 1] - t[:, 0]), med(t[:, 2] - t[:, 1]),
                              med(t[:, 3] - t[:, 2]), med(t[:, 4] - t[:, 3]), float(end.max()), med(end),
                              float(np.percentile(end, 5)), float(np.percentile(end, 95)),
                              med((t[:, 13] - t[:, 12]) / np.maximum(t[:, 4] - t[:, 0], 1.0)) * 0.1, med(t[:, 11])]
                             + [med(loop_end[:, w]) for w in range(waves)])
            else:
                waits = t[:, 5:8]
                b1 = np.where(t[:, 9] > 0, t[:, 9], t[:, 3])
                b2 = np.where(t[:, 10] > 0, t[:, 10], t[:, 3])
                spans = np.stack([b1 - t[:, 1], b2 - b1, t[:, 3] - b2], axis=1)   # the thirds of a wave's units
                heavy.append([med(t[:, 3] - t[:, 1]), med(waits.sum(axis=1)), med(t[:, 8])]
                             + [v for k3 in range(3) for v in (med(spans[:, k3]), med(waits[:, k3]))])
        tick_us = 0.01  # s_memrealtime counts a constant 100 MHz clock
        if light:
            col = lambda c, rows=light: round(statistics.median(r[c] for r in rows) * tick_us, 3)  # noqa: E731
            out["timeline_us"] = {
                "clock": "s_memrealtime, 100 MHz (10 ns per tick); medians over the waves of a launch, then over launches",
                "wave_start_after_first_wave_median": col(0), "wave_start_after_first_wave_last": col(1),
                "start_to_first_unit_requested": col(2), "requested_to_first_block_arrived": col(3),
                "first_block_to_last_unit_computed": col(4), "last_unit_to_outputs_stored": col(5),
                "first_wave_start_to_last_store": col(6),
                "wave_end_after_first_wave_start": {"median": col(7), "p5": col(8), "p95": col(9), "last": col(6)},
                "last_unit_computed_by_wave_of_the_workgroup": [col(12 + w) for w in range(waves)],
                "units_per_wave": light[-1][11],
                "shader_clock_GHz": round(statistics.median(r[10] for r in light), 3),
                "shader_clock_note": "s_memtime ticks per s_memrealtime tick over a wave's life: the clock the compute units "
                                     "ran at during the probe launch (the power management lowers it under load)",
                "waves": n_waves, "launches": len(light)}
            if heavy:
                col = lambda c, rows=heavy: round(statistics.median(r[c] for r in rows) * tick_us, 3)  # noqa: E731
                out["timeline_us"]["unit_loop"] = {
                    "length": col(0), "waiting_in_front_of_units": col(1), "longest_single_wait": col(2),
                    "by_third_of_units": [{"third": k3 + 1, "length": col(3 + 2 * k3), "waiting": col(4 + 2 * k3)} for k3 in range(3)],
                    "note": "from the build that also times the explicit wait in front of every unit (operands and first weight "
                            "block of the unit); what is left of the loop is arithmetic, which the waves of a SIMD share, and "
                            "the waits for a unit's later blocks inside it"}
    return out


def ceilings_of_rows(wl, use_graph):
    """The same for a small-batch launch on the matrix cores (the LDS-staged kernel with shared stages):
    a plain streaming read of the weight bytes with the launch's shape, the kernel with its loads,
    staging and barriers but no arithmetic, and the kernel with only each wave's first k step loaded."""
    import torch
    import mixed_gemv_amd as mg
    plan = mg.query_launch(wl.n_out, wl.m_batch, wl.k, 4, wl.group)
    kstat = plan["matrix_core"] == 3
    if wl.bits != 4 or wl.quant_op != 3 or not (kstat or (plan["matrix_core"] == 2 and plan["tiles_per_wg"] >= 2)):
        return None
    w_bytes = wl.w[0].numel()
    sink = torch.zeros(1, dtype=torch.int32, device=wl.y.device)
    waves = plan["threads"] // 64
    out = {"weight_bytes": w_bytes, "algorithmic_bytes": wl.bytes,
           "kernel": "k-stationary matrix-core kernel" if kstat else "LDS-staged matrix-core kernel",
           "launch": {k: plan[k] for k in ("workgroups", "threads", "split_k", "tiles_per_wg", "steps_per_wave", "tiles_in_sequence")}}
    probe = _Launches(lambda i: mg.probe_stream_read(wl.w[i % wl.sets], w_bytes, plan["workgroups"], waves, 2, sink), wl.sets)
    _, ev_us, *_ = time_workload(probe, 300, 20, use_graph=use_graph, repetitions=5)
    out["stream_read"] = {"us_per_launch": round(ev_us, 3), "note": "plain streaming read of the weight bytes, the launch's shape"}
    notes = (("every load, the operand's way through LDS, the parking of the partial sums, the barrier and the combine; no arithmetic",
              "only the first tile's unit of each wave loaded; its arithmetic repeated for every tile of the walk") if kstat else
             ("every load, the staging of the activation rows and the barriers; no arithmetic",
              "only the first k step of each wave loaded; its staging and arithmetic repeated per k step"))
    for key, kind, note in (("loads_only", mg.PROBE_LOADS_ONLY, notes[0]), ("compute_only", mg.PROBE_COMPUTE_ONLY, notes[1])):
        probe = _Launches(lambda i, kind=kind: mg.probe_gemv_rows(kind, wl.m_batch, wl.w[i % wl.sets], wl.x, wl.s[i % wl.sets],
                                                                  wl.z[i % wl.sets], wl.y, wl.n_out, wl.k, wl.group), wl.sets)
        _, ev_us, *_ = time_workload(probe, 300, 20, use_graph=use_graph, repetitions=5)
        out[key] = {"us_per_launch": round(ev_us, 3), "note": note}
    return out


def _oracle_operands(wl, j):
    import numpy as np
    ops = wl.host_operands(j)
    w = ops["w_raw"]
    if w is None:
        raise RuntimeError(f"buffer set {j}: raw weights were not kept")
    if wl.bits == 8:
        w = w.view(np.int8)
    return w, ops


def parity_of_set(wl, j, threads, with_dequant=True):
    """GPU result on buffer set j against the CPU oracle (all rows): errors under both
    denominator floors, and the kernels' own dequantiser against the oracle's, bit for bit."""
    import numpy as np
    import torch
    import oracle as orc  # the checker, never the thing measured

    w, ops = _oracle_operands(wl, j)
    ref = orc.gemv(w, ops["x"], ops["scale"], ops["zero"], ops["bias"], wl.n_out, wl.m_batch, wl.k, wl.group,
                   wl.quant_op, wl.bits, threads=threads).astype(np.float64)
    wl.y.zero_()
    wl.launch(j)
    torch.cuda.synchronize()
    got = wl.y.cpu().numpy().astype(np.float64)
    rms = float(np.sqrt(np.mean(ref * ref)))
    abs_err = np.abs(got - ref)
    out = {"set": j, "max_abs_err": float(abs_err.max())}
    # 2^-7 * rms: the floor the tolerance is asked under (below it, the order in which fp32 adds
    # thousands of cancelling terms decides the error -- tests/helpers.py:error_report);
    # 2^-10 * rms: reported beside it
    for tag, frac in (("2^-7", 2.0 ** -7), ("2^-10", 2.0 ** -10)):
        floor = max(rms * frac, 2.0 ** -24)
        out[f"max_rel_err_floor_{tag}_rms"] = float((abs_err / np.maximum(np.abs(ref), floor)).max())
        out[f"outputs_below_floor_{tag}_rms"] = int((np.abs(ref) < floor).sum())
    out["rms_ref"] = rms
    if with_dequant:
        dq_ref = orc.dequantize(w, ops["scale"], ops["zero"], wl.n_out, wl.k, wl.group, wl.quant_op, wl.bits)
        dq_gpu = torch.empty((wl.n_out, wl.k), dtype=torch.half, device=wl.y.device)
        wl.mg.dequantize(wl.w[j], wl.s[j], wl.z[j], dq_gpu, wl.n_out, wl.k, wl.group, wl.quant_op, wl.bits)
        torch.cuda.synchronize()
        out["dequantized_weight_mismatches"] = int(
            (dq_gpu.cpu().numpy().view(np.uint16) != np.asarray(dq_ref).reshape(wl.n_out, wl.k).view(np.uint16)).sum())
        del dq_gpu, dq_ref
    out["ok"] = bool(out["max_rel_err_floor_2^-7_rms"] <= 2e-3 and out.get("dequantized_weight_mismatches", 0) == 0)
    return out


def parity_summary(wl, sets, threads, with_dequant=True):
    per_set = [parity_of_set(wl, j, threads, with_dequant) for j in sets]
    worst = lambda key: max(p[key] for p in per_set)  # noqa: E731
    return {"buffer_sets_checked": list(sets), "tolerance_rel": 2e-3,
            "max_abs_err": worst("max_abs_err"),
            "max_rel_err": worst("max_rel_err_floor_2^-7_rms"),
            "max_rel_err_floor_2^-10_rms": worst("max_rel_err_floor_2^-10_rms"),
            "outputs_below_floor_2^-7_rms": sum(p["outputs_below_floor_2^-7_rms"] for p in per_set),
            "outputs_below_floor_2^-10_rms": sum(p["outputs_below_floor_2^-10_rms"] for p in per_set),
            "outputs_checked": len(per_set) * wl.m_batch * wl.n_out,
            "dequantized_weight_mismatches": (sum(p["dequantized_weight_mismatches"] for p in per_set)
                                              if with_dequant else None),
            "ok": all(p["ok"] for p in per_set)}


def host_cores():
    import oracle as orc
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    return max(1, min(cores, orc.max_threads()))


def cpu_baseline(wl, budget_seconds=8.0):
    """The CPU oracle (a port of the reference's single-threaded HOST_CHECK loop) timed on this
    host on buffer set 0 of the workload, and the same loop with OpenMP over the rows."""
    import oracle as orc
    w, ops = _oracle_operands(wl, 0)
    call = lambda threads: orc.gemv(w, ops["x"], ops["scale"], ops["zero"], ops["bias"], wl.n_out, wl.m_batch, wl.k,  # noqa: E731
                                    wl.group, wl.quant_op, wl.bits, threads=threads)
    reps, elapsed = 0, 0.0
    while reps < 2 or (elapsed < budget_seconds and reps < 64):
        t0 = time.perf_counter()
        call(1)
        elapsed += time.perf_counter() - t0
        reps += 1
    cores = host_cores()
    t_all, r_all = 0.0, 0
    while r_all < 3 or (t_all < 2.0 and r_all < 200):
        t0 = time.perf_counter()
        call(cores)
        t_all += time.perf_counter() - t0
        r_all += 1
    return dict(seconds=elapsed / reps, reps=reps, all_seconds=t_all / r_all, all_reps=r_all, cores=cores)


def measure(wl, steps, warmup, use_graph):
    wall, ev_us, st, warm_done, reps, wall_min = time_workload(wl, steps, warmup, use_graph=use_graph)
    batch = getattr(wl, "batch", 0) or 1
    return {"us_per_call": round(wall * 1e6 / st, 3), "us_per_call_min": round(wall_min * 1e6 / st, 3),
            "us_per_problem": round(wall * 1e6 / st / batch, 3),
            "value_GBps": round(batch * wl.bytes / (wall / st) / 1e9, 1),
            "kernel_us_avg_events": round(ev_us, 3),
            "roofline_frac": round(batch * wl.bytes / (ev_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "algorithmic_bytes_per_call": batch * wl.bytes, "buffer_sets_rotated": wl.sets, "steps": st,
            "repetitions": reps, "warmup_steps_run": warm_done}


# what `--extra default` measures beside the headline: every benchmark configuration (c4 at each
# activation row count), the vocabulary projection, batched and routed launches and the bfloat16 entry points
DEFAULT_EXTRA = "c1,c2,c3a,c3b,c4:m1,c4:m2,c4:m4,c4:m8,c4:m16,c5,c5:m4,c5:m16,vocab,nsx8,nsx16,routed,ns:bf16,c5:bf16"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="ns", choices=sorted(WORKLOADS))
    ap.add_argument("--m-batch", type=int, default=None)
    ap.add_argument("--launch", default="graph", choices=["graph", "stream"],
                    help="graph: the steps are replayed from captured HIP graphs (one kernel node per step); "
                         "stream: one host launch per step")
    ap.add_argument("--extra", default=DEFAULT_EXTRA,
                    help="comma list of further workloads reported under 'other_workloads' ('' = none); "
                         "'<name>x<B>' runs B problems per launch through the batched entry point, "
                         "'<name>:bf16' the bfloat16 entry point, '<name>:m<M>' M activation rows, 'routed' one token's "
                         "8 of 256 experts in one routed launch (and in 8 launches)")
    ap.add_argument("--extra-steps", type=int, default=200, help="timed steps of each further workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and every oracle check")
    ap.add_argument("--no-warm-cache", action="store_true",
                    help="skip the warm-cache and launch-floor side measurements (keeps a kernel trace to the cold launches)")
    ap.add_argument("--no-ceilings", action="store_true",
                    help="skip the ceiling measurements (plain streaming reads, the kernel without its arithmetic, "
                         "the timeline of one launch)")
    ap.add_argument("--no-traffic", action="store_true",
                    help="do not measure the headline kernel's HBM traffic with rocprofv3 child runs (about a minute); "
                         "roofline.traffic then carries the figure of the committed profile")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only copy 512 MiB device to device four times and exit: the known-size kernel against which "
                         "the FETCH_SIZE / WRITE_SIZE counters of `rocprofv3 --pmc` are scaled")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (a GEMV over one weight matrix held by one MI355X); "
              "--gpus above 1 is not supported", file=sys.stderr)
        sys.exit(2)

    # the counter passes run first, as children, before this process touches the GPU
    live_traffic = (None, "not asked for")
    if not args.no_traffic and not args.copy_calibration and (args.m_batch in (None, 1)):
        live_traffic = measure_traffic_live(args.workload, log=lambda t: print(t, file=sys.stderr, flush=True))

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
    use_graph = args.launch == "graph"
    threads = 1 if args.no_cpu else host_cores()

    wl = Workload(args.workload, device, m_batch=args.m_batch)
    m = measure(wl, args.steps, args.warmup, use_graph)
    plan = mg.query_launch(wl.n_out, wl.m_batch, wl.k, wl.bits, wl.k if wl.quant_op == 1 else wl.group)
    # The kernel's average duration for the roofline: HIP events around at least 1000 back-to-back
    # launches, so that the start-up of a graph replay (several microseconds, once per region) does
    # not pass for kernel time when the timed region is as short as 20 steps.
    long_steps = max(args.steps, 1000)
    m_long = m if long_steps == args.steps else measure(wl, long_steps, 0, use_graph)
    kernel_us_long = m_long["kernel_us_avg_events"]
    kernel_us = m["kernel_us_avg_events"]          # HIP events round the timed region itself: what the roofline is priced at
    achieved = wl.bytes / (kernel_us * 1e-6) / 1e9
    achieved_long = wl.bytes / (kernel_us_long * 1e-6) / 1e9

    out = {
        "metric": "HBM GB/s & % of peak, us/call; int4-g128 GEMV M=1, N=K=4096",
        "value": m["value_GBps"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "warmup_steps_run": m["warmup_steps_run"],
        "repetitions": m["repetitions"],
        "timing": "median over the repetitions of a region of exactly `steps` launches, each bracketed by a device "
                  "synchronisation with nothing else in between; every repetition continues the rotation of the buffer "
                  "sets; kernel times (roofline) come from interleaved repetitions of their own with a HIP event pair "
                  "round the same launches",
        "ms_per_step": round(m["us_per_call"] / 1e3, 6),
        "ms_per_step_min": round(m["us_per_call_min"] / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": wl.description, "name": wl.name, "n_out": wl.n_out, "k": wl.k, "m_batch": wl.m_batch,
                   "weight_bits": wl.bits, "quant_op": wl.quant_op, "group_size": wl.group, "bias": wl.has_bias,
                   "buffer_sets_rotated": wl.sets, "launch": "hip_graph" if use_graph else "stream", "plan": plan},
        "us_per_call": m["us_per_call"],
        "pct_of_hbm_peak": round(100.0 * m["value_GBps"] / HBM_PEAK_GBS, 2),
        "algorithmic_bytes_per_call": wl.bytes,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": live_traffic[0] if live_traffic[0] is not None else measured_traffic_bytes(wl.name, wl.m_batch),
                     "traffic_source": live_traffic[1] if live_traffic[0] is not None else (
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of this workload, scaled by a 512 MiB "
                         "copy (profiles/); not re-measured by this run: " + live_traffic[1]),
                     "kernel_us_avg_events": kernel_us, "kernel_us_measured_over_steps": args.steps,
                     "note": "achieved / frac: algorithmic bytes over the kernel's average duration by HIP events round the timed "
                             "region of exactly `steps` launches; a region of 20 launches also carries the start of its graph "
                             "replay (0.3-0.5 us per launch), which the *_long_region figures, from regions of at least 1000 "
                             "launches, do not",
                     "kernel_us_avg_events_long_region": kernel_us_long, "long_region_steps": long_steps,
                     "achieved_long_region": round(achieved_long, 1), "frac_long_region": round(achieved_long / HBM_PEAK_GBS, 4)},
    }
    # the same launches on ONE buffer set, i.e. out of the Infinity Cache: reported beside the cold
    # figure, never as `value`
    if not args.no_warm_cache:
        all_sets, wl.sets = wl.sets, 1
        w = measure(wl, max(200, args.steps), 20, use_graph)
        wl.sets = all_sets
        out["warm_cache"] = {"us_per_call": w["us_per_call"], "GBps": w["value_GBps"],
                             "note": "one buffer set re-read from the 256 MB Infinity Cache; not an HBM figure"}
        floor = launch_floor_us(use_graph)
        out["launch_floor"] = {"us_per_launch": round(floor, 3),
                               "kernel_us_above_floor": round(kernel_us_long - floor, 3),
                               "note": "cadence of an empty kernel (mgemv_probe_empty_launch) launched like the timed steps"}
    if not args.no_ceilings:
        out["ceilings"] = {wl.name: ceilings_of(wl, use_graph, timeline=True)}
    if not args.no_cpu:
        cpu = cpu_baseline(wl)
        out["cpu_baseline"] = {
            "value": round(wl.bytes / cpu["seconds"] / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"the whole workload ({wl.n_out} rows x {wl.k}), single-threaded HOST_CHECK loop, "
                      f"mean of {cpu['reps']} runs, {cpu['seconds']:.3f} s each",
            "us_per_call": round(cpu["seconds"] * 1e6, 1)}
        out["cpu_baseline_all_cores"] = {
            "value": round(wl.bytes / cpu["all_seconds"] / 1e9, 4), "unit": "GB/s", "cores": cpu["cores"],
            "kind": "port", "cpu_model": cpu_model(),
            "sample": f"the same loop with OpenMP over the rows, mean of {cpu['all_reps']} runs",
            "us_per_call": round(cpu["all_seconds"] * 1e6, 1)}
        out["parity"] = parity_summary(wl, [0], threads)
    wl_name = wl.name
    del wl
    torch.cuda.empty_cache()

    others = {}
    built = {}   # (base, element) -> Workload, reused across activation row counts
    for name in [n for n in args.extra.split(",") if n and n != args.workload]:
        if name == "routed":
            built.clear()
            torch.cuda.empty_cache()
            rw = RoutedWorkload(device)
            entry = {"workload": rw.description + ", one routed launch (mgemv_gemv_routed)"}
            entry.update(measure(rw, args.extra_steps, max(20, args.warmup // 4), use_graph))
            rw.routed = False
            apart = measure(rw, args.extra_steps, max(20, args.warmup // 4), use_graph)
            rw.routed = True
            entry["separate_launches"] = {"launches_per_step": rw.top, "kernel_us_avg_events": apart["kernel_us_avg_events"],
                                          "us_per_call": apart["us_per_call"]}
            if not args.no_cpu:
                entry["parity"] = rw.parity(threads)
            others[name] = entry
            del rw
            continue
        # "<workload>[x<B>][:bf16][:m<M>]"
        base, *mods = name.split(":")
        base, _, batch = base.partition("x")
        batch = int(batch) if batch else 1
        element = "bf16" if "bf16" in mods else "f16"
        rows = next((int(t[1:]) for t in mods if t[:1] == "m" and t[1:].isdigit()), None)
        key = (base, element, batch)
        if key not in built:
            built.clear()
            torch.cuda.empty_cache()
            built[key] = Workload(base, device, min_sets=5 * batch if batch > 1 else None, element=element,
                                  keep_raw="all" if (base == "c5" and element == "f16" and not args.no_cpu) else (0,))
            if batch > 1:
                built[key].enable_batched(batch)
        w2 = built[key]
        if rows is not None and rows != w2.m_batch:
            w2.set_m_batch(rows)
        entry = {"workload": w2.description + (f", M={w2.m_batch}" if rows is not None else "")
                 + (f", {batch} independent problems per launch" if batch > 1 else "")
                 + (", bfloat16 activations / scales / outputs" if element == "bf16" else "")}
        entry.update(measure(w2, args.extra_steps, max(20, args.warmup // 4), use_graph))
        entry["plan"] = mg.query_launch(w2.n_out, w2.m_batch, w2.k, w2.bits, w2.k if w2.quant_op == 1 else w2.group,
                                        element=element)
        if not args.no_cpu and element == "f16" and batch == 1:
            # config 5 names 8 distinct rotated buffers: all of them are checked, not only the first
            sets = list(range(w2.sets)) if (base == "c5" and rows is None) else [0]
            entry["parity"] = parity_summary(w2, sets, threads, with_dequant=(rows in (None, 1)))
        if base == "c5" and rows is None and element == "f16" and batch == 1 and not args.no_ceilings:
            out.setdefault("ceilings", {})[base] = ceilings_of(w2, use_graph, timeline=True)
        if ((base == "c4" and rows in (8, 16)) or (base == "c5" and rows in (4, 16))) and element == "f16" and batch == 1 and not args.no_ceilings:
            c = ceilings_of_rows(w2, use_graph)
            if c is not None:
                out.setdefault("ceilings", {})[name] = c
        others[name] = entry
    built.clear()
    torch.cuda.empty_cache()
    # every BASELINE entry at a glance: name -> [kernel us by events, fraction of the HBM peak, parity ok (1 / 0, -1 = not checked)]
    by_workload = {wl_name: [round(kernel_us, 3), round(achieved / HBM_PEAK_GBS, 4),
                             -1 if "parity" not in out else int(bool(out["parity"].get("ok")))]}
    for name, e in others.items():
        by_workload[name] = [e["kernel_us_avg_events"], e["roofline_frac"],
                             -1 if "parity" not in e else int(bool(e["parity"].get("ok")))]
    out["roofline"]["by_workload"] = by_workload
    if others:
        out["other_workloads"] = others
        out["all_parity_ok"] = bool(out.get("parity", {}).get("ok", True)
                                    and all(e.get("parity", {}).get("ok", True) for e in others.values()))
    out["launch_plans"] = {"built_in_table_entries": mg.default_plan_count(), "caller_table_entries": mg.tuned_plan_count(),
                           "note": "rules of plan_launch plus the library's compiled-in table (mixed_gemv_amd/default_plans.json); "
                                   "nothing is tuned or installed by this run"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
