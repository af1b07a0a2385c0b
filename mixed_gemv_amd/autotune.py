"""Launch-plan tuner: measures the launch geometries the kernels support for one problem on the
GPU at hand and installs the fastest as that problem's tuned plan.

The reference fixes its ThreadBlockShape / WarpShape / kStages at compile time
(mixed_gemv_test.cu:40, 67-70; the 1- and 2-stage main loops of
gemv/threadblock/default_dq_mma_simt.h:224-234, 394-404) and a user re-compiles per shape.
Here the same choice is a table keyed on (n_out, k, weight_bits, group_size, m_batch) that a
deployment fills once -- `tune()` per layer shape -- and can carry along as JSON
(`save_table` / `load_table`).

Timing is cold-cache: weight / scale / zero sets are rotated so that more than the 256 MB
Infinity Cache is touched between two uses of a set, the launches are replayed from a HIP
graph, and the kernel time is taken with an event pair on the launch stream.
"""
import json
import time

from . import api

_CACHE_BYTES = (256 << 20) + (32 << 20)
_KERNEL_NAMES = {api.KERNEL_AUTO: "auto", api.KERNEL_VALU: "valu",
                 api.KERNEL_MATRIX_CORE_REGISTER_OPERAND: "matrix_core_register_operand",
                 api.KERNEL_MATRIX_CORE_LDS_STAGED: "matrix_core_lds_staged",
                 api.KERNEL_MATRIX_CORE_K_STATIONARY: "matrix_core_k_stationary"}
_installed = {}  # key tuple -> entry dict, what save_table writes


def candidate_plans(n_out, k, weight_bits, m_batch):
    """Knob settings worth measuring, as dicts for set_tuned_plan (duplicates in effect are
    removed later by comparing the geometry the library reports)."""
    out = [dict(kernel=api.KERNEL_AUTO), dict(kernel=api.KERNEL_AUTO, stages=1)]
    wave_limit = 8 if m_batch >= 3 else 16
    for tiles_per_wg in (1, 2, 4):
        for split_k in (1, 2, 4, 8, 16):
            if tiles_per_wg * split_k > wave_limit:
                continue
            for cap in (0, 256, 512):
                out.append(dict(kernel=api.KERNEL_VALU, split_k=split_k, tiles_per_wg=tiles_per_wg,
                                max_workgroups=cap))
    if m_batch >= 2:
        for tiles_per_wg in (1, 2, 4):   # 1 or 2 tiles share 8 staged rows, 2 or 4 share 16; others fall back to 2
            for split_k in (1, 2, 4):
                out.append(dict(kernel=api.KERNEL_MATRIX_CORE_LDS_STAGED, split_k=split_k, tiles_per_wg=tiles_per_wg))
        for tiles_per_wave in (1, 2):
            for split_k in (2, 4, 8):
                out.append(dict(kernel=api.KERNEL_MATRIX_CORE_REGISTER_OPERAND, split_k=split_k,
                                tiles_per_wave=tiles_per_wave))
    # one wave per k step, one workgroup per compute unit (or two) walking the tiles; where the kernel does not exist
    # (more than 16 k steps, bf16) the library falls back to its usual choice and the duplicate is dropped later
    for cap in (0, 512):
        out.append(dict(kernel=api.KERNEL_MATRIX_CORE_K_STATIONARY, max_workgroups=cap))
    return out


class _Problem:
    """Synthetic operands of one problem, resident in device memory.  Any byte string is a valid
    preprocessed weight buffer, so the weights are random bytes."""

    def __init__(self, n_out, k, weight_bits, quant_op, group_size, m_batch, bias, device, seed, cold_bytes,
                 element="f16"):
        import torch
        dtype = torch.bfloat16 if element == "bf16" else torch.half
        self.args = (n_out, m_batch, k, group_size, int(quant_op), weight_bits)
        qt = api.QuantType.W4_A16 if weight_bits == 4 else api.QuantType.W8_A16
        w_bytes = api.preprocessed_size((k, n_out), qt)
        groups = 1 if quant_op == api.WeightOnlyQuantOp.PER_COLUMN_SCALE_ONLY else k // group_size
        per_set = w_bytes + 2 * groups * n_out * 2
        self.sets = max(4, -(-cold_bytes // per_set) + 1)
        gen = torch.Generator(device=device).manual_seed(seed)
        self.w = torch.randint(0, 256, (self.sets, w_bytes), dtype=torch.uint8, device=device, generator=gen)
        self.s = (torch.rand((self.sets, groups, n_out), device=device, generator=gen) * 0.019 + 0.001).to(dtype)
        self.z = (torch.rand((self.sets, groups, n_out), device=device, generator=gen) * 0.1 - 0.05).to(dtype)
        self.x = (torch.rand((m_batch, k), device=device, generator=gen) * 2 - 1).to(dtype)
        self.bias = (torch.rand((n_out,), device=device, generator=gen) * 0.2 - 0.1).to(dtype) if bias else None
        self.y = torch.empty((m_batch, n_out), dtype=dtype, device=device)

    def launch(self, i):
        n_out, m_batch, k, group_size, quant_op, bits = self.args
        j = i % self.sets
        api.device_gemv(self.w[j], self.x, self.s[j], self.z[j] if quant_op == 3 else None, self.bias, self.y, 1,
                        n_out, m_batch, k, group_size, quant_op, bits)

    def time_us(self, launches):
        """Average microseconds per launch over whole rotations of the operand sets."""
        import torch
        nodes = self.sets * max(1, -(-32 // self.sets))
        self.launch(0)  # any lazy initialisation happens outside the capture
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(nodes):
                    self.launch(i)
        torch.cuda.current_stream().wait_stream(side)
        replays = max(2, -(-launches // nodes))
        graph.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (replays * nodes)


def _key(n_out, k, weight_bits, quant_op, group_size, m_batch, element="f16"):
    per_column = int(quant_op) == int(api.WeightOnlyQuantOp.PER_COLUMN_SCALE_ONLY)
    return (int(n_out), int(k), int(weight_bits), int(k if per_column else group_size), int(m_batch),
            "bf16" if element == "bf16" else "f16")


def _entry_key(entry):
    return (entry["n_out"], entry["k"], entry["weight_bits"], entry["group_size"], entry["m_batch"],
            entry.get("element", "f16"))


def install(entry):
    """Installs one table entry (a dict as produced by tune / stored by save_table)."""
    api.set_tuned_plan(entry["n_out"], entry["k"], entry["weight_bits"], entry["group_size"], entry["m_batch"],
                       kernel=entry.get("kernel", 0), split_k=entry.get("split_k", 0),
                       tiles_per_wg=entry.get("tiles_per_wg", 0), tiles_per_wave=entry.get("tiles_per_wave", 0),
                       max_workgroups=entry.get("max_workgroups", 0), stages=entry.get("stages", 0),
                       element=entry.get("element", "f16"))
    _installed[_entry_key(entry)] = dict(entry)


def erase(key):
    """Removes the entry of one key (n_out, k, weight_bits, group_size, m_batch, element) from the
    library's table and from what save_table writes."""
    api.erase_tuned_plan(*key[:5], element=key[5])
    _installed.pop(key, None)


def tune(n_out, k, weight_bits=4, quant_op=api.WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS, group_size=128,
         m_batch=1, bias=False, device="cuda:0", launches=400, rounds=2, min_gain=0.02, seed=1,
         cold_bytes=_CACHE_BYTES, log=None, element="f16"):
    """Measures the candidate plans for this problem and installs the fastest, unless it beats the
    built-in plan by less than `min_gain` (then the key ends up without an entry: one left by an
    earlier run is removed, since the built-in plan has just been measured to be as good).  Every
    candidate, the built-in plan included, is measured with a process-wide override set, which
    makes the library ignore the table, so an entry that already exists never stands in for the
    built-in plan.  Returns a
    dict with the chosen entry (or None), the built-in time and every measurement.  `cold_bytes`
    is how much operand data is rotated between two uses of the same buffers (default: more than
    the Infinity Cache).  `element` ("f16" / "bf16") picks the entry points that are timed; an entry
    serves launches of its own element type only.

    Must not run while other threads launch GEMVs: the candidates are applied through the
    process-wide overrides."""
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError("autotune.tune needs the GPU")
    device = torch.device(device)
    key = _key(n_out, k, weight_bits, quant_op, group_size, m_batch, element)
    cus = torch.cuda.get_device_properties(device).multi_processor_count
    prob = _Problem(n_out, k, weight_bits, api.WeightOnlyQuantOp(quant_op), key[3], m_batch, bias, device, seed,
                    cold_bytes, element)
    seen, results = {}, []
    try:
        with torch.cuda.device(device):
            _apply(dict(kernel=api.KERNEL_AUTO))
            spin = time.perf_counter()
            while time.perf_counter() - spin < 0.5:  # an idle device needs a while to reach its clocks
                prob.time_us(launches)
            for cand in candidate_plans(n_out, k, weight_bits, m_batch):
                _apply(cand)
                geometry = tuple(sorted(api.query_launch(n_out, m_batch, k, weight_bits, key[3], element=element,
                                                         num_compute_units=cus).items()))
                if geometry in seen:
                    continue
                seen[geometry] = cand
                us = min(prob.time_us(launches) for _ in range(rounds))
                results.append((us, cand, dict(geometry)))
                if log:
                    log(f"{us:8.2f} us  {_describe(cand)}  -> {dict(geometry)}")
            builtin_us = results[0][0]
            best_us, best, best_geometry = min(results, key=lambda r: r[0])
            if best is not results[0][1]:
                # confirm the winner against the built-in plan, alternating, before believing it
                for _ in range(3):
                    _apply(results[0][1])
                    builtin_us = min(builtin_us, prob.time_us(launches))
                    _apply(best)
                    best_us = min(best_us, prob.time_us(launches))
    finally:
        _apply(dict(kernel=api.KERNEL_AUTO))
        api.set_prefetch_stages(0)
    entry = None
    if best is not results[0][1] and best_us < builtin_us * (1.0 - min_gain):
        entry = dict(n_out=key[0], k=key[1], weight_bits=key[2], group_size=key[3], m_batch=key[4],
                     kernel=best.get("kernel", 0), split_k=best.get("split_k", 0),
                     tiles_per_wg=best.get("tiles_per_wg", 0), tiles_per_wave=best.get("tiles_per_wave", 0),
                     max_workgroups=best.get("max_workgroups", 0), stages=best.get("stages", 0), element=key[5],
                     us=round(best_us, 3), builtin_us=round(builtin_us, 3))
        install(entry)
    else:
        erase(key)
    return dict(entry=entry, builtin_us=builtin_us, best_us=best_us, best_geometry=best_geometry,
                builtin_geometry=results[0][2],
                measurements=[(us, _describe(c)) for us, c, _ in results])


def reconfirm(entry, device="cuda:0", launches=400, rounds=5, seed=1, cold_bytes=_CACHE_BYTES, quant_op=None, bias=False):
    """Measures an existing table entry against the built-in plan once more, in alternation, on the
    device at hand, and appends the gain in per cent (positive: the entry is ahead) to
    entry["confirmations"].  A gain found on one machine at one time can be that machine's: boxes of
    the same kind differ by several per cent among themselves (28672 x 8192: 22.4-24.4 us from lease
    to lease), so an entry should only ship after `confirmed()` -- the gain shown again on another
    lease.  Returns the gain.  Like tune(), must not run while other threads launch GEMVs."""
    import statistics
    import torch
    device = torch.device(device)
    element = entry.get("element", "f16")
    per_column = entry["group_size"] == entry["k"]
    qop = api.WeightOnlyQuantOp(quant_op) if quant_op is not None else (
        api.WeightOnlyQuantOp.PER_COLUMN_SCALE_ONLY if per_column else api.WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS)
    prob = _Problem(entry["n_out"], entry["k"], entry["weight_bits"], qop, entry["group_size"], entry["m_batch"], bias,
                    device, seed, cold_bytes, element)
    cand = {k: entry.get(k, 0) for k in ("kernel", "split_k", "tiles_per_wg", "tiles_per_wave", "max_workgroups")}
    if entry.get("stages"):
        cand["stages"] = entry["stages"]
    builtin, tuned = [], []
    try:
        with torch.cuda.device(device):
            _apply(dict(kernel=api.KERNEL_AUTO))
            spin = time.perf_counter()
            while time.perf_counter() - spin < 0.5:
                prob.time_us(launches)
            for _ in range(rounds):
                _apply(dict(kernel=api.KERNEL_AUTO))
                builtin.append(prob.time_us(launches))
                _apply(cand)
                tuned.append(prob.time_us(launches))
    finally:
        _apply(dict(kernel=api.KERNEL_AUTO))
        api.set_prefetch_stages(0)
    gain = round(100.0 * (statistics.median(builtin) / statistics.median(tuned) - 1.0), 2)
    entry.setdefault("confirmations", []).append(gain)
    return gain


def confirmed(entry, min_gain=0.02, leases=2):
    """True when the entry's gain over the built-in plan reached `min_gain` in at least `leases`
    separate confirmation runs (reconfirm) and it was never behind by that much."""
    gains = entry.get("confirmations", [])
    return (sum(1 for g in gains if g >= 100.0 * min_gain) >= leases) and all(g > -100.0 * min_gain for g in gains)


def _apply(cand):
    kernel = cand.get("kernel", api.KERNEL_AUTO)
    api.set_prefetch_stages(cand.get("stages", 2))  # 2 is the built-in value; any override set bypasses the table
    api.set_launch_override(cand.get("split_k", 0), cand.get("tiles_per_wg", 0), cand.get("tiles_per_wave", 0),
                            cand.get("max_workgroups", 0))
    api.set_matrix_core_threshold({api.KERNEL_AUTO: 0, api.KERNEL_VALU: 17}.get(kernel, 1))
    api.set_matrix_core_variant({api.KERNEL_MATRIX_CORE_REGISTER_OPERAND: api.MATRIX_CORE_REGISTER_OPERAND,
                                 api.KERNEL_MATRIX_CORE_LDS_STAGED: api.MATRIX_CORE_LDS_STAGED,
                                 api.KERNEL_MATRIX_CORE_K_STATIONARY: api.MATRIX_CORE_K_STATIONARY}
                                .get(kernel, api.MATRIX_CORE_AUTO))


def _describe(cand):
    knobs = ", ".join(f"{k}={v}" for k, v in cand.items() if k != "kernel" and v)
    return f"{_KERNEL_NAMES[cand.get('kernel', 0)]}({knobs})"


def save_table(path):
    """Writes every entry installed through this module as JSON."""
    with open(path, "w") as f:
        json.dump({"format": 1, "plans": [_installed[k] for k in sorted(_installed)]}, f, indent=1)


def load_table(path):
    """Installs every entry of a table written by save_table; returns how many."""
    with open(path) as f:
        table = json.load(f)
    if table.get("format") != 1:
        raise ValueError(f"{path}: not a tuned-plan table")
    for entry in table["plans"]:
        install(entry)
    return len(table["plans"])


def clear():
    api.clear_tuned_plans()
    _installed.clear()
