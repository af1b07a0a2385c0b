"""Builds the HIP library in-tree: mixed_gemv_amd/lib/libmixed_gemv_amd.so (gfx950 only)."""
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")   # objects and the compiler's intermediate files (the device assembly among them)
LIB_PATH = os.path.join(LIB_DIR, "libmixed_gemv_amd.so")
LINT_REPORT = os.path.join(LIB_DIR, "isa_lint.json")
MIN_DOT_INSTRUCTIONS = 10000

# One translation unit per family of kernel instantiations, so that they compile side by side.
SOURCES = ["launch_valu_f16.hip", "launch_valu_bf16.hip", "launch_mfma.hip", "launch_mfma_kstat.hip", "gemv_kernels.hip", "probes.hip",
           "host_utils.cpp"]

# -ffp-contract=off: the dequantiser is a separately rounded fp16 multiply and add.
# -packed-fp32-ops off: keep the compiler from forming v_pk_*_f32.
# -amdgpu-kernarg-preload-count=14: the first 14 dwords of kernel arguments arrive in SGPRs with
# the wave (measured: 0.1 us off the 4 us launches).
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-fvisibility=hidden", "-DMGEMV_BUILDING_LIBRARY", "-fopenmp",
    "-Wall", "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def lint_device_code(verbose=True):
    """Runs isa_lint over the device assembly the compiler left beside the objects and writes the
    report next to the library; raises if the compiled code has a hazard the compiler cannot see."""
    import glob
    import json
    from . import isa_lint
    files = sorted(glob.glob(os.path.join(OBJ_DIR, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if not files:
        raise RuntimeError(f"isa_lint: no device assembly (*-hip-amdgcn-amd-amdhsa-gfx950.s) under {OBJ_DIR}: "
                           "the compiled kernels cannot be checked")
    reports = [isa_lint.lint_file(f) for f in files]
    with open(LINT_REPORT, "w") as f:
        json.dump(reports, f, indent=1)
    bad = sum(len(r["findings"]) for r in reports)
    if verbose:
        print(f"isa_lint: {sum(r['dot_instructions'] for r in reports)} dot instructions in "
              f"{sum(r['kernels_with_dots'] for r in reports)} kernels of {len(files)} files, {bad} findings", flush=True)
    if bad:
        raise RuntimeError(f"isa_lint: {bad} hazards in the compiled kernels, see {LINT_REPORT}")
    # the VALU kernels alone hold tens of thousands of dot instructions: a check that saw (almost) none checked nothing
    if sum(r["dot_instructions"] for r in reports) < MIN_DOT_INSTRUCTIONS:
        raise RuntimeError(f"isa_lint: only {sum(r['dot_instructions'] for r in reports)} dot instructions found in "
                           f"{len(files)} files; the check did not see the kernels")
    return reports


DEFAULT_PLANS = os.path.join(PKG_DIR, "default_plans.json")
KERNEL_IDS = {"auto": 0, "valu": 1, "matrix_core_register_operand": 2, "matrix_core_lds_staged": 3,
              "matrix_core_k_stationary": 4}


def write_default_plans(path):
    """default_plans.json -> the initialiser list of the library's built-in tuned-plan table
    (one mgemv_tuned_plan per line), included by csrc/gemv_kernels.hip."""
    import json
    with open(DEFAULT_PLANS) as f:
        table = json.load(f)
    if table.get("format") != 1:
        raise RuntimeError(f"{DEFAULT_PLANS}: not a tuned-plan table")
    lines = []
    for e in table["plans"]:
        kernel = e.get("kernel", 0)
        kernel = KERNEL_IDS[kernel] if isinstance(kernel, str) else int(kernel)
        element = 1 if e.get("element", "f16") == "bf16" else 0
        fields = [e["n_out"], e["k"], e["weight_bits"], e["group_size"], e["m_batch"], kernel, e.get("split_k", 0),
                  e.get("tiles_per_wg", 0), e.get("tiles_per_wave", 0), e.get("max_workgroups", 0), e.get("stages", 0),
                  element]
        lines.append("{" + ", ".join(str(int(v)) for v in fields) + "},")
    text = "// generated from mixed_gemv_amd/default_plans.json by mixed_gemv_amd/build.py\n" + "\n".join(lines) + "\n"
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)
    return len(lines)


def build_library(verbose=True, extra_flags=(), jobs=None, lint=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    write_default_plans(os.path.join(OBJ_DIR, "default_plans.inc"))
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 16)

    def compile_one(src):
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc(), *HIP_FLAGS, *extra_flags, "-save-temps=obj", "-I", os.path.join(REPO_DIR, "include"), "-I", CSRC,
               "-I", OBJ_DIR, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fopenmp", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    if lint:
        lint_device_code(verbose)
    return LIB_PATH


if __name__ == "__main__":
    build_library(extra_flags=tuple(sys.argv[1:]))
