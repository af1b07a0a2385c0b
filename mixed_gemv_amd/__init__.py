"""MI355X-native weight-only-quantised GEMV (int4/int8 weights x fp16 activations).

Python mirror of the reference's host-side interface (names and argument meaning follow
mixed_gemv_test.cu, utils/preprocess.h and gemv/device/gemv_adaptor.h of
JJXiangJiaoJun/mixed_gemv) on top of the C-ABI in include/mixed_gemv.h.
"""
from .api import (  # noqa: F401
    GemvAdaptor,
    LayoutType,
    MixedGemvWeightPreprocessor,
    QuantType,
    SubBytePacker,
    WeightOnlyQuantOp,
    ZeroPointPreprocessor,
    dequantize,
    device_gemv,
    device_gemv_routed,
    gemv_arguments,
    host_gemv,
    static_scratch_bytes_needed,
    STATIC_SCRATCH_BYTES,
    probe_empty_grid,
    probe_empty_launch,
    probe_gemv,
    probe_gemv_rows,
    probe_stream_read,
    PROBE_COMPUTE_ONLY,
    PROBE_LOADS_ONLY,
    PROBE_TIMELINE,
    PROBE_TIMELINE_WAITS,
    PROBE_TIMELINE_WORDS,
    preprocessed_size,
    plan_coverage,
    query_launch,
    set_launch_override,
    set_matrix_core_threshold,
    set_dequant_form,
    set_prefetch_stages,
    set_matrix_core_variant,
    MATRIX_CORE_AUTO,
    MATRIX_CORE_REGISTER_OPERAND,
    MATRIX_CORE_LDS_STAGED,
    MATRIX_CORE_K_STATIONARY,
    DEQUANT_AUTO,
    DEQUANT_EXACT_INTEGER,
    unpreprocess_weights,
    erase_tuned_plan,
    set_tuned_plan,
    clear_tuned_plans,
    default_plan_count,
    set_default_plans,
    tuned_plan_count,
    KERNEL_AUTO,
    KERNEL_VALU,
    KERNEL_MATRIX_CORE_REGISTER_OPERAND,
    KERNEL_MATRIX_CORE_LDS_STAGED,
    KERNEL_MATRIX_CORE_K_STATIONARY,
)
from . import autotune  # noqa: F401
from ._lib import LIB_PATH, MixedGemvError  # noqa: F401

__version__ = "0.1.0"
