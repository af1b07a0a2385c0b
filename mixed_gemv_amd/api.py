"""Host-side mirror of the reference's operator interface, bound to the C-ABI.

Host utilities take and return numpy arrays.  Device entry points take anything exposing a
device address: a torch tensor on the GPU, or a plain integer address.  PyTorch is used only
as the owner of device memory and streams.
"""
import ctypes
import enum

import numpy as np

from . import _lib


class WeightOnlyQuantOp(enum.IntEnum):
    """gemv/weight_only_quant_op.h:12-18"""
    UNDEFINED = 0
    PER_COLUMN_SCALE_ONLY = 1
    FINEGRAINED_SCALE_ONLY = 2
    FINEGRAINED_SCALE_AND_ZEROS = 3


class QuantType(enum.IntEnum):
    """utils/type_base.h:7-11"""
    W8_A16 = 0
    W4_A16 = 1
    W4_AFP8 = 2


class LayoutType(enum.IntEnum):
    """utils/type_base.h:13-16"""
    kRowMajor = 0
    kColumnMajor = 1


def _host_ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def _dev_ptr(t):
    if t is None:
        return ctypes.c_void_p(0)
    if isinstance(t, int):
        return ctypes.c_void_p(t)
    if hasattr(t, "data_ptr"):
        if not t.is_cuda:
            raise ValueError("device entry points need GPU tensors; there is no CPU path")
        if not t.is_contiguous():
            raise ValueError("tensors must be contiguous")
        return ctypes.c_void_p(t.data_ptr())
    raise TypeError(f"cannot take a device address from {type(t)!r}")


def _is_bf16(element, probe):
    """element: "f16", "bf16" or None = take it from the dtype of a torch tensor operand (the
    reference's ElementB / ElementScale / ElementOutput template arguments)."""
    if element is None:
        dtype = getattr(probe, "dtype", None)
        return dtype is not None and str(dtype) == "torch.bfloat16"
    if element not in ("f16", "bf16"):
        raise ValueError("element must be 'f16', 'bf16' or None")
    return element == "bf16"


def _stream_ptr(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def _shape_arg(shape):
    shape = [int(s) for s in shape]
    return (ctypes.c_size_t * len(shape))(*shape), len(shape)


class SubBytePacker:
    """utils/preprocess.h:16-85 for <int4b_t, int8_t>."""

    @staticmethod
    def pack(unpacked):
        unpacked = np.ascontiguousarray(unpacked, dtype=np.int8).reshape(-1)
        packed = np.empty(unpacked.size // 2, dtype=np.uint8)
        _lib.check(_lib.lib().mgemv_pack_int4(_host_ptr(packed), _host_ptr(unpacked), unpacked.size), "pack")
        return packed

    @staticmethod
    def unpack(packed):
        packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
        unpacked = np.empty(packed.size * 2, dtype=np.int8)
        _lib.check(_lib.lib().mgemv_unpack_int4(_host_ptr(unpacked), _host_ptr(packed), packed.size), "unpack")
        return unpacked


class ZeroPointPreprocessor:
    """utils/preprocess.h:88-102"""

    @staticmethod
    def neg_zero_point_multiplies_scale(scales, zeros, element="f16"):
        """element="bf16": scales and result are bfloat16 bit patterns in uint16 arrays."""
        s = np.ascontiguousarray(scales)
        if s.dtype == np.float16 and element == "f16":
            s = s.view(np.uint16)
        if s.dtype != np.uint16:
            raise TypeError("scales must be float16 (or uint16 bit patterns of the element type)")
        z = np.ascontiguousarray(zeros, dtype=np.int8)
        if z.size != s.size:
            raise ValueError("scales and zeros differ in size")
        out = np.empty(s.shape, dtype=np.uint16)
        if _is_bf16(element, None):
            _lib.check(_lib.lib().mgemv_fold_zero_points_bf16(_host_ptr(out), _host_ptr(s), _host_ptr(z), s.size), "fold")
            return out
        _lib.check(_lib.lib().mgemv_fold_zero_points(_host_ptr(out), _host_ptr(s), _host_ptr(z), s.size), "fold")
        return out.view(np.float16)


def preprocessed_size(shape, quant_type):
    arr, rank = _shape_arg(shape)
    return int(_lib.lib().mgemv_preprocessed_size(arr, rank, int(quant_type)))


class MixedGemvWeightPreprocessor:
    """utils/preprocess.h:480-524.  Same arguments; returns the preprocessed bytes (the
    buffer may be larger than the input because rows and k are padded to whole tiles)."""

    @staticmethod
    def run(quantized_weight, shape, weight_layout=LayoutType.kColumnMajor, quant_type=QuantType.W4_A16,
            force_interleave=False):
        del force_interleave  # accepted and ignored, as in the reference (utils/preprocess.h:484)
        src = np.ascontiguousarray(quantized_weight).reshape(-1).view(np.uint8)
        arr, rank = _shape_arg(shape)
        size = int(_lib.lib().mgemv_preprocessed_size(arr, rank, int(quant_type)))
        if rank in (2, 3) and int(quant_type) in (0, 1):
            n_elem = int(np.prod([int(s) for s in shape]))
            need = n_elem * (4 if int(quant_type) == QuantType.W4_A16 else 8) // 8
            if src.size < need:
                raise ValueError(f"weight buffer holds {src.size} bytes, shape needs {need}")
        dst = np.empty(max(size, 1), dtype=np.uint8)
        _lib.check(_lib.lib().mgemv_preprocess_weights(_host_ptr(dst), _host_ptr(src), arr, rank,
                                                       int(weight_layout), int(quant_type)), "preprocess")
        return dst[:size]


def unpreprocess_weights(preprocessed, shape, quant_type=QuantType.W4_A16):
    src = np.ascontiguousarray(preprocessed, dtype=np.uint8).reshape(-1)
    arr, rank = _shape_arg(shape)
    n_elem = int(np.prod([int(s) for s in shape]))
    bits = 4 if int(quant_type) == QuantType.W4_A16 else 8
    dst = np.empty(n_elem * bits // 8, dtype=np.uint8)
    _lib.check(_lib.lib().mgemv_unpreprocess_weights(_host_ptr(dst), _host_ptr(src), arr, rank, int(quant_type)),
               "unpreprocess")
    return dst


class _Arguments(ctypes.Structure):
    """mgemv_arguments (include/mixed_gemv.h)."""
    _fields_ = [("n_out", ctypes.c_int), ("m_batch", ctypes.c_int), ("k", ctypes.c_int),
                ("weights", ctypes.c_void_p), ("lda", ctypes.c_int64),
                ("x", ctypes.c_void_p), ("ldb", ctypes.c_int64),
                ("scale", ctypes.c_void_p), ("ld_scale", ctypes.c_int64),
                ("zero_add", ctypes.c_void_p), ("ld_zero", ctypes.c_int64),
                ("bias", ctypes.c_void_p), ("ldc", ctypes.c_int64),
                ("y", ctypes.c_void_p), ("ldd", ctypes.c_int64),
                ("alpha", ctypes.c_float), ("beta", ctypes.c_float),
                ("group_size", ctypes.c_int), ("batch_count", ctypes.c_int),
                ("batch_stride_weights", ctypes.c_int64), ("batch_stride_x", ctypes.c_int64),
                ("batch_stride_scale", ctypes.c_int64), ("batch_stride_bias", ctypes.c_int64),
                ("batch_stride_y", ctypes.c_int64),
                ("quant_op", ctypes.c_int), ("weight_bits", ctypes.c_int), ("element", ctypes.c_int)]


def gemv_arguments(ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_C, ptr_D, M, N, K, group_size, quant_op, weight_bits=4,
                   alpha=1.0, beta=1.0, leading_dims=None, batch_count=1, batch_strides=None, stream=None, element=None):
    """GemvAdaptor::Arguments + operator() in one call (mgemv_gemv_arguments): the epilogue's alpha and
    beta, and the reference's leading dimensions (lda, ldb, ld_scale, ld_zero, ldc, ldd; None = dense)."""
    lda, ldb, lds, ldz, ldc, ldd = leading_dims or (0, int(K) if int(N) > 1 else 0, 0, 0, 0, 0)
    sa, sb, ss, sc, sd = batch_strides or (0, 0, 0, 0, 0)
    val = lambda p: _dev_ptr(p).value  # noqa: E731
    a = _Arguments(int(M), int(N), int(K), val(ptr_A), int(lda), val(ptr_B), int(ldb), val(ptr_scale), int(lds),
                   val(ptr_zero_point), int(ldz), val(ptr_C), int(ldc), val(ptr_D), int(ldd), float(alpha), float(beta),
                   int(group_size), int(batch_count), int(sa), int(sb), int(ss), int(sc), int(sd), int(quant_op),
                   int(weight_bits), 1 if _is_bf16(element, ptr_B) else 0)
    _lib.check(_lib.lib().mgemv_gemv_arguments(ctypes.byref(a), _stream_ptr(stream)), "gemv_arguments")


STATIC_SCRATCH_BYTES = 16 << 20


def static_scratch_bytes_needed(M, N, K, group_size, quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS,
                                weight_bits=4, has_bias=False):
    """Bytes of the static arrays host_gemv(..., static_scratch=True) would use; 0 for an illegal problem."""
    return int(_lib.lib().mgemv_static_scratch_bytes_needed(int(M), int(N), int(K), int(group_size), int(quant_op),
                                                            int(weight_bits), 1 if has_bias else 0))


def host_gemv(ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_C, B, M, N, K, group_size,
              quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS, weight_bits=4, static_scratch=False):
    """host_gemv of mixed_gemv_test.cu:167-181, i.e. host::reference::MixedGemv::operator()
    (host/mixed_gemv.h:60-70), with the GPU behind it: numpy arrays in host memory, UN-preprocessed
    packed weights [M][K], int8 zero points [K/group_size][M] (mode 3), optional fp16 bias.  Returns
    the fp16 result [N][M].  There is no CPU path: without a gfx950 device this raises.
    static_scratch=True calls mgemv_host_gemv_static, which allocates nothing (problems up to
    STATIC_SCRATCH_BYTES of staging)."""
    w = np.ascontiguousarray(ptr_A).reshape(-1).view(np.uint8)
    x = np.ascontiguousarray(ptr_B, dtype=np.float16)
    s = np.ascontiguousarray(ptr_scale, dtype=np.float16)
    z = None if ptr_zero_point is None else np.ascontiguousarray(ptr_zero_point, dtype=np.int8)
    b = None if ptr_C is None else np.ascontiguousarray(ptr_C, dtype=np.float16)
    need = int(M) * int(K) * int(weight_bits) // 8
    if w.size < need or x.size < int(N) * int(K):
        raise ValueError("operand smaller than the problem")
    y = np.empty((int(N), int(M)), dtype=np.float16)
    null = ctypes.c_void_p(0)
    fn = _lib.lib().mgemv_host_gemv_static if static_scratch else _lib.lib().mgemv_host_gemv
    st = fn(int(B), int(M), int(N), int(K), int(group_size), _host_ptr(w), _host_ptr(x), _host_ptr(s),
            _host_ptr(z) if z is not None else null, _host_ptr(b) if b is not None else null, _host_ptr(y),
            int(quant_op), int(weight_bits))
    _lib.check(st, "host_gemv")
    return y


def device_gemv(ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_C, ptr_D, B, M, N, K, group_size,
                quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS, weight_bits=4, stream=None,
                batch_strides=None, element=None):
    """mixed_gemv_test.cu:124-165.  Reference letters: M = output features, N = activation
    rows, K = reduction, B = batch count.  ptr_A is the PREPROCESSED weight buffer,
    ptr_zero_point the folded fp16 term -z*s, ptr_C an optional fp16 bias.  The quant mode is
    a run-time argument (a compile-time constant in the reference).  element: "f16" / "bf16" for
    every 16-bit operand; None takes it from ptr_B when that is a torch tensor, else fp16."""
    bf16 = _is_bf16(element, ptr_B)
    gemv = _lib.lib().mgemv_gemv_bf16 if bf16 else _lib.lib().mgemv_gemv
    gemv_batched = _lib.lib().mgemv_gemv_batched_bf16 if bf16 else _lib.lib().mgemv_gemv_batched
    if B == 1 and not batch_strides:
        st = gemv(_dev_ptr(ptr_A), _dev_ptr(ptr_B), _dev_ptr(ptr_scale), _dev_ptr(ptr_zero_point),
                                   _dev_ptr(ptr_C), _dev_ptr(ptr_D), int(M), int(N), int(K), int(group_size),
                                   int(quant_op), int(weight_bits), _stream_ptr(stream))
    else:
        sa, sb, ss, sc, sd = batch_strides or (0, 0, 0, 0, 0)
        st = gemv_batched(_dev_ptr(ptr_A), _dev_ptr(ptr_B), _dev_ptr(ptr_scale),
                          _dev_ptr(ptr_zero_point), _dev_ptr(ptr_C), _dev_ptr(ptr_D), int(B), int(M),
                          int(N), int(K), int(group_size), int(quant_op), int(weight_bits),
                          int(sa), int(sb), int(ss), int(sc), int(sd), _stream_ptr(stream))
    _lib.check(st, "device_gemv")


def device_gemv_routed(ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_C, ptr_D, route, stack_entries, B, M, N, K,
                       group_size, batch_strides, quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS,
                       weight_bits=4, stream=None, element=None):
    """device_gemv over an expert stack (the 3-D shapes of utils/preprocess.h:134-136), routed: problem
    b of B takes the weights, scales, zeros and bias of entry route[b] (a DEVICE array of int32) of the
    stack of stack_entries matrices; x and y are stepped by b.  batch_strides = (weights in bytes, x,
    scale, bias, y) as in device_gemv; a stride of 0 for x gives every problem the same activations.
    The reference steps through a stack at a fixed stride only (gemv/kernel/mixed_gemv.h:140-149)."""
    fn = _lib.lib().mgemv_gemv_routed_bf16 if _is_bf16(element, ptr_B) else _lib.lib().mgemv_gemv_routed
    sa, sb, ss, sc, sd = batch_strides
    st = fn(_dev_ptr(ptr_A), _dev_ptr(ptr_B), _dev_ptr(ptr_scale), _dev_ptr(ptr_zero_point), _dev_ptr(ptr_C),
            _dev_ptr(ptr_D), _dev_ptr(route), int(stack_entries), int(B), int(M), int(N), int(K), int(group_size),
            int(quant_op), int(weight_bits), int(sa), int(sb), int(ss), int(sc), int(sd), _stream_ptr(stream))
    _lib.check(st, "device_gemv_routed")


class GemvAdaptor:
    """gemv/device/gemv_adaptor.h:114-261: Arguments / initialize / run / __call__."""

    class Arguments:
        def __init__(self, problem_size, ref_A, ref_B, ref_scale, ref_zero_point, ref_C, ref_D, group_size=64,
                     batch_count=1, batch_stride_A=0, batch_stride_B=0, batch_stride_scale=0, batch_stride_C=0,
                     batch_stride_D=0):
            self.problem_size = tuple(int(v) for v in problem_size)  # (M, N, K)
            self.ref_A, self.ref_B, self.ref_scale = ref_A, ref_B, ref_scale
            self.ref_zero_point, self.ref_C, self.ref_D = ref_zero_point, ref_C, ref_D
            self.group_size, self.batch_count = int(group_size), int(batch_count)
            self.batch_strides = (batch_stride_A, batch_stride_B, batch_stride_scale, batch_stride_C, batch_stride_D)

    def __init__(self, quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS, weight_bits=4, element=None):
        """element: "f16" / "bf16" (the reference's ElementB / ElementScale / ElementOutput), None = from ref_B."""
        self.quant_op, self.weight_bits, self.element = WeightOnlyQuantOp(quant_op), int(weight_bits), element
        self._args = None

    def initialize(self, args, stream=None):
        del stream
        if self.quant_op != WeightOnlyQuantOp.PER_COLUMN_SCALE_ONLY and args.group_size < 64:
            # gemv_adaptor.h:199-203 prints and exits; here it is an error
            raise _lib.MixedGemvError(5, "GemvAdaptor.initialize")
        self._args = args

    def run(self, stream=None):
        a = self._args
        if a is None:
            raise RuntimeError("GemvAdaptor.run before initialize")
        m, n, k = a.problem_size
        zero = a.ref_zero_point if self.quant_op == WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS else None
        device_gemv(a.ref_A, a.ref_B, a.ref_scale, zero, a.ref_C, a.ref_D, a.batch_count, m, n, k, a.group_size,
                    self.quant_op, self.weight_bits, stream,
                    a.batch_strides if (a.batch_count != 1 or any(a.batch_strides)) else None, self.element)

    def __call__(self, args, stream=None):
        self.initialize(args, stream)
        self.run(stream)


def dequantize(ptr_A, ptr_scale, ptr_zero_point, ptr_out, M, K, group_size,
               quant_op=WeightOnlyQuantOp.FINEGRAINED_SCALE_AND_ZEROS, weight_bits=4, stream=None, element=None):
    """Writes dequantised weights [M][K] (fp16, or bf16 with element="bf16" / a torch.bfloat16 scale
    tensor) with the kernels' own converter + dequantiser."""
    fn = _lib.lib().mgemv_dequantize_bf16 if _is_bf16(element, ptr_scale) else _lib.lib().mgemv_dequantize
    st = fn(_dev_ptr(ptr_A), _dev_ptr(ptr_scale), _dev_ptr(ptr_zero_point), _dev_ptr(ptr_out),
                                     int(M), int(K), int(group_size), int(quant_op), int(weight_bits),
                                     _stream_ptr(stream))
    _lib.check(st, "dequantize")


def set_launch_override(split_k_waves=0, tiles_per_workgroup=0, tiles_per_wave=0, max_workgroups=0):
    _lib.check(_lib.lib().mgemv_set_launch_override(int(split_k_waves), int(tiles_per_workgroup), int(tiles_per_wave),
                                                    int(max_workgroups)), "set_launch_override")


def set_matrix_core_threshold(min_m_batch=0):
    _lib.check(_lib.lib().mgemv_set_matrix_core_threshold(int(min_m_batch)), "set_matrix_core_threshold")


MATRIX_CORE_AUTO = 0
MATRIX_CORE_REGISTER_OPERAND = 1
MATRIX_CORE_LDS_STAGED = 2
MATRIX_CORE_K_STATIONARY = 3


def set_matrix_core_variant(variant=MATRIX_CORE_AUTO):
    """Which matrix-core kernel serves the small batches; see mgemv_set_matrix_core_variant."""
    _lib.check(_lib.lib().mgemv_set_matrix_core_variant(int(variant)), "set_matrix_core_variant")


DEQUANT_AUTO = 0
DEQUANT_EXACT_INTEGER = 1


def set_dequant_form(form=DEQUANT_AUTO):
    """Which int4 dequantiser the kernels may use (same bits either way); see mgemv_set_dequant_form."""
    _lib.check(_lib.lib().mgemv_set_dequant_form(int(form)), "set_dequant_form")


def query_launch(n_out, m_batch, k, weight_bits=4, group_size=0, element="f16", num_compute_units=None):
    """The geometry mgemv_gemv (element="bf16": mgemv_gemv_bf16) would use on an unpartitioned MI355X, or on
    a device of num_compute_units compute units; group_size as passed to the GEMV (it only selects tuned
    plans)."""
    if num_compute_units is None:
        out = (ctypes.c_int * 8)()
        fn = _lib.lib().mgemv_query_launch_bf16 if _is_bf16(element, None) else _lib.lib().mgemv_query_launch
        _lib.check(fn(int(n_out), int(m_batch), int(k), int(weight_bits), int(group_size), ctypes.byref(out)),
                   "query_launch")
    else:
        out = (ctypes.c_int * 12)()
        _lib.check(_lib.lib().mgemv_query_launch_for(int(n_out), int(m_batch), int(k), int(weight_bits),
                                                     int(group_size), 1 if _is_bf16(element, None) else 0,
                                                     int(num_compute_units), ctypes.byref(out)), "query_launch")
    keys = ("workgroups", "threads", "split_k", "tiles_per_wg", "steps_per_wave", "matrix_core", "tiles_per_wave",
            "tiles_in_sequence", "lds_bytes", "max_threads", "stages", "launches")
    return dict(zip(keys, list(out)))


def plan_coverage(n_out, m_batch, k, weight_bits=4, group_size=0, element="f16", num_compute_units=256):
    """Host replay of every wave's index arithmetic for the launch plan of this problem (mgemv_plan_coverage)."""
    out = (ctypes.c_int64 * 8)()
    _lib.check(_lib.lib().mgemv_plan_coverage(int(n_out), int(m_batch), int(k), int(weight_bits), int(group_size),
                                              1 if _is_bf16(element, None) else 0, int(num_compute_units),
                                              ctypes.byref(out)), "plan_coverage")
    keys = ("tiles_miscovered", "bad_waves", "max_descriptor_bytes", "lds_bytes_used", "lds_bytes", "busy_waves",
            "idle_waves", "max_units_per_wave")
    return dict(zip(keys, list(out)))


def set_prefetch_stages(stages):
    """1: the VALU kernel waits for every load before it computes; 2: the next unit's loads are in flight
    meanwhile; 0: built-in choice (mgemv_set_prefetch_stages)."""
    _lib.check(_lib.lib().mgemv_set_prefetch_stages(int(stages)), "set_prefetch_stages")


def probe_gemv_rows(kind, N, ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_D, M, K, group_size, stream=None):
    """PROBE_LOADS_ONLY / PROBE_COMPUTE_ONLY builds for a launch of N activation rows (mgemv_probe_gemv_rows)."""
    _lib.check(_lib.lib().mgemv_probe_gemv_rows(int(kind), int(N), _dev_ptr(ptr_A), _dev_ptr(ptr_B), _dev_ptr(ptr_scale),
                                                _dev_ptr(ptr_zero_point), _dev_ptr(ptr_D), int(M), int(K), int(group_size),
                                                _stream_ptr(stream)), "probe_gemv_rows")


PROBE_LOADS_ONLY = 1
PROBE_TIMELINE = 2
PROBE_COMPUTE_ONLY = 3
PROBE_TIMELINE_WAITS = 4


def probe_empty_launch(stream=None):
    """One empty kernel launch (mgemv_probe_empty_launch)."""
    _lib.check(_lib.lib().mgemv_probe_empty_launch(_stream_ptr(stream)), "probe_empty_launch")


def probe_empty_grid(workgroups, waves_per_workgroup, stream=None):
    """An empty kernel with the given grid (mgemv_probe_empty_grid)."""
    _lib.check(_lib.lib().mgemv_probe_empty_grid(int(workgroups), int(waves_per_workgroup), _stream_ptr(stream)),
               "probe_empty_grid")


def probe_stream_read(src, nbytes, workgroups, waves_per_workgroup, units_in_flight, sink=None, stream=None):
    """Plain streaming read of nbytes at src with the GEMV's weight loads (mgemv_probe_stream_read)."""
    _lib.check(_lib.lib().mgemv_probe_stream_read(_dev_ptr(src), int(nbytes), int(workgroups), int(waves_per_workgroup),
                                                  int(units_in_flight), _dev_ptr(sink), _stream_ptr(stream)),
               "probe_stream_read")


PROBE_TIMELINE_WORDS = 14


def probe_gemv(kind, trace, ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_D, M, K, group_size, stream=None):
    """Measurement builds of the headline kernel (mgemv_probe_gemv): PROBE_LOADS_ONLY, PROBE_COMPUTE_ONLY or PROBE_TIMELINE
    (trace: int64 device tensor of PROBE_TIMELINE_WORDS entries per wave; its size is passed on as the capacity, and a
    launch of more waves than it holds is refused)."""
    capacity = 0 if trace is None else int(trace.numel()) // PROBE_TIMELINE_WORDS
    _lib.check(_lib.lib().mgemv_probe_gemv(int(kind), _dev_ptr(trace), capacity, _dev_ptr(ptr_A), _dev_ptr(ptr_B),
                                           _dev_ptr(ptr_scale), _dev_ptr(ptr_zero_point), _dev_ptr(ptr_D), int(M), int(K),
                                           int(group_size), _stream_ptr(stream)), "probe_gemv")


KERNEL_AUTO = 0
KERNEL_VALU = 1
KERNEL_MATRIX_CORE_REGISTER_OPERAND = 2
KERNEL_MATRIX_CORE_LDS_STAGED = 3
KERNEL_MATRIX_CORE_K_STATIONARY = 4


def set_tuned_plan(n_out, k, weight_bits, group_size, m_batch, kernel=KERNEL_AUTO, split_k=0, tiles_per_wg=0,
                   tiles_per_wave=0, max_workgroups=0, stages=0, element="f16"):
    """Installs the launch plan for exactly this problem and element type; see mgemv_tuned_plan_set
    (group_size 0 = any)."""
    plan = (ctypes.c_int * 12)(int(n_out), int(k), int(weight_bits), int(group_size), int(m_batch), int(kernel),
                               int(split_k), int(tiles_per_wg), int(tiles_per_wave), int(max_workgroups), int(stages),
                               1 if _is_bf16(element, None) else 0)
    _lib.check(_lib.lib().mgemv_tuned_plan_set(ctypes.byref(plan)), "set_tuned_plan")


def erase_tuned_plan(n_out, k, weight_bits, group_size, m_batch, element="f16"):
    """Removes the table entry of exactly this key, if any (mgemv_tuned_plan_erase)."""
    plan = (ctypes.c_int * 12)(int(n_out), int(k), int(weight_bits), int(group_size), int(m_batch), 0, 0, 0, 0, 0, 0,
                               1 if _is_bf16(element, None) else 0)
    _lib.check(_lib.lib().mgemv_tuned_plan_erase(ctypes.byref(plan)), "erase_tuned_plan")


def set_default_plans(enable=True):
    """Switches the library's built-in tuned-plan table (default_plans.json) on or off."""
    _lib.check(_lib.lib().mgemv_set_default_plans(1 if enable else 0), "set_default_plans")


def default_plan_count():
    return int(_lib.lib().mgemv_default_plan_count())


def clear_tuned_plans():
    _lib.check(_lib.lib().mgemv_tuned_plan_clear(), "clear_tuned_plans")


def tuned_plan_count():
    return int(_lib.lib().mgemv_tuned_plan_count())
