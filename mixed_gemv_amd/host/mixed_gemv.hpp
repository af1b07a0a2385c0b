// C++ host-side mirror of the reference's call sites on top of the C-ABI (include/mixed_gemv.h).
//
// A caller of JJXiangJiaoJun/mixed_gemv uses three things: the host utilities of
// utils/preprocess.h (SubBytePacker, ZeroPointPreprocessor, MixedGemvWeightPreprocessor), the
// device adaptor of gemv/device/gemv_adaptor.h (Arguments / initialize / run), and the
// device_gemv wrapper of mixed_gemv_test.cu:124-165.  The classes below keep those names,
// argument orders and meanings, so a port is a change of namespace and of the half type
// (fp16 crosses this interface as uint16_t bit patterns; `half_t` here is that alias).
//
// Differences a caller sees, all deliberate:
//   * the quantisation mode and weight width are run-time constructor arguments of
//     GemvAdaptor (template parameters in the reference, one binary per mode);
//   * MixedGemvWeightPreprocessor::run writes preprocessed_size() bytes, which can exceed the
//     input size (rows padded to 16, k to one wave step); the layout is the gfx950 tile
//     layout, not RowMajorTileInterleave<8,4>;
//   * where the reference prints a message and calls exit(-1), these throw mixed_gemv::Error
//     carrying the C-ABI status (define MIXED_GEMV_EXIT_ON_ERROR to get print + exit(-1)).
#ifndef MIXED_GEMV_AMD_HOST_MIXED_GEMV_HPP_
#define MIXED_GEMV_AMD_HOST_MIXED_GEMV_HPP_

#include <cstdint>
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

#include "mixed_gemv.h"

namespace mixed_gemv {

using half_t = uint16_t;  // IEEE binary16 bit pattern

// gemv/weight_only_quant_op.h:12-18
enum class WeightOnlyQuantOp { UNDEFINED = 0, PER_COLUMN_SCALE_ONLY = 1, FINEGRAINED_SCALE_ONLY = 2, FINEGRAINED_SCALE_AND_ZEROS = 3 };
constexpr bool isFinegrained(WeightOnlyQuantOp op) { return op == WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS || op == WeightOnlyQuantOp::FINEGRAINED_SCALE_ONLY; }
constexpr bool hasZero(WeightOnlyQuantOp op) { return op == WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS; }

// utils/type_base.h:7-16
enum class QuantType { W8_A16 = 0, W4_A16 = 1, W4_AFP8 = 2 };
enum class LayoutType { kRowMajor = 0, kColumnMajor = 1 };
// The reference's ElementB = ElementScale = ElementOutput template arguments (host/mixed_gemv.h:24-31):
// what the 16-bit operands (typed half_t below) hold.
enum class ElementType { kFloat16 = 0, kBFloat16 = 1 };

class Error : public std::runtime_error {
 public:
  Error(int status, const std::string& where)
      : std::runtime_error(where + ": " + mgemv_status_string(status)), status_(status) {}
  int status() const { return status_; }

 private:
  int status_;
};

inline void check(int status, const char* where) {
  if (status == MGEMV_OK) return;
#ifdef MIXED_GEMV_EXIT_ON_ERROR
  std::cout << where << ": " << mgemv_status_string(status) << std::endl;
  std::exit(-1);
#else
  throw Error(status, where);
#endif
}

// utils/preprocess.h:16-85
struct SubBytePacker {
  static void unpack(int8_t* unpacked_output, const int8_t* packed_input, size_t packed_num_elements) {
    check(mgemv_unpack_int4(unpacked_output, reinterpret_cast<const uint8_t*>(packed_input), packed_num_elements), "SubBytePacker::unpack");
  }
  static void pack(int8_t* packed_output, const int8_t* unpacked_input, size_t unpacked_num_elements) {
    check(mgemv_pack_int4(reinterpret_cast<uint8_t*>(packed_output), unpacked_input, unpacked_num_elements), "SubBytePacker::pack");
  }
};

// utils/preprocess.h:88-102
struct ZeroPointPreprocessor {
  static void neg_zero_point_multiplies_scale(half_t* neg_zeros_x_scales, const half_t* scales, const int8_t* zeros, int n,
                                              ElementType element = ElementType::kFloat16) {
    check(element == ElementType::kBFloat16
              ? mgemv_fold_zero_points_bf16(neg_zeros_x_scales, scales, zeros, static_cast<size_t>(n))
              : mgemv_fold_zero_points(neg_zeros_x_scales, scales, zeros, static_cast<size_t>(n)),
          "ZeroPointPreprocessor");
  }
};

// utils/preprocess.h:480-524
struct MixedGemvWeightPreprocessor {
  static size_t preprocessed_size(const std::vector<size_t>& shape, QuantType quant_type) {
    return mgemv_preprocessed_size(shape.data(), static_cast<int>(shape.size()), static_cast<int>(quant_type));
  }
  // shape = {K, M} or {experts, K, M}; preprocessed_quantized_weight must hold preprocessed_size() bytes.
  static void run(int8_t* preprocessed_quantized_weight, const int8_t* quantized_weight, const std::vector<size_t>& shape,
                  LayoutType weight_layout, QuantType quant_type, bool /*force_interleave: ignored, as in the reference*/) {
    check(mgemv_preprocess_weights(reinterpret_cast<uint8_t*>(preprocessed_quantized_weight),
                                   reinterpret_cast<const uint8_t*>(quantized_weight), shape.data(),
                                   static_cast<int>(shape.size()), static_cast<int>(weight_layout), static_cast<int>(quant_type)),
          "MixedGemvWeightPreprocessor::run");
  }
};

struct GemmCoord {
  int m_, n_, k_;
  int m() const { return m_; }
  int n() const { return n_; }
  int k() const { return k_; }
};

template <typename T>
struct TensorRef {
  T* ptr;
  int ld;
  T* data() const { return ptr; }
  int stride() const { return ld; }
};

// cutlass::epilogue::thread::LinearCombination<...>::Params as the reference's Arguments carry it
// (gemv/device/gemv_adaptor.h:123; mixed_gemv_test.cu:72-81): D = alpha * accumulator + beta * C.
// The reference's `{}` is alpha = 1, beta = 0 with a scaling type that never reads C; here beta
// only matters when ref_C is set, and defaults to 1 so that ref_C is the bias of
// host/mixed_gemv.h:102-103.
struct EpilogueParams {
  float alpha = 1.0f;
  float beta = 1.0f;
};

// gemv/device/gemv_adaptor.h:114-261.  Reference letters: M = output features, N = activation
// rows, K = reduction.  The operands are dense: a leading dimension must be 0 or the value the
// reference's caller passes (ref_A 4K, ref_B 0 for one row or K, the others M); any other value
// is refused with MGEMV_ERR_LEADING_DIMENSION instead of being ignored.
class GemvAdaptor {
 public:
  struct Arguments {
    GemmCoord problem_size;
    TensorRef<const void> ref_A;             // PREPROCESSED weights
    TensorRef<const half_t> ref_B;           // activations
    TensorRef<const half_t> ref_scale;
    TensorRef<const half_t> ref_zero_point;  // folded -z*s
    TensorRef<const half_t> ref_C;           // optional bias, nullptr = none
    TensorRef<half_t> ref_D;
    EpilogueParams epilogue;
    int group_size = 64;
    int batch_count = 1;
    long long batch_stride_A = 0;            // BYTES of the preprocessed buffer
    long long batch_stride_B = 0, batch_stride_scale = 0, batch_stride_C = 0, batch_stride_D = 0;  // elements
  };

  GemvAdaptor(WeightOnlyQuantOp quant_op = WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS, int weight_bits = 4,
              ElementType element = ElementType::kFloat16)
      : quant_op_(quant_op), weight_bits_(weight_bits), element_(element) {}

  void initialize(const Arguments& args, void* /*stream*/ = nullptr) {
    // gemv_adaptor.h:199-203
    if (quant_op_ != WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY && args.group_size < 64) check(MGEMV_ERR_GROUP_SIZE, "GemvAdaptor::initialize");
    args_ = args;
    initialized_ = true;
  }

  void run(void* stream = nullptr) {
    if (!initialized_) throw std::logic_error("GemvAdaptor::run before initialize");
    const Arguments& a = args_;
    mgemv_arguments c{};
    c.n_out = a.problem_size.m();
    c.m_batch = a.problem_size.n();
    c.k = a.problem_size.k();
    c.weights = a.ref_A.ptr;
    c.lda = a.ref_A.ld;
    c.x = a.ref_B.ptr;
    c.ldb = a.ref_B.ld == 0 && c.m_batch > 1 ? c.k : a.ref_B.ld;  // the reference's stride-0 single row, repeated per row
    c.scale = a.ref_scale.ptr;
    c.ld_scale = a.ref_scale.ld;
    c.zero_add = hasZero(quant_op_) ? a.ref_zero_point.ptr : nullptr;  // mixed_gemv_test.cu:145-147
    c.ld_zero = a.ref_zero_point.ld;
    c.bias = a.ref_C.ptr;
    c.ldc = a.ref_C.ld;
    c.y = a.ref_D.ptr;
    c.ldd = a.ref_D.ld;
    c.alpha = a.epilogue.alpha;
    c.beta = a.epilogue.beta;
    c.group_size = a.group_size;
    c.batch_count = a.batch_count;
    c.batch_stride_weights = a.batch_stride_A;
    c.batch_stride_x = a.batch_stride_B;
    c.batch_stride_scale = a.batch_stride_scale;
    c.batch_stride_bias = a.batch_stride_C;
    c.batch_stride_y = a.batch_stride_D;
    c.quant_op = static_cast<int>(quant_op_);
    c.weight_bits = weight_bits_;
    c.element = element_ == ElementType::kBFloat16 ? MGEMV_ELEMENT_BF16 : MGEMV_ELEMENT_F16;
    check(mgemv_gemv_arguments(&c, stream), "GemvAdaptor::run");
  }

  void operator()(const Arguments& args, void* stream = nullptr) {
    initialize(args, stream);
    run(stream);
  }

  // gemv/device/gemv_adaptor.h:190-196 (get_grid_size / get_block_size of Params).  The reference's
  // launch shape is a compile-time function of the problem's rows (ceil(M / 64) blocks of 128
  // threads); here it is the launch plan of the problem (mgemv_query_launch_for: built-in rules,
  // tuned plans, overrides), so both take the arguments and, since the plan is made for the
  // compute units of the device the launch goes to, that count (256: an unpartitioned MI355X).
  struct Dim3 {
    unsigned x, y, z;
  };
  Dim3 get_grid_size(const Arguments& args, int num_compute_units = 256) const {
    const LaunchShape s = launch_shape(args, num_compute_units);
    return Dim3{(unsigned)((s.workgroups + 7) / 8 * 8), 1u, (unsigned)args.batch_count};  // whole rounds over the 8 XCDs
  }
  Dim3 get_block_size(const Arguments& args, int num_compute_units = 256) const {
    const LaunchShape s = launch_shape(args, num_compute_units);
    return Dim3{(unsigned)(64 * s.k_split_waves), (unsigned)s.tiles_per_workgroup, 1u};
  }

 private:
  struct LaunchShape {
    int workgroups, k_split_waves, tiles_per_workgroup;
  };
  LaunchShape launch_shape(const Arguments& a, int num_compute_units) const {
    int out[12] = {0};
    const int group = quant_op_ == WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY ? a.problem_size.k() : a.group_size;
    check(mgemv_query_launch_for(a.problem_size.m(), a.problem_size.n(), a.problem_size.k(), weight_bits_, group,
                                 element_ == ElementType::kBFloat16 ? MGEMV_ELEMENT_BF16 : MGEMV_ELEMENT_F16,
                                 num_compute_units, out),
          "GemvAdaptor::get_grid_size");
    return LaunchShape{out[0], out[2], out[3]};
  }

  WeightOnlyQuantOp quant_op_;
  int weight_bits_;
  ElementType element_;
  Arguments args_{};
  bool initialized_ = false;
};

// mixed_gemv_test.cu:124-165.  Same argument order; the quant mode, a compile-time constant in
// the reference, and the stream are trailing arguments.
inline void device_gemv(const void* ptr_A, const half_t* ptr_B, const half_t* ptr_scale, const half_t* ptr_zero_point,
                        const half_t* ptr_C, half_t* ptr_D, int B, int M, int N, int K, int group_size,
                        WeightOnlyQuantOp quant_op = WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS, int weight_bits = 4,
                        void* stream = nullptr, ElementType element = ElementType::kFloat16) {
  if (quant_op == WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY) group_size = K;            // :142-143
  if (quant_op != WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS) ptr_zero_point = nullptr;  // :145-147
  GemvAdaptor::Arguments args;
  args.problem_size = GemmCoord{M, N, K};
  args.ref_A = {ptr_A, K * 4};
  args.ref_B = {ptr_B, 0};
  args.ref_scale = {ptr_scale, M};
  args.ref_zero_point = {ptr_zero_point, M};
  args.ref_C = {ptr_C, M};
  args.ref_D = {ptr_D, M};
  args.group_size = group_size;
  args.batch_count = B;
  GemvAdaptor op(quant_op, weight_bits, element);
  op.initialize(args);
  op.run(stream);
}

namespace host {
namespace reference {

// host::reference::MixedGemv (host/mixed_gemv.h:23-105) with the GPU behind it: operator() has
// the reference's argument list and meaning -- UN-preprocessed packed weights [M][K], int8 zero
// points, optional bias, host pointers -- and runs preprocess, zero fold, upload, the device GEMV
// and the download.  The reference's template parameters that select the instantiation (int4
// weights with zero points is the only one it defines) are constructor arguments.
class MixedGemv {
 public:
  explicit MixedGemv(WeightOnlyQuantOp quant_op = WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS, int weight_bits = 4)
      : quant_op_(quant_op), weight_bits_(weight_bits) {}

  // A: packed weights as vector_subbyte<int4b_t>::data() holds them (utils/vector_subbyte.h:150-156), or int8.
  void operator()(int32_t batch, int32_t M, int32_t N, int32_t K, int32_t group_size, const uint8_t* A, const half_t* B,
                  const half_t* scale, const int8_t* zero_point, const half_t* bias, half_t* output) const {
    check(mgemv_host_gemv(batch, M, N, K, group_size, A, B, scale, zero_point, bias, output,
                          static_cast<int>(quant_op_), weight_bits_),
          "host::reference::MixedGemv");
  }

 private:
  WeightOnlyQuantOp quant_op_;
  int weight_bits_;
};

}  // namespace reference
}  // namespace host

// mixed_gemv_test.cu:167-181: the HOST_CHECK call site.
inline void host_gemv(const uint8_t* ptr_A, const half_t* ptr_B, const half_t* ptr_scale, const int8_t* ptr_zero_point,
                      const half_t* ptr_C, half_t* ptr_D, int B, int M, int N, int K, int group_size,
                      WeightOnlyQuantOp quant_op = WeightOnlyQuantOp::FINEGRAINED_SCALE_AND_ZEROS, int weight_bits = 4) {
  host::reference::MixedGemv op(quant_op, weight_bits);
  op(B, M, N, K, group_size, ptr_A, ptr_B, ptr_scale, ptr_zero_point, ptr_C, ptr_D);
}

}  // namespace mixed_gemv

#endif  // MIXED_GEMV_AMD_HOST_MIXED_GEMV_HPP_
