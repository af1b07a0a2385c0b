// Counterpart of the reference's only executable (mixed_gemv_test.cu:184-321), written against
// the C++ host mirror.  It does what that main() does -- initialise, pack and read back, fold
// the zero points, preprocess, upload, launch 20 times, download, compare with the CPU
// HOST_CHECK loop -- with two differences the reference lacks: the inputs are seeded, and the
// process exits non-zero when the comparison fails.
//
// The CPU side (input generator and HOST_CHECK loop) comes from the test oracle, which is why
// this program lives under tests/.
//
// usage: mixed_gemv_test [M K group_size quant_op weight_bits bias]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../mixed_gemv_amd/host/mixed_gemv.hpp"

extern "C" {
float orc_f16_to_f32(uint16_t h);
void orc_fill_int8(int8_t* out, size_t n, uint64_t seed, int lo, int hi);
void orc_fill_uniform_f16(uint16_t* out, size_t n, uint64_t seed, float lo, float hi);
int orc_gemv(uint16_t* y, const void* W, const uint16_t* x, const uint16_t* scale, const void* zero, const uint16_t* bias,
             int zero_kind, int n_out, int m_batch, int k, int group_size, int quant_op, int bits, int threads);
int orc_max_threads(void);
}

#define HIP_CHECK(expr)                                                                    \
  do {                                                                                     \
    hipError_t e_ = (expr);                                                                \
    if (e_ != hipSuccess) {                                                                \
      std::printf("Execution error: %s (%s)\n", hipGetErrorString(e_), #expr);             \
      return 2;                                                                            \
    }                                                                                      \
  } while (0)

using namespace mixed_gemv;

int main(int argc, char** argv) {
  const int B = 1, kGemmN = 1;
  int M = argc > 1 ? std::atoi(argv[1]) : 11008, K = argc > 2 ? std::atoi(argv[2]) : 2048;
  int group_size = argc > 3 ? std::atoi(argv[3]) : 128;
  const WeightOnlyQuantOp quant_op = static_cast<WeightOnlyQuantOp>(argc > 4 ? std::atoi(argv[4]) : 3);
  const int bits = argc > 5 ? std::atoi(argv[5]) : 4;
  const bool with_bias = argc > 6 ? std::atoi(argv[6]) != 0 : false;
  if (quant_op == WeightOnlyQuantOp::PER_COLUMN_SCALE_ONLY) group_size = K;
  const int total_group = (K + group_size - 1) / group_size;
  const size_t n_elts = (size_t)M * K;

  // Host A (m, k), uniform over the weight type's range
  std::vector<int8_t> h_A_storage(n_elts);
  orc_fill_int8(h_A_storage.data(), n_elts, 1, bits == 4 ? -8 : -128, bits == 4 ? 7 : 127);
  std::vector<int8_t> h_A(bits == 4 ? n_elts / 2 : n_elts);
  if (bits == 4) {
    SubBytePacker::pack(h_A.data(), h_A_storage.data(), n_elts);
    std::vector<int8_t> readback(n_elts);
    SubBytePacker::unpack(readback.data(), h_A.data(), n_elts / 2);
    size_t diffs = 0;
    for (size_t i = 0; i < n_elts; ++i) diffs += readback[i] != h_A_storage[i];
    if (diffs) {
      std::printf("host pack diff: %zu elements\n", diffs);
      return 3;
    }
  } else {
    h_A = h_A_storage;
  }

  std::vector<half_t> h_B((size_t)B * kGemmN * K), h_scale((size_t)total_group * M), h_bias(M);
  orc_fill_uniform_f16(h_B.data(), h_B.size(), 2, -1.0f, 1.0f);
  orc_fill_uniform_f16(h_scale.data(), h_scale.size(), 3, 0.1f, 0.3f);   // mixed_gemv_test.cu:225
  orc_fill_uniform_f16(h_bias.data(), h_bias.size(), 5, -0.1f, 0.1f);
  std::vector<int8_t> h_zero_point((size_t)total_group * M, 0);
  if (hasZero(quant_op)) orc_fill_int8(h_zero_point.data(), h_zero_point.size(), 4, -8, 7);  // :231

  std::vector<half_t> h_neg_zeros_x_scales((size_t)total_group * M);
  ZeroPointPreprocessor::neg_zero_point_multiplies_scale(h_neg_zeros_x_scales.data(), h_scale.data(), h_zero_point.data(),
                                                         total_group * M);

  const QuantType qt = bits == 4 ? QuantType::W4_A16 : QuantType::W8_A16;
  const std::vector<size_t> shape = {size_t(K), size_t(M)};
  std::vector<int8_t> h_A_processed(MixedGemvWeightPreprocessor::preprocessed_size(shape, qt));
  MixedGemvWeightPreprocessor::run(h_A_processed.data(), h_A.data(), shape, LayoutType::kColumnMajor, qt, false);

  void* d_A;
  half_t *d_B, *d_scale, *d_zero_point, *d_bias, *d_D;
  HIP_CHECK(hipMalloc(&d_A, h_A_processed.size()));
  HIP_CHECK(hipMalloc(&d_B, h_B.size() * 2));
  HIP_CHECK(hipMalloc(&d_scale, h_scale.size() * 2));
  HIP_CHECK(hipMalloc(&d_zero_point, h_scale.size() * 2));
  HIP_CHECK(hipMalloc(&d_bias, h_bias.size() * 2));
  HIP_CHECK(hipMalloc(&d_D, (size_t)B * M * kGemmN * 2));
  HIP_CHECK(hipMemcpy(d_A, h_A_processed.data(), h_A_processed.size(), hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d_B, h_B.data(), h_B.size() * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d_scale, h_scale.data(), h_scale.size() * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d_zero_point, h_neg_zeros_x_scales.data(), h_scale.size() * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(d_bias, h_bias.data(), h_bias.size() * 2, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemset(d_D, 0xff, (size_t)B * M * kGemmN * 2));

  {
    // the launch shape, under the reference's names (gemv/device/gemv_adaptor.h:190-196)
    GemvAdaptor::Arguments shape_args;
    shape_args.problem_size = GemmCoord{M, kGemmN, K};
    shape_args.group_size = group_size;
    shape_args.batch_count = B;
    GemvAdaptor op(quant_op, bits);
    const GemvAdaptor::Dim3 grid = op.get_grid_size(shape_args), block = op.get_block_size(shape_args);
    std::printf("grid (%u, %u, %u) block (%u, %u, %u)\n", grid.x, grid.y, grid.z, block.x, block.y, block.z);
    if (grid.x == 0 || grid.x % 8 != 0 || grid.y != 1 || grid.z != (unsigned)B || block.x % 64 != 0 || block.x == 0 ||
        block.y == 0 || block.x * block.y > 1024 || block.z != 1) {
      std::printf("implausible launch shape\n");
      return 6;
    }
  }

  try {
    for (int i = 0; i < 20; i++)
      device_gemv(d_A, d_B, d_scale, d_zero_point, with_bias ? d_bias : nullptr, d_D, B, M, kGemmN, K, group_size, quant_op, bits);
  } catch (const Error& e) {
    std::printf("%s\n", e.what());
    return 4;
  }
  std::vector<half_t> result_D((size_t)B * M * kGemmN);
  HIP_CHECK(hipMemcpy(result_D.data(), d_D, result_D.size() * 2, hipMemcpyDeviceToHost));
  HIP_CHECK(hipDeviceSynchronize());
  HIP_CHECK(hipGetLastError());

  // The reference's HOST_CHECK call site (mixed_gemv_test.cu:167-181) with the GPU behind it:
  // un-preprocessed weights and int8 zero points in, result out.  Same kernels on the same
  // values, so it must reproduce the device result bit for bit.
  std::vector<half_t> h_D_call_site((size_t)B * M * kGemmN);
  try {
    host_gemv(reinterpret_cast<const uint8_t*>(h_A.data()), h_B.data(), h_scale.data(), h_zero_point.data(),
              with_bias ? h_bias.data() : nullptr, h_D_call_site.data(), B, M, kGemmN, K, group_size, quant_op, bits);
  } catch (const Error& e) {
    std::printf("host_gemv: %s\n", e.what());
    return 4;
  }
  size_t call_site_diffs = 0;
  for (size_t i = 0; i < result_D.size(); ++i) call_site_diffs += h_D_call_site[i] != result_D[i];
  if (call_site_diffs) {
    std::printf("host::reference::MixedGemv differs from device_gemv in %zu outputs\n", call_site_diffs);
    return 5;
  }

  // HOST_CHECK: un-preprocessed weights, int8 zero points (host/mixed_gemv.h:60-105)
  std::vector<half_t> h_D((size_t)B * M * kGemmN);
  orc_gemv(h_D.data(), h_A.data(), h_B.data(), h_scale.data(), h_zero_point.data(), with_bias ? h_bias.data() : nullptr,
           /*int8 zeros*/ 1, M, kGemmN, K, group_size, static_cast<int>(quant_op), bits, orc_max_threads());

  double sq = 0;
  for (int m = 0; m < M; ++m) sq += (double)orc_f16_to_f32(h_D[m]) * orc_f16_to_f32(h_D[m]);
  const double rms = std::sqrt(sq / M), floor = rms / 128.0;
  double max_abs = 0, max_rel = 0;
  for (int m = 0; m < M; ++m) {
    const double cpu = orc_f16_to_f32(h_D[m]), gpu = orc_f16_to_f32(result_D[m]);
    const double abs_err = std::fabs(cpu - gpu);
    const double rel = abs_err / std::fmax(std::fabs(cpu), floor);
    if (rel > 2e-3) std::printf("m: %d cpu: %f\tgpu: %f\tdiff: %f\n", m, cpu, gpu, abs_err);  // mixed_gemv_test.cu:296-300
    max_abs = std::fmax(max_abs, abs_err);
    max_rel = std::fmax(max_rel, rel);
  }
  std::printf("M=%d K=%d group=%d quant_op=%d bits=%d bias=%d: max_abs_err=%.3e max_rel_err=%.3e (floor %.3e) -> %s\n", M, K,
              group_size, static_cast<int>(quant_op), bits, (int)with_bias, max_abs, max_rel, floor,
              max_rel <= 2e-3 ? "PASS" : "FAIL");
  (void)hipFree(d_A); (void)hipFree(d_B); (void)hipFree(d_scale); (void)hipFree(d_zero_point); (void)hipFree(d_bias); (void)hipFree(d_D);
  return max_rel <= 2e-3 ? 0 : 1;
}
