// Measurement probes: the kernels behind the "ceilings" that the benchmark reports beside the
// GEMV figures -- what an empty launch costs, what a plain streaming read of the same bytes with
// the same launch shape achieves, what the GEMV's own loads take with the arithmetic removed and
// its arithmetic with the loads removed, and when the phases of one launch happen.  None of this is on a product path and nothing here
// has a counterpart in the reference.
#include "gemv_dpp_kernel.h"

namespace mgemv {

__global__ void __launch_bounds__(64) empty_kernel() {}
__global__ void __launch_bounds__(kWave * kMaxWavesPerWorkgroup) empty_grid_kernel() {}

// Every wave streams its own contiguous range of 4-KiB units with the loads of the GEMV kernel
// (one 1-KiB block per wave-wide 128-bit load, streaming cache hint), DEPTH units requested
// before the first is consumed and each requested again as soon as it has been folded into an
// exclusive-or -- a GEMV without scales, activations and arithmetic.
template <int DEPTH>
__global__ void __launch_bounds__(kWave * kMaxWavesPerWorkgroup)
stream_read_kernel(const uint8_t* src, int units_per_wave, uint32_t* sink) {
  const int lane = threadIdx.x % kWave;
  const size_t wave = (size_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  const __amdgpu_buffer_rsrc_t rsrc =
      make_rsrc(src + wave * (size_t)units_per_wave * kUnitBytes, (uint32_t)units_per_wave * (uint32_t)kUnitBytes);
  u32x4 buf[DEPTH][kBlocksPerUnit];
  u32x4 acc = {0, 0, 0, 0};
  int offset = lane * kChunkBytes;
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
    for (int b = 0; b < kBlocksPerUnit; ++b)
      buf[d][b] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, offset + b * kBlockBytes, 0, kCacheStream);
    offset += kUnitBytes;
    __builtin_amdgcn_sched_barrier(0);
  }
  for (int u = 0; u < units_per_wave; u += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
      for (int b = 0; b < kBlocksPerUnit; ++b) acc ^= buf[d][b];
      __builtin_amdgcn_sched_barrier(0);
      // past the wave's range the offsets are out of the descriptor's range: zero, no memory access
#pragma unroll
      for (int b = 0; b < kBlocksPerUnit; ++b)
        buf[d][b] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, offset + b * kBlockBytes, 0, kCacheStream);
      offset += kUnitBytes;
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u && sink != nullptr) sink[0] = 1;  // keeps the loads alive
}

template <int PROBE>
hipError_t launch_gemv_probe_kind(const GemvLaunch& g) {
  const auto args = [&](auto kernel) {
    return launch(kernel, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale, g.zero_add, g.n_out, g.k,
                  pack_steps(num_ksteps(g.k, 4), g.plan.steps_per_wave), g.plan.workgroups, g.tail.num_groups,
                  pack_group(g.group_size, g.plan.tiles_per_wg, g.tail.route != nullptr), g.tail);
  };
  return g.plan.tiles_in_sequence > 1
             ? args(gemv_dpp_kernel<4, MGEMV_FINEGRAINED_SCALE_AND_ZEROS, 1, 1, true, kActF16, PROBE>)
             : args(gemv_dpp_kernel<4, MGEMV_FINEGRAINED_SCALE_AND_ZEROS, 1, 1, false, kActF16, PROBE>);
}

hipError_t launch_gemv_probe(const GemvLaunch& g, int probe) {
  switch (probe) {
    case kProbeLoadsOnly: return launch_gemv_probe_kind<kProbeLoadsOnly>(g);
    case kProbeComputeOnly: return launch_gemv_probe_kind<kProbeComputeOnly>(g);
    default: return launch_gemv_probe_kind<kProbeTimeline>(g);
  }
}

}  // namespace mgemv

extern "C" {

int mgemv_probe_empty_launch(void* stream) {
  return mgemv::launch(mgemv::empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream)) == hipSuccess
             ? MGEMV_OK
             : MGEMV_ERR_LAUNCH;
}

int mgemv_probe_empty_grid(int workgroups, int waves_per_workgroup, void* stream) {
  if (workgroups < 1 || workgroups > (1 << 20) || waves_per_workgroup < 1 || waves_per_workgroup > mgemv::kMaxWavesPerWorkgroup)
    return MGEMV_ERR_SIZE;
  return mgemv::launch(mgemv::empty_grid_kernel, dim3((unsigned)workgroups), dim3((unsigned)(mgemv::kWave * waves_per_workgroup)),
                       0, static_cast<hipStream_t>(stream)) == hipSuccess
             ? MGEMV_OK
             : MGEMV_ERR_LAUNCH;
}

int mgemv_probe_stream_read(const void* src, size_t bytes, int workgroups, int waves_per_workgroup, int units_in_flight,
                            uint32_t* sink, void* stream) {
  if (src == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (workgroups < 1 || waves_per_workgroup < 1 || waves_per_workgroup > mgemv::kMaxWavesPerWorkgroup) return MGEMV_ERR_SIZE;
  if (reinterpret_cast<uintptr_t>(src) % 16) return MGEMV_ERR_ALIGNMENT;
  const size_t waves = (size_t)workgroups * (size_t)waves_per_workgroup;
  const size_t units_per_wave = bytes / mgemv::kUnitBytes / waves;
  if (units_per_wave < 1 || units_per_wave * mgemv::kUnitBytes >= (1ull << 31)) return MGEMV_ERR_SIZE;
  const dim3 grid((unsigned)workgroups), block((unsigned)(mgemv::kWave * waves_per_workgroup));
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* p = static_cast<const uint8_t*>(src);
  hipError_t e;
  switch (units_in_flight) {
    case 2: e = mgemv::launch(mgemv::stream_read_kernel<2>, grid, block, 0, st, p, (int)units_per_wave, sink); break;
    case 4: e = mgemv::launch(mgemv::stream_read_kernel<4>, grid, block, 0, st, p, (int)units_per_wave, sink); break;
    case 8: e = mgemv::launch(mgemv::stream_read_kernel<8>, grid, block, 0, st, p, (int)units_per_wave, sink); break;
    default: return MGEMV_ERR_SIZE;
  }
  return e == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
}

}  // extern "C"
