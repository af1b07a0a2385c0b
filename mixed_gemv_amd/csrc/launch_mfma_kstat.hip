// The k-stationary matrix-core GEMV kernel for gfx950 (MI355X), wave64, and its dispatcher.
#include <atomic>
#include <mutex>

#include "kernel_common.h"
#include "mfma_units.h"

namespace mgemv {

// ---------------------------------------------------------------------------------------------
// Matrix-core kernel whose waves stay on one k step.
//
// blockDim = 64 * ksteps (at most 16 waves): wave kw of a workgroup owns k step kw of EVERY tile
// the workgroup walks.  The activation operand of a k step -- x[batch row lane % 16][the lane's 8 k
// of each of the 16 matrix instructions], 64 registers for int4 -- therefore never changes: it is
// loaded once, in front of the walk, and the loop over the tiles holds nothing but the weight
// stream (one unit of 4 KiB per wave and tile, the next tile's unit in flight while one is
// computed), the dequantiser and sixteen matrix instructions.  No LDS stage, no barrier and no
// activation traffic inside the loop; a wave's partial products of a tile (a 16 x 16 fp32 block, of
// which m_batch columns matter) are parked in LDS, and after the walk one barrier separates the
// walks from the combine: wave r sums the ksteps partial blocks of tiles r, r + waves, ... and
// stores them.  Per eight int4 weights a lane issues 13 VALU instructions and one matrix
// instruction, against 17 VALU instructions of the DPP-dot kernel, whatever the number of rows.
// It replaces nothing in the reference, whose kernel is fixed to one activation row
// (gemv/threadblock/default_mma_core_simt.h:68-70); the dequantiser is the one of every kernel here
// (gemv/warp/warp_dequantizer.h:52-59, 86-92), the epilogue host/mixed_gemv.h:102-103.
// Dynamic LDS: waves x 8 activation rows (the stage each wave turns its operand round in, at the start) and
// tiles of the longest walk x 4 x m_batch x 17 x 16 bytes (the partial sums) -- one behind the other where
// both fit, else sharing the space, with a barrier between the two uses.
// ---------------------------------------------------------------------------------------------
constexpr int kParkSlots = kKStationaryParkSlots;  // entries of one block of partial sums: one per possible wave and one to spare

template <int BITS, int QOP, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_unit_kstat(MfmaWeights<BITS, GROUPS_PER_RUN>& f, __amdgpu_buffer_rsrc_t w_rsrc,
                                                const ScaleTables& tables, int weight_offset,
                                                const int (&table_offset)[GROUPS_PER_RUN]) {
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i)
    f.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, weight_offset + i * kBlockBytes, 0, kCacheStream);
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
    f.s[gi] = load_b16_low(tables.scale, table_offset[gi]);  // per-column mode: the row's scale, group 0
    if constexpr (QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS) f.z[gi] = load_b16_low(tables.zero, table_offset[gi]);
  }
}

// PROBE (measurement builds, wrong results): kProbeLoadsOnly keeps every load, the operand's way through LDS, the
// parking, the barrier and the combine, and replaces the arithmetic of a unit by taking its registers;
// kProbeComputeOnly requests only the first tile's unit and repeats its arithmetic for every tile of the walk.
template <int BITS, int QOP, int GROUPS_PER_RUN, int ACT, int PROBE = kProbeNone>
__global__ void __launch_bounds__(kWave * kMaxWavesPerWorkgroup)
gemv_mfma_kstat_kernel(const uint8_t* weights, const half_t* x, const half_t* scale, const half_t* zero_add, int n_out,
                       int k, uint32_t packed_steps, int workgroups, int num_groups, uint32_t packed_group,
                       GemvTail tail) {
  extern __shared__ float partials[];
  using G = Geometry<BITS>;
  Problem p;
  p.weights = weights;
  p.x = x;
  p.scale = scale;
  p.zero_add = zero_add;
  p.n_out = n_out;
  p.k = k;
  p.ksteps = (int)(packed_steps & 0xffffu);
  p.steps_per_wave = 1;
  p.workgroups = workgroups;
  p.wgs_per_xcd = (workgroups + kNumXcd - 1) / kNumXcd;
  p.group_size = (int)(packed_group & 0xffffffu);
  p.tiles_per_wg = 1;
  const long long batch = blockIdx.z;
  long long owner = batch;  // routed launch: whose weights, scales, zeros and bias the problem takes
  if ((blockIdx.z | (packed_group & kRoutedLaunch)) != 0) {
    if ((packed_group & kRoutedLaunch) != 0) {
      const int entry = tail.route[batch];
      if ((unsigned)entry >= (unsigned)tail.route_extent) return;  // whole workgroup, before any barrier
      owner = entry;
    }
    p.weights += owner * tail.stride_weights;
    p.x += batch * tail.stride_x;
    p.scale += owner * tail.stride_scale;
    p.zero_add += owner * tail.stride_scale;
  }
  const bool has_bias = tail.bias != nullptr;
  tail.bias += owner * tail.stride_bias;
  tail.y += batch * tail.stride_y;
  const int m_batch = tail.m_batch;

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;  // whole workgroup leaves before the barrier

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // this wave's k step
  const int waves = p.ksteps;
  const WaveWork work = valu_wave_work(true, wg, 0, 0, 1, tail.seq_base, tail.seq_rem, 0, 1, 1);
  const int tile0 = work.tile_begin;
  const int my_tiles = work.tiles;  // >= 1 by the host's geometry
  const int m = lane % kTileRows;
  const int slice = lane / kTileRows;

  const int tile_stride = p.ksteps * kUnitBytes;  // bytes from a unit to the same k step of the next tile
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(
      p.weights + ((size_t)tile0 * (size_t)p.ksteps + (size_t)kw) * (size_t)kUnitBytes,
      (uint32_t)(my_tiles - 1) * (uint32_t)tile_stride + (uint32_t)kUnitBytes);
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(p.x, (uint32_t)m_batch * (uint32_t)p.k * 2u);
  ScaleTables tables;
  const uint32_t table_bytes = (uint32_t)num_groups * (uint32_t)p.n_out * 2u;
  tables.scale = make_rsrc(p.scale, table_bytes);
  tables.zero = make_rsrc(p.zero_add, QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? table_bytes : 0u);

  // Byte offset of the first row of this lane's scale / zero groups; a tile's entries are its row further on.
  // Rows past n_out (padding of the last tile) read the last row's: never stored.
  int group_offset[GROUPS_PER_RUN];
  {
    const int k_run = kw * G::kStepK + slice * G::kRunK;
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
      const int grp = QOP == MGEMV_PER_COLUMN_SCALE_ONLY ? 0 : group_of(p, k_run + gi * (G::kRunK / GROUPS_PER_RUN));
      group_offset[gi] = grp * p.n_out * 2;
    }
  }
  // A tile past the walk (the loop requests one or two) is sent past the tables: such a load comes back at
  // once, where a real one would have to land before the combine may reuse its register.
  auto offsets_of_tile = [&](int i, int (&off)[GROUPS_PER_RUN]) {
    const int row = (tile0 + i) * kTileRows + m;
    const uint32_t row_bytes = (uint32_t)(row < p.n_out ? row : p.n_out - 1) * 2u + (i < my_tiles ? 0u : 0x40000000u);
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) off[gi] = (int)((uint32_t)group_offset[gi] + row_bytes);
  };

  MfmaActivations<BITS> xa;
  MfmaWeights<BITS, GROUPS_PER_RUN> wa, wb;
  auto request_first_unit = [&]() {
    int off[GROUPS_PER_RUN];
    offsets_of_tile(0, off);
    load_unit_kstat<BITS, QOP, GROUPS_PER_RUN>(wa, w_rsrc, tables, lane * kChunkBytes, off);
  };
  // The activation operand: rows of this wave's k step come in whole (one fully coalesced load per row), pass
  // through a stage of 8 rows that belongs to this wave alone, and are read back in operand shape -- lane
  // (slice, m) takes the sixteen 16-byte pieces of row m that its matrix instructions pair with its weights.
  // (Read straight from x in operand shape, every load instruction touches 64 cache lines for 16 bytes each.)
  // More than 8 rows: a second round for the lanes of rows 8-15.  Lanes of rows that do not exist keep zeros.
  {
    using XS = XStage<BITS>;
    uint8_t* const stage = reinterpret_cast<uint8_t*>(partials) + kw * (8 * XS::kRowStride);
    const uint8_t* const mine = stage + (m & 7) * XS::kRowStride + slice * (G::kRunK * 2);
#pragma unroll
    for (int i = 0; i < kBlocksPerUnit; ++i)
#pragma unroll
      for (int j = 0; j < (BITS == 4 ? 4 : 2); ++j) xa.x[i][j] = u32x4{0u, 0u, 0u, 0u};
    for (int first = 0; first < m_batch; first += 8) {
      const int rows_here = m_batch - first < 8 ? m_batch - first : 8;
      XRows<BITS, 8> rows;
      fetch_x_rows<BITS, 8>(rows, p, x_rsrc, kw, lane, first, 1, rows_here);
      // The first unit of weights is requested behind the first rows of x (an L2 hit, back long before it):
      // the operand is turned round while the weights are still on their way.
      if (first == 0) request_first_unit();
      __builtin_amdgcn_sched_barrier(0);
      park_x_rows<BITS, 8>(rows, stage, lane, 0, 1, rows_here);
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");  // the LDS executes a wave's accesses in order
      __builtin_amdgcn_wave_barrier();
      if (m >= first && m < first + rows_here) {
#pragma unroll
        for (int i = 0; i < kBlocksPerUnit; ++i)
#pragma unroll
          for (int j = 0; j < (BITS == 4 ? 4 : 2); ++j)
            xa.x[i][j] = *reinterpret_cast<const u32x4*>(mine + (i * G::kChunkK + j * 8) * 2);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
  const bool park_behind_stage = (tail.flags & kParkBehindStage) != 0;
  if (!park_behind_stage) __syncthreads();  // the stages make room for the partial sums
  const bool short_allowed = (tail.flags & kExactIntegerFormOnly) == 0;
  const ConvertRegs c = make_convert_regs();

  // Partial sums in LDS: for every (tile of the walk, row group, batch row) a block of kParkSlots entries of
  // four floats, entry w written by wave w (the odd block length spreads the lanes over the banks).  The lane
  // that later sums a block finds its entries side by side, at offsets known to the compiler.
  f32x4* const park = reinterpret_cast<f32x4*>(reinterpret_cast<uint8_t*>(partials) +
                                               (park_behind_stage ? waves * (8 * XStage<BITS>::kRowStride) : 0));
  const int park_tile_stride = kKSlices * m_batch * kParkSlots;  // entries from a tile to the next
  f32x4* const my_park = park + (slice * m_batch + m) * kParkSlots + kw;
  auto compute_and_park = [&](const MfmaWeights<BITS, GROUPS_PER_RUN>& f, int i) {
    f32x4 acc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    half2_t col_scale = half2_t{};
    bool short_ok = short_allowed;
    if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
      col_scale = splat_low(f.s[0]);
      const uint32_t bits[1] = {f.s[0]};
      short_ok = short_ok && wave_scales_permit_short_form<ACT>(bits);
    }
    if constexpr (PROBE == kProbeLoadsOnly) {
      uint32_t t = xa.x[0][0][0];
#pragma unroll
      for (int b = 0; b < kBlocksPerUnit; ++b) t ^= f.w[b][0] ^ f.w[b][1] ^ f.w[b][2] ^ f.w[b][3];
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) t ^= f.s[gi] ^ f.z[gi];
      acc[0] += __builtin_bit_cast(float, t & 0x3fffffffu);
    } else {
      compute_unit_mfma<BITS, QOP, GROUPS_PER_RUN, ACT>(acc, f, xa, c, col_scale, short_ok);
    }
    if (m < m_batch) my_park[i * park_tile_stride] = acc;
  };
  // arithmetic-only build: the next unit is the first one again; the compiler must assume its registers changed
  auto repeat_first_unit = [&](MfmaWeights<BITS, GROUPS_PER_RUN>& to, const MfmaWeights<BITS, GROUPS_PER_RUN>& from) {
    to = from;
#pragma unroll
    for (int b = 0; b < kBlocksPerUnit; ++b) asm volatile("" : "+v"(to.w[b]));
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) asm volatile("" : "+v"(to.s[gi]), "+v"(to.z[gi]));
  };

  int i = 0;
  do {
    if constexpr (PROBE == kProbeComputeOnly) {
      repeat_first_unit(wb, wa);
    } else {
      int off[GROUPS_PER_RUN];
      offsets_of_tile(i + 1, off);
      load_unit_kstat<BITS, QOP, GROUPS_PER_RUN>(wb, w_rsrc, tables, (i + 1) * tile_stride + lane * kChunkBytes, off);
    }
    __builtin_amdgcn_sched_barrier(0);
    compute_and_park(wa, i);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PROBE == kProbeComputeOnly) {
      repeat_first_unit(wa, wb);
    } else {
      int off[GROUPS_PER_RUN];
      offsets_of_tile(i + 2, off);
      load_unit_kstat<BITS, QOP, GROUPS_PER_RUN>(wa, w_rsrc, tables, (i + 2) * tile_stride + lane * kChunkBytes, off);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (i + 1 < my_tiles) compute_and_park(wb, i + 1);
    __builtin_amdgcn_sched_barrier(0);
    i += 2;
  } while (i < my_tiles);

  // The combine.  Wave r sums tiles r, r + waves, ... of the walk; lane (slice, m) the four rows
  // 4 * slice .. + 3 of batch row m.  A wave that reaches the barrier waits for the slowest one, and behind
  // the barrier it is alone on its SIMD, where every instruction costs its full latency: whatever does not
  // need the other waves' sums -- addresses, the bias, zeros in the entries of waves that do not exist --
  // is done in front of it.
  const bool sums = m < m_batch && kw < my_tiles;
  f32x4* block = park + (kw * kKSlices + slice) * (m_batch * kParkSlots) + m * kParkSlots;
  int n0 = (tile0 + kw) * kTileRows + 4 * slice;
  float bias[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  auto fetch_bias = [&]() {
    if (has_bias) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int n = n0 + v < p.n_out ? n0 + v : p.n_out - 1;
        if constexpr (ACT == kActBf16)
          bias[v] = bf16_low_to_f32(reinterpret_cast<const uint16_t*>(tail.bias)[n]);
        else
          bias[v] = (float)tail.bias[n];
      }
    }
  };
  if (sums) {
    fetch_bias();
    if (waves < kMaxWavesPerWorkgroup)
      for (int t = kw; t < my_tiles; t += waves)
        for (int w = waves; w < kMaxWavesPerWorkgroup; ++w)
          block[(t - kw) * park_tile_stride + w] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  uint16_t* dst = reinterpret_cast<uint16_t*>(tail.y) + (size_t)m * (size_t)p.n_out + n0;
  const size_t dst_step = (size_t)waves * kTileRows;  // outputs from a tile this wave sums to the next
  const bool wide_store = ((reinterpret_cast<uintptr_t>(tail.y) | (uintptr_t)((size_t)p.n_out * 2)) & 7u) == 0;

  __syncthreads();
  if (sums) {
    for (int t = kw; t < my_tiles; t += waves) {
      f32x4 piece[kMaxWavesPerWorkgroup];
#pragma unroll
      for (int w = 0; w < kMaxWavesPerWorkgroup; ++w) piece[w] = block[w];
      f32x4 sum = piece[0];
#pragma unroll
      for (int w = 1; w < kMaxWavesPerWorkgroup; ++w) sum += piece[w];  // ascending k
      // n_out is a multiple of 4 and so is n0: the four outputs of a lane are all inside or all outside, and
      // they are neighbours in y -- one 8-byte store where y allows it
      if (n0 < p.n_out) {
        float r[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) r[v] = epilogue_value(tail, sum[v], has_bias, bias[v]);
        uint32_t lo, hi;
        if constexpr (ACT == kActBf16) {
          lo = pack_bf16(r[0], r[1]);
          hi = pack_bf16(r[2], r[3]);
        } else {
          lo = as_u32(half2_t{(half_t)r[0], (half_t)r[1]});
          hi = as_u32(half2_t{(half_t)r[2], (half_t)r[3]});
        }
        if (wide_store) {
          *reinterpret_cast<u32x2*>(dst) = u32x2{lo, hi};
        } else {
          dst[0] = (uint16_t)lo; dst[1] = (uint16_t)(lo >> 16); dst[2] = (uint16_t)hi; dst[3] = (uint16_t)(hi >> 16);
        }
      }
      // walks longer than the workgroup has waves: on to this wave's next tile
      block += waves * park_tile_stride;
      n0 += waves * kTileRows;
      dst += dst_step;
      if (t + waves < my_tiles) fetch_bias();
    }
  }
}

template <int BITS, int QOP, int GPR, int ACT, int PROBE = kProbeNone>
hipError_t launch_mfma_kstat_kernel(const GemvLaunch& g) {
  const auto kernel = gemv_mfma_kstat_kernel<BITS, QOP, GPR, ACT, PROBE>;
  if (g.lds > 48 * 1024) {
    // More than 48 KiB of dynamic LDS has to be granted per kernel and device; remember the
    // largest grant so that only the first such launch pays for the call.
    constexpr int kMaxDevices = 64;
    static std::atomic<int> granted[kMaxDevices];
    static std::mutex grant_mutex;
    const int device = g.device;
    const bool tracked = device >= 0 && device < kMaxDevices;
    if (!tracked || granted[device].load() < (int)g.lds) {
      std::lock_guard<std::mutex> lock(grant_mutex);
      if (!tracked || granted[device].load() < (int)g.lds) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds);
        if (e != hipSuccess) return e;
        if (tracked) granted[device].store((int)g.lds);
      }
    }
  }
  return launch(kernel, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale, g.zero_add, g.n_out, g.k,
                pack_steps(num_ksteps(g.k, BITS), 1), g.plan.workgroups, g.tail.num_groups, pack_group(g.group_size, 1, g.tail.route != nullptr),
                g.tail);
}

template <int BITS, int QOP, int ACT>
hipError_t launch_mfma_kstat_gpr(const GemvLaunch& g, int gpr) {
  if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
    return launch_mfma_kstat_kernel<BITS, QOP, 1, ACT>(g);
  } else {
    switch (gpr) {
      case 1: return launch_mfma_kstat_kernel<BITS, QOP, 1, ACT>(g);
      case 2: return launch_mfma_kstat_kernel<BITS, QOP, 2, ACT>(g);
      default: return launch_mfma_kstat_kernel<BITS, QOP, 4, ACT>(g);
    }
  }
}

template <int ACT>
hipError_t launch_mfma_kstat_act(const GemvLaunch& g, int bits, int qop, int gpr) {
  if (bits == 4) {
    switch (qop) {
      case 1: return launch_mfma_kstat_gpr<4, 1, ACT>(g, gpr);
      case 2: return launch_mfma_kstat_gpr<4, 2, ACT>(g, gpr);
      default: return launch_mfma_kstat_gpr<4, 3, ACT>(g, gpr);
    }
  }
  switch (qop) {
    case 1: return launch_mfma_kstat_gpr<8, 1, ACT>(g, gpr);
    case 2: return launch_mfma_kstat_gpr<8, 2, ACT>(g, gpr);
    default: return launch_mfma_kstat_gpr<8, 3, ACT>(g, gpr);
  }
}

// Measurement builds exist for int4 scale-and-zero fp16 launches with one or two groups per lane run.
bool mfma_kstat_probe_exists(int bits, int qop, int gpr, int act) {
  return bits == 4 && qop == MGEMV_FINEGRAINED_SCALE_AND_ZEROS && (gpr == 1 || gpr == 2) && act == kActF16;
}

hipError_t launch_mfma_kstat_probe(const GemvLaunch& g, int gpr, int probe) {
  constexpr int kQ = MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  if (probe == kProbeLoadsOnly)
    return gpr == 1 ? launch_mfma_kstat_kernel<4, kQ, 1, kActF16, kProbeLoadsOnly>(g)
                    : launch_mfma_kstat_kernel<4, kQ, 2, kActF16, kProbeLoadsOnly>(g);
  return gpr == 1 ? launch_mfma_kstat_kernel<4, kQ, 1, kActF16, kProbeComputeOnly>(g)
                  : launch_mfma_kstat_kernel<4, kQ, 2, kActF16, kProbeComputeOnly>(g);
}

hipError_t launch_mfma_kstat(const GemvLaunch& g, int bits, int qop, int gpr, int act) {
  // fp16 only: with the bf16 dequantiser the kernel does not fit the 128 registers of a 16-wave workgroup, and with
  // spills it is behind the other kernels; the planner never asks for it
  if (act != kActF16) return hipErrorInvalidValue;
  return launch_mfma_kstat_act<kActF16>(g, bits, qop, gpr);
}

}  // namespace mgemv
