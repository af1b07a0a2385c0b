// The matrix-core GEMV kernels for gfx950 (MI355X), wave64 (small batches of activation rows),
// and the dispatchers that pick their instantiations.
#include <atomic>
#include <mutex>

#include "kernel_common.h"
#include "mfma_units.h"

namespace mgemv {

// ---------------------------------------------------------------------------------------------
// Small-batch variant on the matrix cores (5 <= m_batch <= 16, padded to 16 columns).
//
// The tile layout already has the operand shape of v_mfma_f32_16x16x32_f16: lane l holds
// row l % 16 of the tile and k slice l / 16, and one 32-bit weight word dequantises to the 8
// consecutive-k fp16 values (4 VGPRs) that lane contributes to the 16 x 32 weight operand.
// The activation operand is read straight from x: lane l supplies x[l % 16][same 8 k].  The
// instruction pairs operand elements of equal (k slice, element) position, so the result is
// D[row][batch row] = sum_k dq[row][k] * x[batch row][k], accumulated in fp32 across the
// wave's whole k range: the VALU only converts and dequantises (no dot instructions), which
// is what makes this path faster than repeating the VALU kernel once activation rows multiply.
// It replaces nothing in the reference, whose kernel is fixed to one activation row
// (gemv/threadblock/default_mma_core_simt.h:68-70).
// ---------------------------------------------------------------------------------------------


// blockDim = (64 * split_k, tiles_per_wg); each wave works on T consecutive tiles so that the
// activation operands of a k step are fetched once and used T times.  Dynamic LDS:
// tiles_per_wg * split_k * T * 256 floats (none when split_k == 1).
template <int BITS, int QOP, int GROUPS_PER_RUN, int T>
__global__ void __launch_bounds__(kWave * kMaxWavesPerMfmaWorkgroup)
gemv_mfma_kernel(const uint8_t* weights, const half_t* x, const half_t* scale, const half_t* zero_add, int n_out, int k,
                 uint32_t packed_steps, int workgroups, int wgs_per_xcd, uint32_t packed_group, GemvTail tail) {
  extern __shared__ float partials[];
  Problem p;
  p.weights = weights;
  p.x = x;
  p.scale = scale;
  p.zero_add = zero_add;
  p.n_out = n_out;
  p.k = k;
  p.ksteps = (int)(packed_steps & 0xffffu);
  p.steps_per_wave = (int)(packed_steps >> 16);
  p.workgroups = workgroups;
  p.wgs_per_xcd = wgs_per_xcd;
  p.group_size = (int)(packed_group & 0xffffffu);
  p.tiles_per_wg = tiles_per_wg_of(packed_group);
  asm volatile("" ::"s"(weights), "s"(x), "s"(scale), "s"(zero_add), "s"(n_out), "s"(k), "s"(packed_steps),
               "s"(workgroups), "s"(wgs_per_xcd), "s"(packed_group), "s"(tail.bias), "s"(tail.y), "s"(tail.split_k),
               "s"(tail.m_batch), "s"(tail.num_groups), "s"(tail.flags), "s"(tail.stride_weights), "s"(tail.stride_x), "s"(tail.stride_scale),
               "s"(tail.stride_bias), "s"(tail.stride_y));
  const long long batch = blockIdx.z;
  long long owner = batch;  // routed launch: whose weights, scales, zeros and bias the problem takes
  if (packed_group & kRoutedLaunch) {
    const int entry = tail.route[batch];
    if ((unsigned)entry >= (unsigned)tail.route_extent) return;  // whole workgroup, before any barrier
    owner = entry;
  }
  p.weights += owner * tail.stride_weights;
  p.x += batch * tail.stride_x;
  p.scale += owner * tail.stride_scale;
  p.zero_add += owner * tail.stride_scale;
  const bool has_bias = tail.bias != nullptr;
  tail.bias += owner * tail.stride_bias;
  tail.y += batch * tail.stride_y;
  const int m_batch = tail.m_batch;

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  const WaveWork work = mfma_wave_work(T, wg, ty, kw, p.tiles_per_wg, tiles, p.steps_per_wave, p.ksteps);
  const int tile0 = work.tile_begin;
  int row[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int r = (tile0 + t) * kTileRows + lane % kTileRows;
    row[t] = r < p.n_out ? r : p.n_out - 1;
  }

  f32x4 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int ks_begin = work.ks_begin;
  if (work.tiles > 0 && work.units > 0) {
    const int units = work.units;
    const int my_tiles = work.tiles;
    const int tile_stride = p.ksteps * kUnitBytes;  // bytes from a unit to the same k step of the next tile
    // One descriptor spans the wave's tiles.
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(
        p.weights + ((size_t)tile0 * (size_t)p.ksteps + (size_t)ks_begin) * (size_t)kUnitBytes,
        (uint32_t)(my_tiles - 1) * (uint32_t)tile_stride + (uint32_t)units * (uint32_t)kUnitBytes);
    const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(p.x, (uint32_t)m_batch * (uint32_t)p.k * 2u);
    half2_t col_scale[T];
    bool short_ok[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      col_scale[t] = half2_t{};
      short_ok[t] = (tail.flags & kExactIntegerFormOnly) == 0;
      if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
        col_scale[t] = splat(p.scale[row[t]]);
        const uint32_t bits[1] = {as_u32(col_scale[t])};
        short_ok[t] = short_ok[t] && wave_scales_permit_short_form<kActF16>(bits);
      }
    }
    const ConvertRegs c = make_convert_regs();
    for (int u = 0; u < units; ++u) {
      MfmaActivations<BITS> xa;
      MfmaWeights<BITS, GROUPS_PER_RUN> wt[T];
#pragma unroll
      for (int t = 0; t < T; ++t)
        load_weights_mfma<BITS, QOP, GROUPS_PER_RUN>(wt[t], p, w_rsrc, min(t, my_tiles - 1) * tile_stride + u * kUnitBytes,
                                                     ks_begin + u, lane, row[t]);  // tiles past the matrix re-read the last one; never stored
      load_activations_mfma<BITS>(xa, p, x_rsrc, ks_begin + u, lane);
#pragma unroll
      for (int t = 0; t < T; ++t) compute_unit_mfma<BITS, QOP, GROUPS_PER_RUN>(acc[t], wt[t], xa, c, col_scale[t], short_ok[t]);
    }
  }

  // Lane l holds D[rows 4*(l/16) .. +3 of the tile][batch row l % 16] for each of its tiles.
  const int split_k = tail.split_k;
  if (split_k > 1) {
    f32x4* park = reinterpret_cast<f32x4*>(partials) + ((ty * split_k + kw) * T) * kWave + lane;
#pragma unroll
    for (int t = 0; t < T; ++t) park[t * kWave] = acc[t];
    __syncthreads();
    if (tile0 >= tiles) return;
    // wave kw finishes tiles t = kw, kw + split_k, ...
    for (int t = kw; t < T; t += split_k) {
      const f32x4* part = reinterpret_cast<const f32x4*>(partials) + (ty * split_k * T + t) * kWave + lane;
      f32x4 sum = part[0];
      for (int w = 1; w < split_k; ++w) sum += part[w * T * kWave];
      const int m = lane % kTileRows;
      const int n0 = (tile0 + t) * kTileRows + 4 * (lane / kTileRows);
      if (m < m_batch) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int n = n0 + v;
          if (n < p.n_out) {
            const float r = epilogue_value(tail, sum[v], has_bias, has_bias ? (float)tail.bias[n] : 0.0f);
            tail.y[(size_t)m * (size_t)p.n_out + n] = (half_t)r;
          }
        }
      }
    }
    return;
  }
  if (tile0 >= tiles) return;
  const int m = lane % kTileRows;
  if (m < m_batch) {
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int n0 = (tile0 + t) * kTileRows + 4 * (lane / kTileRows);
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int n = n0 + v;
        if (n < p.n_out) {
          const float r = epilogue_value(tail, acc[t][v], has_bias, has_bias ? (float)tail.bias[n] : 0.0f);
          tail.y[(size_t)m * (size_t)p.n_out + n] = (half_t)r;
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Small-batch variant on the matrix cores with the activation operand staged through LDS.
//
// The kernel above reads its activation operand -- 16 rows x 512 k = 16 KiB per k step -- from
// L2 into registers, sixteen 128-bit loads per lane and step; that leaves no registers for
// prefetching, so it hides latency by occupancy alone.  Here the tiles_per_wg waves of a
// workgroup that work on the SAME k range (different tiles) fetch that slice once, together,
// into a double-buffered LDS stage: round r of wave ty brings one whole row (64 lanes x 16
// bytes) of batch row ty + r * tiles_per_wg.  The matrix instructions read their operand from
// LDS just in time (rows 1040 bytes apart, so the 16 lanes of a k slice hit 16 distinct bank
// groups), the registers hold two k steps of weights, and the global loads of step u+1 -- weights
// and activation rows -- are in flight while step u is computed.  One barrier per k step.
// ROUNDS = staged rows / tiles_per_wg; staged rows (8 or 16) >= m_batch.  Lanes of batch rows
// that are not staged read some other row: columns of a matrix product do not mix, and those
// columns are never stored.
// ---------------------------------------------------------------------------------------------
// Measurement builds.  keep_registers: the compiler must assume that a unit's registers changed (so
// that repeating its arithmetic is not hoisted out of the loop); no instruction.  consume_unit: every
// register of the unit and one staged operand have to be there, nothing is computed with them.
template <int BITS, int GROUPS_PER_RUN, int ROUNDS>
__device__ __forceinline__ void keep_registers(MfmaWeights<BITS, GROUPS_PER_RUN>& f, XRows<BITS, ROUNDS>& r) {
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) asm volatile("" : "+v"(f.w[i]));
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) asm volatile("" : "+v"(f.s[gi]), "+v"(f.z[gi]));
#pragma unroll
  for (int j = 0; j < ROUNDS; ++j)
#pragma unroll
    for (int h = 0; h < (BITS == 4 ? 4 : 2); ++h) asm volatile("" : "+v"(r.v[j][h]));
}

template <int BITS, int GROUPS_PER_RUN>
__device__ __forceinline__ void consume_unit(f32x4& acc, const MfmaWeights<BITS, GROUPS_PER_RUN>& f,
                                             const LdsActivations<BITS>& xa) {
  uint32_t t = 0;
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) t ^= f.w[i][0] ^ f.w[i][1] ^ f.w[i][2] ^ f.w[i][3];
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) t ^= f.s[gi] ^ f.z[gi];
  t ^= *reinterpret_cast<const uint32_t*>(xa.lane_base);
  acc[0] += __builtin_bit_cast(float, t & 0x3fffffffu);
}

// blockDim = (64 * split_k, tiles_per_wg), at most 8 waves.  Dynamic LDS: split_k * 2 stages of
// (ROUNDS * tiles_per_wg) rows x kRowStride bytes, then tiles_per_wg * split_k * 256 floats for
// the split-K combine.
// PROBE: kProbeNone the product; kProbeLoadsOnly keeps every load, the staging and the barriers and
// replaces the arithmetic of a unit by taking its registers and one staged operand; kProbeComputeOnly
// requests only the first k step of a wave's range and repeats the staging and the arithmetic of
// that step for every further one (measurement builds, wrong results).
template <int BITS, int QOP, int GROUPS_PER_RUN, int ROUNDS, int ACT, bool SHARED, int PROBE = kProbeNone>
__global__ void __launch_bounds__(kWave * kMaxWavesPerMfmaWorkgroup)
gemv_mfma_lds_kernel(const uint8_t* weights, const half_t* x, const half_t* scale, const half_t* zero_add, int n_out,
                     int k, uint32_t packed_steps, int workgroups, int num_groups, uint32_t packed_group, GemvTail tail) {
  extern __shared__ float partials[];
  using XS = XStage<BITS>;
  Problem p;
  p.weights = weights;
  p.x = x;
  p.scale = scale;
  p.zero_add = zero_add;
  p.n_out = n_out;
  p.k = k;
  p.ksteps = (int)(packed_steps & 0xffffu);
  p.steps_per_wave = (int)(packed_steps >> 16);
  p.workgroups = workgroups;
  p.wgs_per_xcd = (workgroups + kNumXcd - 1) / kNumXcd;
  p.group_size = (int)(packed_group & 0xffffffu);
  p.tiles_per_wg = tiles_per_wg_of(packed_group);
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
  if (wg >= p.workgroups) return;  // whole workgroup leaves before any barrier

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int split_k = tail.split_k;
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  const WaveWork work = staged_wave_work(wg, ty, kw, p.tiles_per_wg, tiles, p.steps_per_wave, p.ksteps);
  const int tile_raw = work.tile_begin;
  const int tile = work.tiles > 0 ? tile_raw : tiles - 1;  // a wave without a tile still stages rows and meets the barriers
  const int row_raw = tile * kTileRows + lane % kTileRows;
  const int row = row_raw < p.n_out ? row_raw : p.n_out - 1;

  const int staged_rows = ROUNDS * p.tiles_per_wg;
  const int stage_bytes = staged_rows * XS::kRowStride;
  uint8_t* const lds = reinterpret_cast<uint8_t*>(partials);
  uint8_t* const my_stages = lds + kw * 2 * stage_bytes;  // the two stages of this k range
  // this lane's operand row: batch row lane % 16 if staged, else any staged row (never stored)
  const int m_read = (lane % kTileRows) & (staged_rows - 1);
  const int operand_offset = m_read * XS::kRowStride + (lane / kTileRows) * Geometry<BITS>::kRunK * 2;

  const int steps = p.steps_per_wave;  // the same for every wave: the barriers are workgroup-wide
  const int ks_begin = work.ks_begin;
  const int units = work.units;  // >= 1 by the host's geometry
  const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(
      p.weights + ((size_t)tile * (size_t)p.ksteps + (size_t)ks_begin) * (size_t)kUnitBytes,
      (uint32_t)units * (uint32_t)kUnitBytes);
  const __amdgpu_buffer_rsrc_t x_rsrc = make_rsrc(p.x, (uint32_t)m_batch * (uint32_t)p.k * 2u);
  ScaleTables tables;
  const uint32_t table_bytes = (uint32_t)num_groups * (uint32_t)p.n_out * 2u;
  tables.scale = make_rsrc(p.scale, table_bytes);
  tables.zero = make_rsrc(p.zero_add, QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? table_bytes : 0u);

  half2_t col_scale = half2_t{};
  bool short_ok = (tail.flags & kExactIntegerFormOnly) == 0;
  if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
    col_scale = splat(p.scale[row]);
    const uint32_t bits[1] = {as_u32(col_scale)};
    short_ok = short_ok && wave_scales_permit_short_form<ACT>(bits);
  }
  const ConvertRegs c = make_convert_regs();

  f32x4 acc = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  XRows<BITS, ROUNDS> xr;
  MfmaWeights<BITS, GROUPS_PER_RUN> wa, wb;
  fetch_x_rows<BITS, ROUNDS>(xr, p, x_rsrc, ks_begin, lane, ty, p.tiles_per_wg);
  load_weights_lds_mfma<BITS, QOP, GROUPS_PER_RUN>(wa, p, w_rsrc, tables, 0, ks_begin, lane, row);
  // A stage is shared by the tiles_per_wg waves that cover the same k range of neighbouring tiles
  // (SHARED).  With one tile per workgroup every wave has its stages to itself: the LDS executes
  // a wave's accesses in order, so nothing but the compiler has to be kept from reordering them,
  // and the waves of the workgroup run free of each other until the split-K combine (4096x14336,
  // 8 rows: 10.4 us against 11.6 with the barriers; 3584x18944: 12.8 against 15.1).
  auto stage_ready = [&]() {
    if constexpr (SHARED) {
      __syncthreads();
    } else {
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  };
  int u = 0;
  do {
    // even step: weights in wa, stage 0
    park_x_rows<BITS, ROUNDS>(xr, my_stages, lane, ty, p.tiles_per_wg);
    stage_ready();
    if constexpr (PROBE == kProbeComputeOnly) {
      wb = wa;
      keep_registers(wb, xr);
    } else {
      fetch_x_rows<BITS, ROUNDS>(xr, p, x_rsrc, ks_begin + u + 1, lane, ty, p.tiles_per_wg);
      load_weights_lds_mfma<BITS, QOP, GROUPS_PER_RUN>(wb, p, w_rsrc, tables, u + 1, ks_begin + u + 1, lane, row);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (u < units) {
      const LdsActivations<BITS> xa{my_stages + operand_offset};
      if constexpr (PROBE == kProbeLoadsOnly)
        consume_unit(acc, wa, xa);
      else
        compute_unit_mfma<BITS, QOP, GROUPS_PER_RUN, ACT>(acc, wa, xa, c, col_scale, short_ok);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (u + 1 < steps) {
      // odd step: weights in wb, stage 1
      park_x_rows<BITS, ROUNDS>(xr, my_stages + stage_bytes, lane, ty, p.tiles_per_wg);
      stage_ready();
      if constexpr (PROBE == kProbeComputeOnly) {
        wa = wb;
        keep_registers(wa, xr);
      } else {
        fetch_x_rows<BITS, ROUNDS>(xr, p, x_rsrc, ks_begin + u + 2, lane, ty, p.tiles_per_wg);
        load_weights_lds_mfma<BITS, QOP, GROUPS_PER_RUN>(wa, p, w_rsrc, tables, u + 2, ks_begin + u + 2, lane, row);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (u + 1 < units) {
        const LdsActivations<BITS> xa{my_stages + stage_bytes + operand_offset};
        if constexpr (PROBE == kProbeLoadsOnly)
          consume_unit(acc, wb, xa);
        else
          compute_unit_mfma<BITS, QOP, GROUPS_PER_RUN, ACT>(acc, wb, xa, c, col_scale, short_ok);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    u += 2;
  } while (u < steps);

  // Lane l holds D[rows 4*(l/16) .. +3 of the tile][batch row l % 16].
  f32x4 sum = acc;
  if (split_k > 1) {
    f32x4* const combine = reinterpret_cast<f32x4*>(lds + split_k * 2 * stage_bytes);
    combine[(ty * split_k + kw) * kWave + lane] = acc;
    __syncthreads();
    if (kw != 0) return;
    const f32x4* part = combine + ty * split_k * kWave + lane;
    sum = part[0];
    for (int w = 1; w < split_k; ++w) sum += part[w * kWave];
  }
  if (tile_raw >= tiles) return;
  const int m = lane % kTileRows;
  const int n0 = tile * kTileRows + 4 * (lane / kTileRows);
  if (m < m_batch) {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int n = n0 + v;
      if (n < p.n_out) {
        if constexpr (ACT == kActBf16) {
          const float b = has_bias ? bf16_low_to_f32(reinterpret_cast<const uint16_t*>(tail.bias)[n]) : 0.0f;
          const float r = epilogue_value(tail, sum[v], has_bias, b);
          reinterpret_cast<uint16_t*>(tail.y)[(size_t)m * (size_t)p.n_out + n] = (uint16_t)pack_bf16(r, 0.0f);
        } else {
          const float r = epilogue_value(tail, sum[v], has_bias, has_bias ? (float)tail.bias[n] : 0.0f);
          tail.y[(size_t)m * (size_t)p.n_out + n] = (half_t)r;
        }
      }
    }
  }
}

template <int BITS, int QOP, int GPR, int T>
hipError_t launch_mfma_kernel_t(const GemvLaunch& g) {
  return launch(gemv_mfma_kernel<BITS, QOP, GPR, T>, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale,
                g.zero_add, g.n_out, g.k, pack_steps(num_ksteps(g.k, BITS), g.plan.steps_per_wave), g.plan.workgroups,
                g.plan.wgs_per_xcd, pack_group(g.group_size, g.plan.tiles_per_wg, g.tail.route != nullptr), g.tail);
}

template <int BITS, int QOP, int GPR>
hipError_t launch_mfma_kernel(const GemvLaunch& g) {
  switch (g.plan.tiles_per_wave) {
    case 1: return launch_mfma_kernel_t<BITS, QOP, GPR, 1>(g);
    case 2: return launch_mfma_kernel_t<BITS, QOP, GPR, 2>(g);
    default: return launch_mfma_kernel_t<BITS, QOP, GPR, 4>(g);
  }
}

template <int BITS, int QOP>
hipError_t launch_mfma_gpr(const GemvLaunch& g, int gpr) {
  if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
    return launch_mfma_kernel<BITS, QOP, 1>(g);
  } else {
    switch (gpr) {
      case 1: return launch_mfma_kernel<BITS, QOP, 1>(g);
      case 2: return launch_mfma_kernel<BITS, QOP, 2>(g);
      default: return launch_mfma_kernel<BITS, QOP, 4>(g);
    }
  }
}

hipError_t launch_mfma(const GemvLaunch& g, int bits, int qop, int gpr) {
  if (bits == 4) {
    switch (qop) {
      case 1: return launch_mfma_gpr<4, 1>(g, gpr);
      case 2: return launch_mfma_gpr<4, 2>(g, gpr);
      default: return launch_mfma_gpr<4, 3>(g, gpr);
    }
  }
  switch (qop) {
    case 1: return launch_mfma_gpr<8, 1>(g, gpr);
    case 2: return launch_mfma_gpr<8, 2>(g, gpr);
    default: return launch_mfma_gpr<8, 3>(g, gpr);
  }
}

// LDS-staged matrix-core kernel: 2 tiles per workgroup share the activation stage.
template <int BITS, int QOP, int GPR, int ROUNDS, int ACT, bool SHARED, int PROBE = kProbeNone>
hipError_t launch_mfma_lds_kernel_r(const GemvLaunch& g) {
  const auto kernel = gemv_mfma_lds_kernel<BITS, QOP, GPR, ROUNDS, ACT, SHARED, PROBE>;
  if (g.lds > 48 * 1024) {
    // More than 48 KiB of dynamic LDS has to be granted per kernel and device; remember the
    // largest grant so that only the first such launch pays for the call.
    constexpr int kMaxDevices = 64;
    static std::atomic<int> granted[kMaxDevices];
    static std::mutex grant_mutex;
    const int device = g.device;  // the device of the launch stream, not the calling thread's current one
    const bool tracked = device >= 0 && device < kMaxDevices;
    if (!tracked || granted[device].load() < (int)g.lds) {
      std::lock_guard<std::mutex> lock(grant_mutex);  // grant and bookkeeping change together
      if (!tracked || granted[device].load() < (int)g.lds) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds);
        if (e != hipSuccess) return e;
        if (tracked) granted[device].store((int)g.lds);
      }
    }
  }
  return launch(kernel, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale, g.zero_add, g.n_out, g.k,
                pack_steps(num_ksteps(g.k, BITS), g.plan.steps_per_wave), g.plan.workgroups, g.tail.num_groups,
                pack_group(g.group_size, g.plan.tiles_per_wg, g.tail.route != nullptr), g.tail);
}

template <int BITS, int QOP, int GPR, int ACT>
hipError_t launch_mfma_lds_kernel(const GemvLaunch& g, int rounds) {
  // rounds = staged rows (8 or 16) / tiles per workgroup: 16 means one tile, 2 and 4 several,
  // 8 either (8 rows for one tile, or 16 rows shared by two).
  switch (rounds) {
    case 2: return launch_mfma_lds_kernel_r<BITS, QOP, GPR, 2, ACT, true>(g);
    case 4: return launch_mfma_lds_kernel_r<BITS, QOP, GPR, 4, ACT, true>(g);
    case 8:
      return g.plan.tiles_per_wg > 1 ? launch_mfma_lds_kernel_r<BITS, QOP, GPR, 8, ACT, true>(g)
                                     : launch_mfma_lds_kernel_r<BITS, QOP, GPR, 8, ACT, false>(g);
    default: return launch_mfma_lds_kernel_r<BITS, QOP, GPR, 16, ACT, false>(g);
  }
}

template <int BITS, int QOP, int ACT>
hipError_t launch_mfma_lds_gpr(const GemvLaunch& g, int gpr, int rounds) {
  if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
    return launch_mfma_lds_kernel<BITS, QOP, 1, ACT>(g, rounds);
  } else {
    switch (gpr) {
      case 1: return launch_mfma_lds_kernel<BITS, QOP, 1, ACT>(g, rounds);
      case 2: return launch_mfma_lds_kernel<BITS, QOP, 2, ACT>(g, rounds);
      default: return launch_mfma_lds_kernel<BITS, QOP, 4, ACT>(g, rounds);
    }
  }
}

template <int ACT>
hipError_t launch_mfma_lds_act(const GemvLaunch& g, int bits, int qop, int gpr, int rounds) {
  if (bits == 4) {
    switch (qop) {
      case 1: return launch_mfma_lds_gpr<4, 1, ACT>(g, gpr, rounds);
      case 2: return launch_mfma_lds_gpr<4, 2, ACT>(g, gpr, rounds);
      default: return launch_mfma_lds_gpr<4, 3, ACT>(g, gpr, rounds);
    }
  }
  switch (qop) {
    case 1: return launch_mfma_lds_gpr<8, 1, ACT>(g, gpr, rounds);
    case 2: return launch_mfma_lds_gpr<8, 2, ACT>(g, gpr, rounds);
    default: return launch_mfma_lds_gpr<8, 3, ACT>(g, gpr, rounds);
  }
}

// Measurement builds exist for int4 scale-and-zero fp16 launches whose workgroups share their stages:
// one or two groups per lane run, 4 or 8 staging rounds per wave (8 or 16 rows over 2 tiles).
template <int PROBE>
hipError_t launch_mfma_lds_probe_kind(const GemvLaunch& g, int gpr, int rounds) {
  constexpr int kQ = MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  if (gpr == 1)
    return rounds == 4 ? launch_mfma_lds_kernel_r<4, kQ, 1, 4, kActF16, true, PROBE>(g)
                       : launch_mfma_lds_kernel_r<4, kQ, 1, 8, kActF16, true, PROBE>(g);
  return rounds == 4 ? launch_mfma_lds_kernel_r<4, kQ, 2, 4, kActF16, true, PROBE>(g)
                     : launch_mfma_lds_kernel_r<4, kQ, 2, 8, kActF16, true, PROBE>(g);
}

bool mfma_lds_probe_exists(int bits, int qop, int gpr, int rounds, int act, int tiles_per_wg) {
  return bits == 4 && qop == MGEMV_FINEGRAINED_SCALE_AND_ZEROS && (gpr == 1 || gpr == 2) && (rounds == 4 || rounds == 8) &&
         act == kActF16 && tiles_per_wg > 1;
}

hipError_t launch_mfma_lds_probe(const GemvLaunch& g, int gpr, int rounds, int probe) {
  return probe == kProbeLoadsOnly ? launch_mfma_lds_probe_kind<kProbeLoadsOnly>(g, gpr, rounds)
                                  : launch_mfma_lds_probe_kind<kProbeComputeOnly>(g, gpr, rounds);
}

hipError_t launch_mfma_lds(const GemvLaunch& g, int bits, int qop, int gpr, int rounds, int act) {
  return act == kActBf16 ? launch_mfma_lds_act<kActBf16>(g, bits, qop, gpr, rounds)
                         : launch_mfma_lds_act<kActF16>(g, bits, qop, gpr, rounds);
}

}  // namespace mgemv
