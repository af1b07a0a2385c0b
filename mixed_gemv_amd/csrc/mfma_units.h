// Device code shared by the matrix-core kernels: the registers of one unit of weights, the
// activation operands of one k step, and the arithmetic of a unit (dequantise, matrix instructions).
#ifndef MIXED_GEMV_AMD_MFMA_UNITS_H_
#define MIXED_GEMV_AMD_MFMA_UNITS_H_

#include "kernel_common.h"

namespace mgemv {

// Activation operands of all matrix instructions of one k step (shared by the wave's tiles).
template <int BITS>
struct MfmaActivations {
  u32x4 x[kBlocksPerUnit][BITS == 4 ? 4 : 2];
};

// Weights, scales and zeros of one unit.
template <int BITS, int GROUPS_PER_RUN>
struct MfmaWeights {
  u32x4 w[kBlocksPerUnit];
  uint32_t s[GROUPS_PER_RUN];
  uint32_t z[GROUPS_PER_RUN];
};

template <int BITS>
__device__ __forceinline__ void load_activations_mfma(MfmaActivations<BITS>& f, const Problem& p,
                                                      __amdgpu_buffer_rsrc_t x_rsrc, int kstep, int lane) {
  using G = Geometry<BITS>;
  constexpr int kFrags = BITS == 4 ? 4 : 2;  // matrix instructions per block
  const int k_run = kstep * G::kStepK + (lane / kTileRows) * G::kRunK;
  const int m = lane % kTileRows;
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) {
    const int k_block = k_run + i * G::kChunkK;
    // Batch rows past m_batch fall outside the descriptor and read as zero; reduction positions
    // past k are sent there (k is a multiple of 8, so each 128-bit piece is wholly inside or outside).
#pragma unroll
    for (int j = 0; j < kFrags; ++j) {
      const uint32_t off = k_block + j * 8 < p.k ? (uint32_t)(m * p.k + k_block + j * 8) * 2u : 0xfffffff0u;
      f.x[i][j] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, kCacheDefault);
    }
  }
}

template <int BITS, int QOP, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_weights_mfma(MfmaWeights<BITS, GROUPS_PER_RUN>& f, const Problem& p,
                                                  __amdgpu_buffer_rsrc_t w_rsrc, int byte_offset, int kstep, int lane,
                                                  int row) {
  using G = Geometry<BITS>;
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i)
    f.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, lane * kChunkBytes, byte_offset + i * kBlockBytes, kCacheStream);
  if constexpr (QOP != MGEMV_PER_COLUMN_SCALE_ONLY) {
    const int k_run = kstep * G::kStepK + (lane / kTileRows) * G::kRunK;
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
      const int grp = group_of(p, k_run + gi * (G::kRunK / GROUPS_PER_RUN));
      const int idx = grp * p.n_out + row;
      f.s[gi] = load_half_bits(p.scale + idx);
      if constexpr (QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS) f.z[gi] = load_half_bits(p.zero_add + idx);
    }
  }
}

// Where the activation operand of matrix instruction (block i, fragment j) comes from:
// registers filled by load_activations_mfma, or the workgroup's LDS stage of the current k step.
template <int BITS>
__device__ __forceinline__ u32x4 mfma_operand(const MfmaActivations<BITS>& xa, int i, int j) { return xa.x[i][j]; }

template <int BITS>
struct LdsActivations {
  const uint8_t* lane_base;  // row (lane % 16) of the stage, at this lane's k slice
};
template <int BITS>
__device__ __forceinline__ u32x4 mfma_operand(const LdsActivations<BITS>& xa, int i, int j) {
  using G = Geometry<BITS>;
  return *reinterpret_cast<const u32x4*>(xa.lane_base + (i * G::kChunkK + j * 8) * 2);
}

// The activation operands of the matrix instructions of block i.
template <int BITS, typename Activations>
__device__ __forceinline__ void load_block_operands(const Activations& xa, int i, u32x4 (&ops)[BITS == 4 ? 4 : 2]) {
#pragma unroll
  for (int j = 0; j < (BITS == 4 ? 4 : 2); ++j) ops[j] = mfma_operand<BITS>(xa, i, j);
}

template <int BITS, int QOP, int GROUPS_PER_RUN, bool SHORT, int ACT, typename Activations>
__device__ __forceinline__ void compute_unit_mfma_form(f32x4& acc, const MfmaWeights<BITS, GROUPS_PER_RUN>& f,
                                                       const Activations& xa, const ConvertRegs& c,
                                                       half2_t col_scale2) {
  constexpr bool kHasZero = QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  constexpr int kFrags = BITS == 4 ? 4 : 2;
  // The operands of block i+1 are requested before block i is dequantised, and the request is
  // pinned there: left alone the compiler reads each operand right in front of its matrix
  // instruction and the wave sits through the LDS latency sixteen times per unit.
  u32x4 ops[2][kFrags];
  load_block_operands<BITS>(xa, 0, ops[0]);
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) {
    if (i + 1 < kBlocksPerUnit) load_block_operands<BITS>(xa, i + 1, ops[(i + 1) & 1]);
    __builtin_amdgcn_sched_barrier(0);
    const u32x4 (&op)[kFrags] = ops[i & 1];
    const int gi = i * GROUPS_PER_RUN / kBlocksPerUnit;
    if constexpr (ACT == kActBf16) {
      // bf16: the same dequantiser as the VALU kernel (SHORT = fused form), v_mfma_f32_16x16x32_bf16
      const uint32_t s_bits = QOP != MGEMV_PER_COLUMN_SCALE_ONLY ? f.s[gi] : as_u32(col_scale2);
      const Bf16Scale bs = make_bf16_scale<BITS, SHORT>(s_bits, kHasZero ? f.z[gi] : 0u);
#pragma unroll
      for (int j = 0; j < kFrags; ++j) {
        u32x4 a;
        if constexpr (BITS == 4) {
          uint32_t d[4];
          dequant_int4_word_bf16<kHasZero, SHORT>(f.w[i][j], c, bs, d);
          a = u32x4{d[0], d[1], d[2], d[3]};
        } else {
          uint32_t d0[2], d1[2];
          dequant_int8_word_bf16<kHasZero, SHORT>(f.w[i][2 * j], bs, d0);
          dequant_int8_word_bf16<kHasZero, SHORT>(f.w[i][2 * j + 1], bs, d1);
          a = u32x4{d0[0], d0[1], d1[0], d1[1]};
        }
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                      __builtin_bit_cast(bf16x8_t, op[j]), acc, 0, 0, 0);
      }
      continue;
    }
    half2_t s2 = col_scale2, z2 = half2_t{};
    if constexpr (QOP != MGEMV_PER_COLUMN_SCALE_ONLY) s2 = splat_low(f.s[gi]);
    if constexpr (kHasZero) z2 = splat_low(f.z[gi]);
    if constexpr (BITS == 4) {
      ShortFormScale sf{};
      if constexpr (SHORT) sf = make_short_form_scale(s2);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half2_t d[4];
        if constexpr (SHORT) {
          dequant_int4_word_short<kHasZero>(f.w[i][j], c, sf, z2, d);
        } else {
          half2_t q[4];
          convert_int4_word(f.w[i][j], c, q);
#pragma unroll
          for (int h = 0; h < 4; ++h) d[h] = dequant_pair<kHasZero>(q[h], s2, z2);
        }
        u32x4 a;
#pragma unroll
        for (int h = 0; h < 4; ++h) a[h] = as_u32(d[h]);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                     __builtin_bit_cast(half8_t, op[j]), acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        half2_t q0[2], q1[2];
        convert_int8_word(f.w[i][2 * j], c, q0);
        convert_int8_word(f.w[i][2 * j + 1], c, q1);
        u32x4 a;
        a[0] = as_u32(dequant_pair<kHasZero>(q0[0], s2, z2));
        a[1] = as_u32(dequant_pair<kHasZero>(q0[1], s2, z2));
        a[2] = as_u32(dequant_pair<kHasZero>(q1[0], s2, z2));
        a[3] = as_u32(dequant_pair<kHasZero>(q1[1], s2, z2));
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                     __builtin_bit_cast(half8_t, op[j]), acc, 0, 0, 0);
      }
    }
  }
}

template <int BITS, int QOP, int GROUPS_PER_RUN, int ACT = kActF16, typename Activations>
__device__ __forceinline__ void compute_unit_mfma(f32x4& acc, const MfmaWeights<BITS, GROUPS_PER_RUN>& f,
                                                  const Activations& xa, const ConvertRegs& c,
                                                  half2_t col_scale2, bool short_allowed) {
  if constexpr (BITS == 4 || ACT == kActBf16) {
    bool take_short = short_allowed;
    if constexpr (QOP != MGEMV_PER_COLUMN_SCALE_ONLY) take_short = take_short && wave_scales_permit_short_form<ACT>(f.s);
    if (take_short) {
      compute_unit_mfma_form<BITS, QOP, GROUPS_PER_RUN, true, ACT>(acc, f, xa, c, col_scale2);
      return;
    }
  }
  compute_unit_mfma_form<BITS, QOP, GROUPS_PER_RUN, false, ACT>(acc, f, xa, c, col_scale2);
}

// Weights, scales and zeros of unit `unit` of the wave's k range through descriptors: everything
// unit-dependent sits in the bounds-checked VGPR offset, so a prefetch past the range reads zeros.
template <int BITS, int QOP, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_weights_lds_mfma(MfmaWeights<BITS, GROUPS_PER_RUN>& f, const Problem& p,
                                                      __amdgpu_buffer_rsrc_t w_rsrc, const ScaleTables& tables, int unit,
                                                      int kstep, int lane, int row) {
  using G = Geometry<BITS>;
  const int voffset = unit * kUnitBytes + lane * kChunkBytes;
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i)
    f.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, voffset + i * kBlockBytes, 0, kCacheStream);
  if constexpr (QOP != MGEMV_PER_COLUMN_SCALE_ONLY) {
    const int k_run = kstep * G::kStepK + (lane / kTileRows) * G::kRunK;
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
      const int grp = group_of(p, k_run + gi * (G::kRunK / GROUPS_PER_RUN));
      const int off = (grp * p.n_out + row) * 2;
      f.s[gi] = load_b16_low(tables.scale, off);
      if constexpr (QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS) f.z[gi] = load_b16_low(tables.zero, off);
    }
  }
}

// Activation rows on their way through LDS: a wave fetches whole rows of a k step (64 lanes x 16 or 8 bytes,
// fully coalesced), parks them row by row, and the lanes read their operand pieces back in matrix-instruction shape.
template <int BITS>
struct XStage {
  static constexpr int kRowBytes = Geometry<BITS>::kStepK * 2;  // 1024 | 512
  static constexpr int kRowStride = kRowBytes + 16;             // bank spread for the operand reads
  static constexpr int kLaneBytes = kRowBytes / kWave;          // 16 | 8
};

template <int BITS, int ROUNDS>
struct XRows {
  uint32_t v[ROUNDS][BITS == 4 ? 4 : 2];
};

template <int BITS, int ROUNDS>
__device__ __forceinline__ void fetch_x_rows(XRows<BITS, ROUNDS>& r, const Problem& p, __amdgpu_buffer_rsrc_t x_rsrc,
                                             int kstep, int lane, int first_row, int row_step, int rows = ROUNDS) {
  using G = Geometry<BITS>;
  const int k0 = kstep * G::kStepK + lane * (XStage<BITS>::kLaneBytes / 2);
#pragma unroll
  for (int j = 0; j < ROUNDS; ++j) {
    if (j >= rows) break;  // wave-uniform
    const int row = first_row + j * row_step;
    // rows past m_batch fall outside the descriptor, reduction positions past k are sent there
    const uint32_t off = k0 < p.k ? (uint32_t)(row * p.k + k0) * 2u : 0xfffffff0u;
    if constexpr (BITS == 4) {
      const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, 0, kCacheDefault);
      r.v[j][0] = t[0]; r.v[j][1] = t[1]; r.v[j][2] = t[2]; r.v[j][3] = t[3];
    } else {
      const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(x_rsrc, (int)off, 0, kCacheDefault);
      r.v[j][0] = t[0]; r.v[j][1] = t[1];
    }
  }
}

template <int BITS, int ROUNDS>
__device__ __forceinline__ void park_x_rows(const XRows<BITS, ROUNDS>& r, uint8_t* stage, int lane, int first_row,
                                            int row_step, int rows = ROUNDS) {
#pragma unroll
  for (int j = 0; j < ROUNDS; ++j) {
    if (j >= rows) break;  // wave-uniform
    uint8_t* dst = stage + (first_row + j * row_step) * XStage<BITS>::kRowStride + lane * XStage<BITS>::kLaneBytes;
    if constexpr (BITS == 4) {
      *reinterpret_cast<u32x4*>(dst) = u32x4{r.v[j][0], r.v[j][1], r.v[j][2], r.v[j][3]};
    } else {
      *reinterpret_cast<u32x2*>(dst) = u32x2{r.v[j][0], r.v[j][1]};
    }
  }
}

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_MFMA_UNITS_H_
