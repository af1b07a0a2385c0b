// The VALU GEMV kernel for gfx950 (MI355X), wave64: 1-4 activation rows.
//
// One wavefront works on a contiguous range of k steps (units of tile_layout.h) of one 16-row
// tile of the weight matrix, or of several consecutive tiles one after the other.  Per unit it
// issues four 1-KiB weight loads, one activation load and the scale/zero loads, dequantises
// in packed fp16 to the bits of gemv/warp/warp_dequantizer.h:52-59 (rounded product, then
// rounded sum), and accumulates in fp32 with v_dot2c_f32_f16 whose activation operand is a DPP
// row broadcast.  Several waves of a workgroup split the k range of the same tiles (split-K);
// their per-lane partial sums meet in LDS, are summed in a fixed order, biased, rounded to
// fp16 and stored.  This covers, for the reference, the main loops
// of gemv/threadblock/dq_mma_singlestage_{finegrained,percol}.h, the reductions of
// gemv/warp/reduce.h and gemv/threadblock/accumulator_combine.h, and the epilogue of
// epilogue/threadblock/epilogue.h.
#ifndef MIXED_GEMV_AMD_GEMV_DPP_KERNEL_H_
#define MIXED_GEMV_AMD_GEMV_DPP_KERNEL_H_

#include "kernel_common.h"

namespace mgemv {

// Everything one lane needs for one unit.  Scale and additive zero are kept as packed
// (s, s) / (z, z) pairs in 32-bit registers.
template <int BITS, int MB, int GROUPS_PER_RUN>
struct UnitFragment {
  u32x4 w[kBlocksPerUnit];                // 4 chunks of this lane's row
  uint32_t x[MB][BITS == 4 ? 4 : 2];      // this lane's piece of the activation run
  uint32_t s[GROUPS_PER_RUN];             // fp16 scale of each group of the run (low 16 bits; the rest is unspecified)
  uint32_t z[GROUPS_PER_RUN];             // fp16 additive zero (low 16 bits; the rest is unspecified)
};

// Where a lane reads for the current unit.  Everything that varies from unit to unit sits in
// the VGPR offset of the buffer loads (the part of the address that the hardware
// bounds-checks), so reads past the wave's last unit return zero instead of touching foreign
// memory.
//
// GROUPS_PER_RUN 1 or 2 ("regular"): the group size divides the k step (or there is a single
// group, the per-column mode), so a lane's scale / zero offset advances by a constant per
// unit.  GROUPS_PER_RUN 4 ("generic", any group size that is a multiple of 32): one lookup
// per block with an integer division.
template <int BITS, int GROUPS_PER_RUN>
struct WaveCursor {
  int w_voffset;                   // byte offset of this lane's chunk of block 0 inside the wave's weight range
  int x_voffset;                   // byte offset of this lane's activations
  int sz_voffset[GROUPS_PER_RUN];  // regular: byte offset of this lane's scale / zero
  int k_run;                       // generic: first reduction index of the lane's run
  int row;                         // generic: this lane's row (not clamped; padded rows are never stored)
};

// A wave walks the same k range of several consecutive tiles, one after the other, as ONE
// stream of units: these are the (wave-uniform) strides of that walk.
struct TileWalk {
  int units;      // units per tile for this wave
  int left;       // units of the current tile not yet addressed
  int w_jump;     // from the last unit of a tile to the first unit of the next tile, bytes
  int x_back;     // activations: back to the start of the k range, bytes
  int k_back;     // the same in reduction elements
  int sz_stride;  // regular: bytes per k step in the scale / zero tables
  int sz_jump;    // regular: from the last unit of a tile to the first of the next (16 rows on)
};

template <int BITS, int GROUPS_PER_RUN>
__device__ __forceinline__ WaveCursor<BITS, GROUPS_PER_RUN> make_cursor(const Problem& p, bool per_column, int ks_begin,
                                                                       int units, int lane, int row, TileWalk& walk) {
  using G = Geometry<BITS>;
  WaveCursor<BITS, GROUPS_PER_RUN> c;
  c.w_voffset = lane * kChunkBytes;
  c.x_voffset = ks_begin * (G::kStepK * 2) + lane * (BITS == 4 ? 16 : 8);
  c.k_run = ks_begin * G::kStepK + (lane / kTileRows) * G::kRunK;
  c.row = row;
  walk.units = units;
  walk.left = units;
  walk.w_jump = (p.ksteps - units + 1) * kUnitBytes;
  walk.x_back = (units - 1) * (G::kStepK * 2);
  walk.k_back = (units - 1) * G::kStepK;
  walk.sz_stride = 0;
  if constexpr (GROUPS_PER_RUN != 4) {
    if (per_column) {
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) c.sz_voffset[gi] = row * 2;
    } else {
      // Regular modes: the group size divides the k step, hence is a power of two; no divisions.
      const int shift = __builtin_ctz((unsigned)p.group_size);
      const int groups_per_step = G::kStepK >> shift;
      walk.sz_stride = groups_per_step * p.n_out * 2;
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
        const int k_local = (lane / kTileRows) * G::kRunK + gi * (G::kRunK / GROUPS_PER_RUN);
        c.sz_voffset[gi] = ((ks_begin * groups_per_step + (k_local >> shift)) * p.n_out + row) * 2;
      }
    }
  } else {
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) c.sz_voffset[gi] = 0;
  }
  walk.sz_jump = kTileRows * 2 - (units - 1) * walk.sz_stride;
  return c;
}

// To the next unit of the stream: the next k step of the same tile or, when the wave walks
// several tiles (MULTI), the first unit of the next tile.
template <bool MULTI, int BITS, int GROUPS_PER_RUN>
__device__ __forceinline__ void advance(WaveCursor<BITS, GROUPS_PER_RUN>& c, TileWalk& walk) {
  using G = Geometry<BITS>;
  bool wrap = false;
  if constexpr (MULTI) {
    walk.left -= 1;
    wrap = walk.left == 0;
  }
  c.w_voffset += wrap ? walk.w_jump : kUnitBytes;
  c.x_voffset += wrap ? -walk.x_back : G::kStepK * 2;
  if constexpr (GROUPS_PER_RUN == 4) {
    c.k_run += wrap ? -walk.k_back : G::kStepK;
    c.row += wrap ? kTileRows : 0;
  } else {
    const int step = wrap ? walk.sz_jump : walk.sz_stride;
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) c.sz_voffset[gi] += step;
  }
  if constexpr (MULTI) walk.left = wrap ? walk.units : walk.left;
}

// The operands that go with a unit's weights: activations, scales, additive zeros.
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_operands(UnitFragment<BITS, MB, GROUPS_PER_RUN>& f, const Problem& p,
                                              const __amdgpu_buffer_rsrc_t (&x_rsrc)[MB], const ScaleTables& tables,
                                              const WaveCursor<BITS, GROUPS_PER_RUN>& c) {
  using G = Geometry<BITS>;
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    if constexpr (BITS == 4) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc[m], c.x_voffset, 0, kCacheDefault);
      f.x[m][0] = v[0]; f.x[m][1] = v[1]; f.x[m][2] = v[2]; f.x[m][3] = v[3];
    } else {
      const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(x_rsrc[m], c.x_voffset, 0, kCacheDefault);
      f.x[m][0] = v[0]; f.x[m][1] = v[1];
    }
  }
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) {
    int voffset;
    if constexpr (GROUPS_PER_RUN == 4) {
      voffset = (group_of(p, c.k_run + gi * G::kChunkK) * p.n_out + c.row) * 2;
    } else {
      voffset = c.sz_voffset[gi];
    }
    f.s[gi] = load_b16_low(tables.scale, voffset);
    if constexpr (QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS)
      f.z[gi] = load_b16_low(tables.zero, voffset);
  }
}

template <int BITS, int MB, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_weights(UnitFragment<BITS, MB, GROUPS_PER_RUN>& f, __amdgpu_buffer_rsrc_t w_rsrc,
                                             int w_voffset) {
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i)
    f.w[i] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, w_voffset + i * kBlockBytes, 0, kCacheStream);
}

// Everything one lane needs for one unit.  The weight blocks go last: loads return in order,
// so block i can be consumed as soon as its own chunk is in, with only the later blocks (and
// the next unit) still outstanding.
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN>
__device__ __forceinline__ void load_unit(UnitFragment<BITS, MB, GROUPS_PER_RUN>& f, const Problem& p,
                                          __amdgpu_buffer_rsrc_t w_rsrc, const __amdgpu_buffer_rsrc_t (&x_rsrc)[MB],
                                          const ScaleTables& tables, const WaveCursor<BITS, GROUPS_PER_RUN>& c) {
  load_operands<BITS, QOP, MB, GROUPS_PER_RUN>(f, p, x_rsrc, tables, c);
  load_weights<BITS, MB, GROUPS_PER_RUN>(f, w_rsrc, c.w_voffset);
}

// Measurement build "arithmetic only": a wave loads its first unit and computes that unit's
// registers again for every further unit of its range.  Nothing is loaded; the registers are made
// opaque each time so that no part of the arithmetic can be hoisted out of the unit loop.
template <int BITS, int MB, int GROUPS_PER_RUN>
__device__ __forceinline__ void reuse_unit(UnitFragment<BITS, MB, GROUPS_PER_RUN>& f) {
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) asm volatile("" : "+v"(f.w[i]));
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int h = 0; h < (BITS == 4 ? 4 : 2); ++h) asm volatile("" : "+v"(f.x[m][h]));
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) asm volatile("" : "+v"(f.s[gi]), "+v"(f.z[gi]));
}

// One 32-bit word of block I: convert, dequantise, dot.  Lane (4 I + J) of the DPP row holds
// the activations that pair with this word.  SHORT selects the single-FMA int4 dequantiser
// (device_math.h); the caller guarantees that every lane's scale permits it.
template <int BITS, bool HAS_ZERO, bool SHORT, int MB, int I, int J>
__device__ __forceinline__ void compute_word(float (&acc)[MB], uint32_t w, const uint32_t (&x)[MB][BITS == 4 ? 4 : 2],
                                             const ConvertRegs& c, half2_t s2, half2_t z2, const ShortFormScale& f) {
  constexpr int kPairs = BITS == 4 ? 4 : 2;
  half2_t d[kPairs];
  if constexpr (BITS == 4 && SHORT) {
    dequant_int4_word_short<HAS_ZERO>(w, c, f, z2, d);
  } else {
    half2_t q[kPairs];
    if constexpr (BITS == 4) convert_int4_word(w, c, q); else convert_int8_word(w, c, q);
#pragma unroll
    for (int h = 0; h < kPairs; ++h) d[h] = dequant_pair<HAS_ZERO>(q[h], s2, z2);
  }
#pragma unroll
  for (int h = 0; h < kPairs; ++h) {
#pragma unroll
    for (int m = 0; m < MB; ++m) dot2_row_bcast<4 * I + J>(acc[m], x[m][h], d[h]);
  }
}

// The same for bf16 operands; SHORT selects the fused form.
template <int BITS, bool HAS_ZERO, bool SHORT, int MB, int I, int J>
__device__ __forceinline__ void compute_word_bf16(float (&acc)[MB], uint32_t w,
                                                  const uint32_t (&x)[MB][BITS == 4 ? 4 : 2], const ConvertRegs& c,
                                                  const Bf16Scale& f) {
  constexpr int kPairs = BITS == 4 ? 4 : 2;
  uint32_t d[kPairs];
  if constexpr (BITS == 4) dequant_int4_word_bf16<HAS_ZERO, SHORT>(w, c, f, d);
  else dequant_int8_word_bf16<HAS_ZERO, SHORT>(w, f, d);
#pragma unroll
  for (int h = 0; h < kPairs; ++h) {
#pragma unroll
    for (int m = 0; m < MB; ++m) dot2_row_bcast_bf16<4 * I + J>(acc[m], x[m][h], d[h]);
  }
}

template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, bool SHORT, int I, int ACT>
__device__ __forceinline__ void compute_block(float (&acc)[MB], const UnitFragment<BITS, MB, GROUPS_PER_RUN>& f,
                                              const ConvertRegs& c) {
  constexpr bool kHasZero = QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  constexpr int gi = I * GROUPS_PER_RUN / kBlocksPerUnit;
  if constexpr (ACT == kActBf16) {
    const Bf16Scale bs = make_bf16_scale<BITS, SHORT>(f.s[gi], kHasZero ? f.z[gi] : 0u);
    compute_word_bf16<BITS, kHasZero, SHORT, MB, I, 0>(acc, f.w[I][0], f.x, c, bs);
    compute_word_bf16<BITS, kHasZero, SHORT, MB, I, 1>(acc, f.w[I][1], f.x, c, bs);
    compute_word_bf16<BITS, kHasZero, SHORT, MB, I, 2>(acc, f.w[I][2], f.x, c, bs);
    compute_word_bf16<BITS, kHasZero, SHORT, MB, I, 3>(acc, f.w[I][3], f.x, c, bs);
  } else {
    const half2_t s2 = splat_low(f.s[gi]);
    half2_t z2 = half2_t{};
    if constexpr (kHasZero) z2 = splat_low(f.z[gi]);
    ShortFormScale sf{};
    if constexpr (BITS == 4 && SHORT) sf = make_short_form_scale(s2);
    compute_word<BITS, kHasZero, SHORT, MB, I, 0>(acc, f.w[I][0], f.x, c, s2, z2, sf);
    compute_word<BITS, kHasZero, SHORT, MB, I, 1>(acc, f.w[I][1], f.x, c, s2, z2, sf);
    compute_word<BITS, kHasZero, SHORT, MB, I, 2>(acc, f.w[I][2], f.x, c, s2, z2, sf);
    compute_word<BITS, kHasZero, SHORT, MB, I, 3>(acc, f.w[I][3], f.x, c, s2, z2, sf);
  }
}

template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, bool SHORT, int ACT>
__device__ __forceinline__ void compute_unit_form(float (&acc)[MB], const UnitFragment<BITS, MB, GROUPS_PER_RUN>& f,
                                                  const ConvertRegs& regs) {
  const ConvertRegs c = (ACT == kActF16 && BITS == 4 && !SHORT) ? general_form_regs(regs) : regs;
  compute_block<BITS, QOP, MB, GROUPS_PER_RUN, SHORT, 0, ACT>(acc, f, c);
  compute_block<BITS, QOP, MB, GROUPS_PER_RUN, SHORT, 1, ACT>(acc, f, c);
  compute_block<BITS, QOP, MB, GROUPS_PER_RUN, SHORT, 2, ACT>(acc, f, c);
  compute_block<BITS, QOP, MB, GROUPS_PER_RUN, SHORT, 3, ACT>(acc, f, c);
  // The two forms meet again after this call, and the compiler may place a register copy of
  // the accumulators at that join: make them safe to read by any instruction first.
#pragma unroll
  for (int m = 0; m < MB; ++m) settle_dot_chain(acc[m]);
}

// short_allowed: wave-uniform.
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, int ACT = kActF16, int PROBE = kProbeNone>
__device__ __forceinline__ void compute_unit(float (&acc)[MB], const UnitFragment<BITS, MB, GROUPS_PER_RUN>& f,
                                             const ConvertRegs& c, bool short_allowed) {
  if constexpr (PROBE == kProbeLoadsOnly) {
    // every register of the unit has to arrive, nothing is computed
    uint32_t t = 0;
#pragma unroll
    for (int gi = 0; gi < GROUPS_PER_RUN; ++gi) t ^= f.s[gi] ^ (QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? f.z[gi] : 0u);
#pragma unroll
    for (int i = 0; i < kBlocksPerUnit; ++i) t ^= f.w[i][0] ^ f.w[i][1] ^ f.w[i][2] ^ f.w[i][3];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
      uint32_t tm = t;
#pragma unroll
      for (int h = 0; h < (BITS == 4 ? 4 : 2); ++h) tm ^= f.x[m][h];
      acc[m] += __builtin_bit_cast(float, tm & 0x3fffffffu);
    }
    return;
  }
  if constexpr (BITS == 4 || ACT == kActBf16) {
    if (short_allowed && wave_scales_permit_short_form<ACT>(f.s)) {
      compute_unit_form<BITS, QOP, MB, GROUPS_PER_RUN, true, ACT>(acc, f, c);
      return;
    }
  }
  compute_unit_form<BITS, QOP, MB, GROUPS_PER_RUN, false, ACT>(acc, f, c);
}

// Epilogue: fp32 add of the bias, one rounding to fp16
// (host/mixed_gemv.h:102-103; epilogue/threadblock/epilogue.h:50-75).
template <int ACT>
__device__ __forceinline__ void store_outputs(const GemvTail& tail, bool has_bias, int n_out, int m, int tile, int lane,
                                              float sum) {
  const int n = tile * kTileRows + lane;
  if (lane < kTileRows && n < n_out) {
    if constexpr (ACT == kActBf16) {
      const uint16_t* bias = reinterpret_cast<const uint16_t*>(tail.bias);
      sum = epilogue_value(tail, sum, has_bias, has_bias ? bf16_low_to_f32(bias[n]) : 0.0f);
      reinterpret_cast<uint16_t*>(tail.y)[(size_t)m * (size_t)n_out + n] = (uint16_t)pack_bf16(sum, 0.0f);
    } else {
      sum = epilogue_value(tail, sum, has_bias, has_bias ? (float)tail.bias[n] : 0.0f);
      tail.y[(size_t)m * (size_t)n_out + n] = (half_t)sum;
    }
  }
}

// A wave has computed the last unit of a tile: park the tile's 64 per-lane partial sums in the
// wave's LDS slot for that tile and start afresh.  (Nothing but LDS is touched inside the unit
// loop: a global store or bias load there would make the compiler drain the prefetched loads.)
template <int MB>
__device__ __forceinline__ void finish_tile(float (&acc)[MB], float* slot) {
#pragma unroll
  for (int m = 0; m < MB; ++m) {
    slot[m * kWave] = acc[m];
    acc[m] = 0.0f;
  }
}

// Timeline probe: what a wave's unit loop waits for.  Before a unit's arithmetic starts, the wave
// stands in an explicit wait for that unit's operands and first weight block (everything requested
// behind them -- the unit's other three blocks and the whole next unit -- may still be on its way);
// the time spent there is added up per third of the wave's units, the longest single wait is
// kept, and the moments at which the second and last third begin are recorded.
struct TimelineWaits {
  uint32_t wait[3];   // ticks of the 100 MHz clock spent waiting, per third of the wave's units
  uint32_t longest;   // the longest single wait
  uint64_t begin[2];  // when the second / last third of the units began
};

// kLoadsBehindFirstBlock: loads issued after block 0 of the unit that is about to be computed.
template <int kLoadsBehindFirstBlock>
__device__ __forceinline__ void timeline_wait(TimelineWaits& t, int u, int total) {
  static_assert(kLoadsBehindFirstBlock >= 3 && kLoadsBehindFirstBlock < 64, "the counter of outstanding loads has 6 bits");
  uint64_t a, b;
  asm volatile("s_memrealtime %0\n\ts_waitcnt vmcnt(%2)\n\ts_memrealtime %1\n\ts_waitcnt lgkmcnt(0)"
               : "=&s"(a), "=&s"(b) : "n"(kLoadsBehindFirstBlock) : "memory");
  const uint32_t d = (uint32_t)(b - a);
  const int third = u * 3 / total;
  t.wait[0] += third == 0 ? d : 0u;
  t.wait[1] += third == 1 ? d : 0u;
  t.wait[2] += third == 2 ? d : 0u;
  t.longest = d > t.longest ? d : t.longest;
  if (third >= 1 && t.begin[0] == 0) t.begin[0] = a;
  if (third >= 2 && t.begin[1] == 0) t.begin[1] = a;
}

// blockDim = (64 * split_k, tiles_per_wg).  Dynamic LDS: ceil(tiles / sequences) * tiles_per_wg *
// split_k * MB * 64 floats.
// One activation row, one group per run: ask for 6 resident waves per SIMD (at most 80 VGPRs).
// The allocation unit is 8 registers, so 81 would already cost a whole wave of occupancy.
// ACT: kActF16 or kActBf16 -- the type of activations, scales, zeros, bias and outputs (the
// pointers are typed as 16-bit storage either way).
// PROBE (measurement builds of this same kernel, see mixed_gemv.h "Measurement probes"):
// kProbeNone the product; kProbeComputeOnly loads a wave's first unit only and repeats its arithmetic
// for every further unit; kProbeLoadsOnly keeps every load and replaces the arithmetic of a unit
// by an exclusive-or over its registers -- what the access pattern alone takes; kProbeTimeline
// records timestamps and the time spent waiting for loads, per wave.
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, bool MULTI, int ACT, int PROBE = kProbeNone>
__global__ void __launch_bounds__(kWave * (MB >= 3 || ACT == kActBf16 ? kMaxWavesPerWideWorkgroup : kMaxWavesPerWorkgroup))
__attribute__((amdgpu_waves_per_eu(ACT == kActF16 && MB == 1 && GROUPS_PER_RUN == 1 ? 6 : 1)))
gemv_dpp_kernel(const uint8_t* weights, const half_t* x, const half_t* scale, const half_t* zero_add, int n_out, int k,
                uint32_t packed_steps, int workgroups, int num_groups, uint32_t packed_group, GemvTail tail) {
  extern __shared__ float partials[];
  uint64_t stamp[5] = {0, 0, 0, 0, 0};
  TimelineWaits waits{};
  int units_computed = 0;
  uint64_t cycles_at_start = 0;
  if constexpr (PROBE == kProbeTimeline) {
    stamp[0] = __builtin_amdgcn_s_memrealtime();
    cycles_at_start = __builtin_readcyclecounter();
  }
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
  // The library is built with kernel-argument preloading: the four pointers and six words in
  // front of GemvTail arrive in SGPRs with the wave (firmware without the feature runs a short
  // prologue that loads them instead).  Nothing on the way to the first weight loads of an
  // unbatched launch whose waves stay on one tile reads the tail, so those loads do not wait
  // for any scalar load at all: `tail` itself is only touched by batched launches and tile
  // walks, everything else reads the copy `late`, fetched once the first unit is requested.
  // Batched launch (gemv/kernel/mixed_gemv.h:140-149, 222-223): problems past the first fetch
  // their strides first.  A routed launch (a bit of a preloaded word says so) looks up whose
  // weights, scales, zeros and bias each problem takes; x and y stay with the problem.
  const long long batch = blockIdx.z;
  long long owner = batch;
  if ((blockIdx.z | (packed_group & kRoutedLaunch)) != 0) {  // one test on the way of an unbatched launch
    if ((packed_group & kRoutedLaunch) != 0) {
      const int entry = tail.route[batch];
      if ((unsigned)entry >= (unsigned)tail.route_extent) return;  // whole workgroup, before any barrier
      owner = entry;
    }
    p.weights += owner * tail.stride_weights;
    p.x += batch * tail.stride_x;
    p.scale += owner * tail.stride_scale;
    p.zero_add += owner * tail.stride_scale;  // only dereferenced in scale+zero mode
  }

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;  // whole workgroup leaves before any barrier

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // position along k
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);         // tile sequence within the workgroup
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  // The host's launch geometry leaves no wave without units (split_k = ceil(ksteps / steps_per_wave)).
  const WaveWork work = valu_wave_work(MULTI, wg, ty, kw, p.tiles_per_wg, MULTI ? tail.seq_base : 0,
                                       MULTI ? tail.seq_rem : 0, tiles, p.steps_per_wave, p.ksteps);
  const int tile_begin = work.tile_begin, my_tiles = work.tiles, ks_begin = work.ks_begin, units = work.units;

  GemvTail late;
  if (my_tiles <= 0) late = read_tail_here();
  if (my_tiles > 0) {
    const int total = MULTI ? my_tiles * units : units;
    const int tile_stride = p.ksteps * kUnitBytes;
    const __amdgpu_buffer_rsrc_t w_rsrc = make_rsrc(
        p.weights + ((size_t)tile_begin * (size_t)p.ksteps + (size_t)ks_begin) * (size_t)kUnitBytes,
        (MULTI ? (uint32_t)(my_tiles - 1) * (uint32_t)tile_stride : 0u) + (uint32_t)units * (uint32_t)kUnitBytes);
    __amdgpu_buffer_rsrc_t x_rsrc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) x_rsrc[m] = make_rsrc(p.x + (size_t)m * (size_t)p.k, (uint32_t)p.k * 2u);
    ScaleTables tables;
    const uint32_t table_bytes = (uint32_t)num_groups * (uint32_t)p.n_out * 2u;
    tables.scale = make_rsrc(p.scale, table_bytes);
    tables.zero = make_rsrc(p.zero_add, QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? table_bytes : 0u);
    TileWalk walk;
    WaveCursor<BITS, GROUPS_PER_RUN> cur = make_cursor<BITS, GROUPS_PER_RUN>(
        p, QOP == MGEMV_PER_COLUMN_SCALE_ONLY, ks_begin, units, lane, tile_begin * kTileRows + lane % kTileRows, walk);

    float acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m] = 0.0f;
    int pending = units;     // MULTI: units of the current tile still to compute

    // Two fragments in flight: the loads of unit u+1 are issued before unit u is computed, so
    // a wave that is waiting for its turn on the VALU still has memory requests outstanding.
    // (The first fragment is loaded ahead of the loop and reaches it through register copies,
    // which wait for its data before the second unit is requested.  A loop that loads both
    // fragments inside, without that wait, measured the same to 2 % on every shape.)
    UnitFragment<BITS, MB, GROUPS_PER_RUN> fa, fb;
    load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fa, p, w_rsrc, x_rsrc, tables, cur);
    __builtin_amdgcn_sched_barrier(0);
    late = read_tail_here();
    const int park_stride = p.tiles_per_wg * late.split_k * MB * kWave;  // floats between consecutive tiles of a sequence
    float* slot = partials + (ty * late.split_k + kw) * MB * kWave + lane;  // MULTI
    if constexpr (PROBE == kProbeTimeline) {
      __builtin_amdgcn_sched_barrier(0);
      stamp[1] = __builtin_amdgcn_s_memrealtime();      // the first unit is requested
      asm volatile("s_waitcnt vmcnt(3)" ::: "memory");   // ... and all but its last three blocks are in
      stamp[2] = __builtin_amdgcn_s_memrealtime();
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (PROBE == kProbeComputeOnly) fb = fa;  // (waits for the first unit; every later "load" re-uses it)
    const bool short_ok = (late.flags & kExactIntegerFormOnly) == 0;
    const ConvertRegs c = make_convert_regs();
    // With two or more activation rows, a wave of exactly two units runs straight-line code: the
    // second unit is requested without waiting for the first and nothing is prefetched past the
    // end (4096x4096: 4.44 / 4.74 / 5.04 us at 2 / 3 / 4 rows against 4.55 / 4.83 / 5.19 through
    // the loop).  A three-unit path lost 5 % to the loop (4096x6144, 2 rows), and in the
    // single-row kernels, which are held to 80 registers, any extra path made the loop beside it
    // 4-7 % slower, so those keep the loop for every length.
    if (total == 1) {
      compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT, PROBE>(acc, fa, c, short_ok);
      if constexpr (MULTI) finish_tile<MB>(acc, slot);
    } else if (MB >= 2 && !MULTI && total == 2) {
      advance<MULTI>(cur, walk);
      if constexpr (PROBE == kProbeComputeOnly) reuse_unit<BITS, MB, GROUPS_PER_RUN>(fb);
      else load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fb, p, w_rsrc, x_rsrc, tables, cur);
      __builtin_amdgcn_sched_barrier(0);
      compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT, PROBE>(acc, fa, c, short_ok);
      __builtin_amdgcn_sched_barrier(0);
      compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT, PROBE>(acc, fb, c, short_ok);
    } else {
      // The prefetches are unconditional: past the wave's last unit every weight offset is out
      // of the descriptor's range, the loads return zero without touching memory, and the
      // compiler can count outstanding loads exactly instead of draining them all before each use.
      // The reference's kStages = 1 main loop (gemv/threadblock/dq_mma_singlestage_finegrained.h:264-310)
      // keeps nothing in flight while it computes; its kStages = 2 loop (dq_mma_pipelined_finegrained.h:
      // 263-352) is this one.  With the single-stage flag every prefetch is waited for as soon as it is
      // issued, which gives that behaviour -- loads and arithmetic strictly one after the other -- to the
      // same code; results do not change.
      const bool single_stage = (late.flags & kSingleStage) != 0;
      int u = 0;
      do {
        advance<MULTI>(cur, walk);
        if constexpr (PROBE == kProbeComputeOnly) reuse_unit<BITS, MB, GROUPS_PER_RUN>(fb);
        else load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fb, p, w_rsrc, x_rsrc, tables, cur);
        if (single_stage) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic it overlaps
        if constexpr (PROBE == kProbeTimeline) {
          if (late.flags & kTimelineWaits) timeline_wait<kBlocksPerUnit - 1 + MB + GROUPS_PER_RUN * 2 + kBlocksPerUnit>(waits, u, total);
          __builtin_amdgcn_sched_barrier(0);
        }
        compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT, PROBE>(acc, fa, c, short_ok);
        if constexpr (MULTI) {
          if (--pending == 0) {
            finish_tile<MB>(acc, slot);
            slot += park_stride; pending = units;
          }
        }
        advance<MULTI>(cur, walk);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (PROBE == kProbeComputeOnly) reuse_unit<BITS, MB, GROUPS_PER_RUN>(fa);
        else load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fa, p, w_rsrc, x_rsrc, tables, cur);
        if (single_stage) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        if (u + 1 < total) {
          if constexpr (PROBE == kProbeTimeline) {
            if (late.flags & kTimelineWaits) timeline_wait<kBlocksPerUnit - 1 + MB + GROUPS_PER_RUN * 2 + kBlocksPerUnit>(waits, u + 1, total);
            __builtin_amdgcn_sched_barrier(0);
          }
          compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT, PROBE>(acc, fb, c, short_ok);
          if constexpr (MULTI) {
            if (--pending == 0) {
              finish_tile<MB>(acc, slot);
              slot += park_stride; pending = units;
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        u += 2;
      } while (u < total);
    }
    if constexpr (PROBE == kProbeTimeline) {
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" :: "v"(acc[0]));
      stamp[3] = __builtin_amdgcn_s_memrealtime();      // the last unit is computed
      units_computed = total;
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!MULTI) finish_tile<MB>(acc, partials + (ty * late.split_k + kw) * MB * kWave + lane_after_loop());
  }
  const int split_k = late.split_k;
  const int park_stride = p.tiles_per_wg * split_k * MB * kWave;
  const bool has_bias = late.bias != nullptr;
  late.bias += owner * late.stride_bias;
  late.y += batch * late.stride_y;

  // Split-K combine (gemv/threadblock/accumulator_combine.h:269-329): every wave has parked
  // its 64 per-lane partial sums of each tile in LDS; after ONE barrier the (tile, activation
  // row) pairs of the sequence are dealt out to its waves, each summing a pair over the waves
  // in ascending order, then over the four k slices.  A wave that has its tiles to itself
  // reads back only what it wrote and needs no barrier.
  if (split_k > 1) __syncthreads();
  const int lane_c = lane_after_loop();
  for (int item = kw; item < my_tiles * MB; item += split_k) {
    const int j = item / MB, m = item % MB;
    const float* part = partials + j * park_stride + (ty * split_k * MB + m) * kWave + lane_c;
    float sum = 0.0f;
    int w = 0;
    for (; w + 4 <= split_k; w += 4) {
      const float a0 = part[(w + 0) * MB * kWave], a1 = part[(w + 1) * MB * kWave];
      const float a2 = part[(w + 2) * MB * kWave], a3 = part[(w + 3) * MB * kWave];
      sum = (((sum + a0) + a1) + a2) + a3;
    }
    for (; w < split_k; ++w) sum += part[w * MB * kWave];
    store_outputs<ACT>(late, has_bias, p.n_out, m, tile_begin + j, lane_c, reduce_k_slices(sum));
  }
  if constexpr (PROBE == kProbeTimeline) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // the outputs are on their way
    stamp[4] = __builtin_amdgcn_s_memrealtime();
    if (late.trace != nullptr && lane_c == 0) {
      unsigned long long* out =
          late.trace + ((size_t)blockIdx.x * (blockDim.x * blockDim.y / kWave) + ty * split_k + kw) * kTimelineWordsPerWave;
#pragma unroll
      for (int i = 0; i < 5; ++i) out[i] = stamp[i];
      out[5] = waits.wait[0]; out[6] = waits.wait[1]; out[7] = waits.wait[2];
      out[8] = waits.longest;
      out[9] = waits.begin[0]; out[10] = waits.begin[1];
      out[11] = (unsigned long long)units_computed;
      out[12] = cycles_at_start;
      out[13] = __builtin_readcyclecounter();
    }
  }
}

// Picks the instantiation for the run-time arguments.
template <int BITS, int QOP, int MB, int GPR, bool MULTI, int ACT>
hipError_t launch_gemv_kernel_m(const GemvLaunch& g) {
  return launch(gemv_dpp_kernel<BITS, QOP, MB, GPR, MULTI, ACT>, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale,
                g.zero_add, g.n_out, g.k, pack_steps(num_ksteps(g.k, BITS), g.plan.steps_per_wave), g.plan.workgroups,
                g.tail.num_groups, pack_group(g.group_size, g.plan.tiles_per_wg, g.tail.route != nullptr), g.tail);
}

template <int BITS, int QOP, int MB, int GPR, int ACT>
hipError_t launch_gemv_kernel(const GemvLaunch& g) {
  return g.plan.tiles_in_sequence > 1 ? launch_gemv_kernel_m<BITS, QOP, MB, GPR, true, ACT>(g)
                                      : launch_gemv_kernel_m<BITS, QOP, MB, GPR, false, ACT>(g);
}

template <int BITS, int QOP, int MB, int ACT>
hipError_t launch_gemv_gpr(const GemvLaunch& g, int gpr) {
  if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
    return launch_gemv_kernel<BITS, QOP, MB, 1, ACT>(g);
  } else {
    switch (gpr) {
      case 1: return launch_gemv_kernel<BITS, QOP, MB, 1, ACT>(g);
      case 2: return launch_gemv_kernel<BITS, QOP, MB, 2, ACT>(g);
      default: return launch_gemv_kernel<BITS, QOP, MB, 4, ACT>(g);
    }
  }
}

template <int BITS, int QOP, int ACT>
hipError_t launch_gemv_mb(const GemvLaunch& g, int mb, int gpr) {
  switch (mb) {
    case 1: return launch_gemv_gpr<BITS, QOP, 1, ACT>(g, gpr);
    case 2: return launch_gemv_gpr<BITS, QOP, 2, ACT>(g, gpr);
    case 3: return launch_gemv_gpr<BITS, QOP, 3, ACT>(g, gpr);
    default: return launch_gemv_gpr<BITS, QOP, 4, ACT>(g, gpr);
  }
}

template <int ACT>
hipError_t launch_gemv_act(const GemvLaunch& g, int bits, int qop, int mb, int gpr) {
  if (bits == 4) {
    switch (qop) {
      case 1: return launch_gemv_mb<4, 1, ACT>(g, mb, gpr);
      case 2: return launch_gemv_mb<4, 2, ACT>(g, mb, gpr);
      default: return launch_gemv_mb<4, 3, ACT>(g, mb, gpr);
    }
  }
  switch (qop) {
    case 1: return launch_gemv_mb<8, 1, ACT>(g, mb, gpr);
    case 2: return launch_gemv_mb<8, 2, ACT>(g, mb, gpr);
    default: return launch_gemv_mb<8, 3, ACT>(g, mb, gpr);
  }
}

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_GEMV_DPP_KERNEL_H_
