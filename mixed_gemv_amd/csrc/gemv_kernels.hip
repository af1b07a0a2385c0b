// GEMV and dequantise kernels for gfx950 (MI355X), wave64, plus their C-ABI launchers.
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
#include <hip/hip_runtime.h>

#include <atomic>
#include <map>
#include <mutex>
#include <tuple>

#include "device_math.h"
#include "mixed_gemv.h"
#include "tile_layout.h"

namespace mgemv {

constexpr int kWave = 64;
constexpr int kMaxWavesPerWorkgroup = 16;
constexpr int kMaxWavesPerWideWorkgroup = 8;  // VALU kernel with 3-4 activation rows: 256 VGPRs per wave
constexpr int kMaxWavesPerMfmaWorkgroup = 8;  // leaves each wave of the matrix-core kernel 256 VGPRs
constexpr int kNumXcd = 8;
constexpr int kNumCus = 256;
constexpr int kMaxValuBatch = 4;  // activation rows handled per launch by the VALU kernel
constexpr int kExactIntegerFormOnly = 1;  // GemvTail::flags: never take the short int4 dequantiser

// Kernel arguments.  The first ten (four pointers and six 32-bit words, 14 dwords) are what a
// wave needs to address its first loads, and they are preloaded into SGPRs (build flag
// -amdgpu-kernarg-preload-count=14); everything else sits in GemvTail.
struct GemvTail {
  const half_t* bias;
  half_t* y;
  int split_k;         // waves of a workgroup that share one tile (blockDim.x / 64)
  int m_batch;         // activation rows (matrix-core kernel)
  int num_groups;      // k / group_size (1 in per-column mode): extent of the scale / zero tables
  int flags;           // kExactIntegerFormOnly or 0
  int seq_base;        // VALU kernel: tiles / sequences ...
  int seq_rem;         // ... and tiles % sequences (the first seq_rem sequences get one tile more)
  long long stride_weights, stride_x, stride_scale, stride_bias, stride_y;  // per batch problem
};

// Scalar view of one problem inside a kernel.
struct Problem {
  const uint8_t* weights;
  const half_t* x;
  const half_t* scale;
  const half_t* zero_add;
  int n_out;
  int k;
  int ksteps;          // ceil(k / kStepK)
  int steps_per_wave;  // units per wave
  int workgroups;      // logical workgroups = ceil(tiles / tiles_per_wg)
  int wgs_per_xcd;     // ceil(workgroups / 8); gridDim.x = 8 * wgs_per_xcd
  int group_size;
  int tiles_per_wg;    // blockDim.y
};

constexpr uint32_t pack_steps(int ksteps, int steps_per_wave) { return (uint32_t)ksteps | ((uint32_t)steps_per_wave << 16); }
constexpr uint32_t pack_group(int group_size, int tiles_per_wg) { return (uint32_t)group_size | ((uint32_t)tiles_per_wg << 24); }

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Neighbouring tiles read
// neighbouring 32-byte pieces of the same scale/zero cache lines, so give each XCD (and its
// private L2) a contiguous range of tiles instead of every eighth one.
__device__ __forceinline__ int logical_workgroup(const Problem& p) {
  const int xcd = blockIdx.x % kNumXcd;
  const int slot = blockIdx.x / kNumXcd;
  return xcd * p.wgs_per_xcd + slot;
}

// Group index of reduction position k_index (host/mixed_gemv.h:88), clamped to the last
// group for the padded positions past k.
__device__ __forceinline__ int group_of(const Problem& p, int k_index) {
  k_index = k_index < p.k ? k_index : p.k - 1;
  const bool pow2 = (p.group_size & (p.group_size - 1)) == 0;
  return pow2 ? (k_index >> __builtin_ctz((unsigned)p.group_size)) : (k_index / p.group_size);
}

// Everything one lane needs for one unit.  Scale and additive zero are kept as packed
// (s, s) / (z, z) pairs in 32-bit registers.
template <int BITS, int MB, int GROUPS_PER_RUN>
struct UnitFragment {
  u32x4 w[kBlocksPerUnit];                // 4 chunks of this lane's row
  uint32_t x[MB][BITS == 4 ? 4 : 2];      // this lane's piece of the activation run
  uint32_t s[GROUPS_PER_RUN];             // fp16 scale of each group of the run (low 16 bits; the rest is unspecified)
  uint32_t z[GROUPS_PER_RUN];             // fp16 additive zero (low 16 bits; the rest is unspecified)
};

// 16-bit buffer load into the low half of a 32-bit register.  The upper half is left
// unspecified on purpose: zero-extending it would be a VALU instruction on the loaded value,
// and the compiler places that instruction -- and the wait for the data -- next to the load,
// in front of the loads that should be issued behind it.
__device__ __forceinline__ uint32_t load_b16_low(__amdgpu_buffer_rsrc_t rsrc, int voffset) {
  const uint16_t bits = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, voffset, 0, kCacheDefault);
  half2_t v;  // element 1 deliberately not set
  v[0] = __builtin_bit_cast(half_t, bits);
  return as_u32(v);
}
__device__ __forceinline__ uint32_t load_half_bits(const half_t* p) {
  return (uint32_t)*reinterpret_cast<const uint16_t*>(p);
}
__device__ __forceinline__ half2_t splat_low(uint32_t bits) {
  const half_t h = __builtin_bit_cast(half_t, (uint16_t)bits);
  return half2_t{h, h};
}

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

struct ScaleTables {
  __amdgpu_buffer_rsrc_t scale, zero;
};

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

// True when the scale of every lane of the wave (all groups of the unit) permits the short
// (fp16, int4) resp. fused (bf16) dequantiser; wave-uniform, so the choice costs one scalar
// branch per unit.
template <int ACT, typename Bits, int GROUPS_PER_RUN>
__device__ __forceinline__ bool wave_scales_permit_short_form(const Bits (&scale_bits)[GROUPS_PER_RUN]) {
  bool ok = true;
#pragma unroll
  for (int gi = 0; gi < GROUPS_PER_RUN; ++gi)
    ok = ok && (ACT == kActBf16 ? fused_form_ok_bf16(scale_bits[gi]) : short_form_ok(scale_bits[gi]));
  return __builtin_amdgcn_ballot_w64(!ok) == 0;
}

// short_allowed: wave-uniform.
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, int ACT = kActF16>
__device__ __forceinline__ void compute_unit(float (&acc)[MB], const UnitFragment<BITS, MB, GROUPS_PER_RUN>& f,
                                             const ConvertRegs& c, bool short_allowed) {
  if constexpr (BITS == 4 || ACT == kActBf16) {
    if (short_allowed && wave_scales_permit_short_form<ACT>(f.s)) {
      compute_unit_form<BITS, QOP, MB, GROUPS_PER_RUN, true, ACT>(acc, f, c);
      return;
    }
  }
  compute_unit_form<BITS, QOP, MB, GROUPS_PER_RUN, false, ACT>(acc, f, c);
}

// Sum over the four k slices of a wave: lanes l, l+16, l+32, l+48 hold the same row.
// The result is valid in lanes 0..15.
__device__ __forceinline__ float reduce_k_slices(float v) {
  v += __shfl_down(v, 32);
  v += __shfl_down(v, 16);
  return v;
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
      if (has_bias) sum += bf16_low_to_f32(bias[n]);
      reinterpret_cast<uint16_t*>(tail.y)[(size_t)m * (size_t)n_out + n] = (uint16_t)pack_bf16(sum, 0.0f);
    } else {
      if (has_bias) sum += (float)tail.bias[n];
      tail.y[(size_t)m * (size_t)n_out + n] = (half_t)sum;
    }
  }
}

// The lane number, recomputed.  Used behind the unit loop so that the value computed in front
// of it need not stay in a register (or be spilled) across the loop.
__device__ __forceinline__ int lane_after_loop() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
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

// blockDim = (64 * split_k, tiles_per_wg).  Dynamic LDS: ceil(tiles / sequences) * tiles_per_wg *
// split_k * MB * 64 floats.
// One activation row, one group per run: ask for 6 resident waves per SIMD (at most 80 VGPRs).
// The allocation unit is 8 registers, so 81 would already cost a whole wave of occupancy.
// ACT: kActF16 or kActBf16 -- the type of activations, scales, zeros, bias and outputs (the
// pointers are typed as 16-bit storage either way).
template <int BITS, int QOP, int MB, int GROUPS_PER_RUN, bool MULTI, int ACT>
__global__ void __launch_bounds__(kWave * (MB >= 3 || ACT == kActBf16 ? kMaxWavesPerWideWorkgroup : kMaxWavesPerWorkgroup))
__attribute__((amdgpu_waves_per_eu(ACT == kActF16 && MB == 1 && GROUPS_PER_RUN == 1 ? 6 : 1)))
gemv_dpp_kernel(const uint8_t* weights, const half_t* x, const half_t* scale, const half_t* zero_add, int n_out, int k,
                uint32_t packed_steps, int workgroups, int num_groups, uint32_t packed_group, GemvTail tail) {
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
  p.wgs_per_xcd = (workgroups + kNumXcd - 1) / kNumXcd;
  p.group_size = (int)(packed_group & 0xffffffu);
  p.tiles_per_wg = (int)(packed_group >> 24);
  // The library is built with kernel-argument preloading: the four pointers and six words in
  // front of GemvTail arrive in SGPRs with the wave (firmware without the feature runs a short
  // prologue that loads them instead).  Nothing on the way to the first weight loads of an
  // unbatched launch reads the tail, so those loads do not wait for any scalar load at all.
  // Batched launch (gemv/kernel/mixed_gemv.h:140-149, 222-223): problems past the first fetch
  // their strides first.
  const long long batch = blockIdx.z;
  if (batch != 0) {
    p.weights += batch * tail.stride_weights;
    p.x += batch * tail.stride_x;
    p.scale += batch * tail.stride_scale;
    p.zero_add += batch * tail.stride_scale;  // only dereferenced in scale+zero mode
  }
  const bool has_bias = tail.bias != nullptr;
  tail.bias += batch * tail.stride_bias;
  tail.y += batch * tail.stride_y;

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;  // whole workgroup leaves before any barrier

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);  // position along k
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);         // tile sequence within the workgroup
  const int split_k = tail.split_k;
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  // The tiles are dealt out evenly, in contiguous runs, to the (workgroups x tiles_per_wg) tile
  // sequences of the launch; the split_k waves of a sequence walk its tiles together, each on
  // its own part of k.
  const int seq = wg * p.tiles_per_wg + ty;
  const int tile_begin = MULTI ? seq * tail.seq_base + min(seq, tail.seq_rem) : seq;
  const int my_tiles = MULTI ? tail.seq_base + (seq < tail.seq_rem ? 1 : 0) : (seq < tiles ? 1 : 0);

  // The host's launch geometry leaves no wave without units (split_k = ceil(ksteps / steps_per_wave)).
  const int ks_begin = kw * p.steps_per_wave;
  const int units = min(ks_begin + p.steps_per_wave, p.ksteps) - ks_begin;
  const int park_stride = p.tiles_per_wg * split_k * MB * kWave;  // floats between consecutive tiles of a sequence

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
    float* slot = partials + (ty * split_k + kw) * MB * kWave + lane;  // MULTI

    // Two fragments in flight: the loads of unit u+1 are issued before unit u is computed, so
    // a wave that is waiting for its turn on the VALU still has memory requests outstanding.
    // (The first fragment is loaded ahead of the loop and reaches it through register copies,
    // which wait for its data before the second unit is requested.  A loop that loads both
    // fragments inside, without that wait, measured the same to 2 % on every shape.)
    UnitFragment<BITS, MB, GROUPS_PER_RUN> fa, fb;
    load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fa, p, w_rsrc, x_rsrc, tables, cur);
    const bool short_ok = (tail.flags & kExactIntegerFormOnly) == 0;
    const ConvertRegs c = make_convert_regs();
    if (total == 1) {
      compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT>(acc, fa, c, short_ok);
      if constexpr (MULTI) finish_tile<MB>(acc, slot);
    } else {
      // The prefetches are unconditional: past the wave's last unit every weight offset is out
      // of the descriptor's range, the loads return zero without touching memory, and the
      // compiler can count outstanding loads exactly instead of draining them all before each use.
      int u = 0;
      do {
        advance<MULTI>(cur, walk);
        load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fb, p, w_rsrc, x_rsrc, tables, cur);
        __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic it overlaps
        compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT>(acc, fa, c, short_ok);
        if constexpr (MULTI) {
          if (--pending == 0) {
            finish_tile<MB>(acc, slot);
            slot += park_stride; pending = units;
          }
        }
        advance<MULTI>(cur, walk);
        __builtin_amdgcn_sched_barrier(0);
        load_unit<BITS, QOP, MB, GROUPS_PER_RUN>(fa, p, w_rsrc, x_rsrc, tables, cur);
        __builtin_amdgcn_sched_barrier(0);
        if (u + 1 < total) {
          compute_unit<BITS, QOP, MB, GROUPS_PER_RUN, ACT>(acc, fb, c, short_ok);
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
    if constexpr (!MULTI) finish_tile<MB>(acc, partials + (ty * split_k + kw) * MB * kWave + lane_after_loop());
  }

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
    store_outputs<ACT>(tail, has_bias, p.n_out, m, tile_begin + j, lane_c, reduce_k_slices(sum));
  }
}

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
    // Batch rows past m_batch and reduction positions past k fall outside the descriptor and
    // read as zero (k is a multiple of the chunk, so a block is wholly inside or outside).
    const uint32_t off = k_block < p.k ? (uint32_t)(m * p.k + k_block) * 2u : 0xfffffff0u;
#pragma unroll
    for (int j = 0; j < kFrags; ++j) f.x[i][j] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)off, j * 16, kCacheDefault);
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
  p.tiles_per_wg = (int)(packed_group >> 24);
  asm volatile("" ::"s"(weights), "s"(x), "s"(scale), "s"(zero_add), "s"(n_out), "s"(k), "s"(packed_steps),
               "s"(workgroups), "s"(wgs_per_xcd), "s"(packed_group), "s"(tail.bias), "s"(tail.y), "s"(tail.split_k),
               "s"(tail.m_batch), "s"(tail.num_groups), "s"(tail.flags), "s"(tail.stride_weights), "s"(tail.stride_x), "s"(tail.stride_scale),
               "s"(tail.stride_bias), "s"(tail.stride_y));
  const long long batch = blockIdx.z;
  p.weights += batch * tail.stride_weights;
  p.x += batch * tail.stride_x;
  p.scale += batch * tail.stride_scale;
  p.zero_add += batch * tail.stride_scale;
  const bool has_bias = tail.bias != nullptr;
  tail.bias += batch * tail.stride_bias;
  tail.y += batch * tail.stride_y;
  const int m_batch = tail.m_batch;

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int tile0 = (wg * p.tiles_per_wg + ty) * T;
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  int row[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const int r = (tile0 + t) * kTileRows + lane % kTileRows;
    row[t] = r < p.n_out ? r : p.n_out - 1;
  }

  f32x4 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const int ks_begin = kw * p.steps_per_wave;
  const int ks_end = min(ks_begin + p.steps_per_wave, p.ksteps);
  if (tile0 < tiles && ks_begin < ks_end) {
    const int units = ks_end - ks_begin;
    const int my_tiles = min(T, tiles - tile0);
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
            float r = sum[v];
            if (has_bias) r += (float)tail.bias[n];
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
          float r = acc[t][v];
          if (has_bias) r += (float)tail.bias[n];
          tail.y[(size_t)m * (size_t)p.n_out + n] = (half_t)r;
        }
      }
    }
  }
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
                                             int kstep, int lane, int first_row, int row_step) {
  using G = Geometry<BITS>;
  const int k0 = kstep * G::kStepK + lane * (XStage<BITS>::kLaneBytes / 2);
#pragma unroll
  for (int j = 0; j < ROUNDS; ++j) {
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
                                            int row_step) {
#pragma unroll
  for (int j = 0; j < ROUNDS; ++j) {
    uint8_t* dst = stage + (first_row + j * row_step) * XStage<BITS>::kRowStride + lane * XStage<BITS>::kLaneBytes;
    if constexpr (BITS == 4) {
      *reinterpret_cast<u32x4*>(dst) = u32x4{r.v[j][0], r.v[j][1], r.v[j][2], r.v[j][3]};
    } else {
      *reinterpret_cast<u32x2*>(dst) = u32x2{r.v[j][0], r.v[j][1]};
    }
  }
}

// blockDim = (64 * split_k, tiles_per_wg), at most 8 waves.  Dynamic LDS: split_k * 2 stages of
// (ROUNDS * tiles_per_wg) rows x kRowStride bytes, then tiles_per_wg * split_k * 256 floats for
// the split-K combine.
template <int BITS, int QOP, int GROUPS_PER_RUN, int ROUNDS, int ACT>
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
  p.tiles_per_wg = (int)(packed_group >> 24);
  const long long batch = blockIdx.z;
  if (batch != 0) {
    p.weights += batch * tail.stride_weights;
    p.x += batch * tail.stride_x;
    p.scale += batch * tail.stride_scale;
    p.zero_add += batch * tail.stride_scale;
  }
  const bool has_bias = tail.bias != nullptr;
  tail.bias += batch * tail.stride_bias;
  tail.y += batch * tail.stride_y;
  const int m_batch = tail.m_batch;

  const int wg = logical_workgroup(p);
  if (wg >= p.workgroups) return;  // whole workgroup leaves before any barrier

  const int lane = threadIdx.x % kWave;
  const int kw = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int ty = __builtin_amdgcn_readfirstlane(threadIdx.y);
  const int split_k = tail.split_k;
  const int tiles = (p.n_out + kTileRows - 1) / kTileRows;
  const int tile_raw = wg * p.tiles_per_wg + ty;
  const int tile = tile_raw < tiles ? tile_raw : tiles - 1;  // a wave without a tile still stages rows and meets the barriers
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
  const int ks_begin = kw * steps;
  const int units = min(ks_begin + steps, p.ksteps) - ks_begin;  // >= 1 by the host's geometry
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
  int u = 0;
  do {
    // even step: weights in wa, stage 0
    park_x_rows<BITS, ROUNDS>(xr, my_stages, lane, ty, p.tiles_per_wg);
    __syncthreads();
    fetch_x_rows<BITS, ROUNDS>(xr, p, x_rsrc, ks_begin + u + 1, lane, ty, p.tiles_per_wg);
    load_weights_lds_mfma<BITS, QOP, GROUPS_PER_RUN>(wb, p, w_rsrc, tables, u + 1, ks_begin + u + 1, lane, row);
    __builtin_amdgcn_sched_barrier(0);
    if (u < units) {
      const LdsActivations<BITS> xa{my_stages + operand_offset};
      compute_unit_mfma<BITS, QOP, GROUPS_PER_RUN, ACT>(acc, wa, xa, c, col_scale, short_ok);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (u + 1 < steps) {
      // odd step: weights in wb, stage 1
      park_x_rows<BITS, ROUNDS>(xr, my_stages + stage_bytes, lane, ty, p.tiles_per_wg);
      __syncthreads();
      fetch_x_rows<BITS, ROUNDS>(xr, p, x_rsrc, ks_begin + u + 2, lane, ty, p.tiles_per_wg);
      load_weights_lds_mfma<BITS, QOP, GROUPS_PER_RUN>(wa, p, w_rsrc, tables, u + 2, ks_begin + u + 2, lane, row);
      __builtin_amdgcn_sched_barrier(0);
      if (u + 1 < units) {
        const LdsActivations<BITS> xa{my_stages + stage_bytes + operand_offset};
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
        float r = sum[v];
        if constexpr (ACT == kActBf16) {
          if (has_bias) r += bf16_low_to_f32(reinterpret_cast<const uint16_t*>(tail.bias)[n]);
          reinterpret_cast<uint16_t*>(tail.y)[(size_t)m * (size_t)p.n_out + n] = (uint16_t)pack_bf16(r, 0.0f);
        } else {
          if (has_bias) r += (float)tail.bias[n];
          tail.y[(size_t)m * (size_t)p.n_out + n] = (half_t)r;
        }
      }
    }
  }
}

struct DequantParams {
  const uint8_t* weights;
  const half_t* scale;
  const half_t* zero_add;
  int n_out, k, group_size, tiles, ksteps, flags;
};

// One wave per unit; writes the dequantised weights of its 16 rows x kStepK columns with the
// same converters, and the same wave-uniform choice between them, as the GEMV kernels.
template <int BITS, int QOP, int ACT>
__global__ void __launch_bounds__(256) dequantize_kernel(const DequantParams p, half_t* __restrict__ out) {
  using G = Geometry<BITS>;
  constexpr bool kHasZero = QOP == MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  const int lane = threadIdx.x % kWave;
  const long long unit = (long long)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (unit >= (long long)p.tiles * p.ksteps) return;  // whole waves only
  const int tile = (int)(unit / p.ksteps), kstep = (int)(unit % p.ksteps);
  const int row = tile * kTileRows + lane % kTileRows;
  const int k_run = kstep * G::kStepK + (lane / kTileRows) * G::kRunK;
  const ConvertRegs c = make_convert_regs();
  const uint8_t* base = p.weights + (size_t)unit * kUnitBytes + (size_t)lane * kChunkBytes;
  const int row_c = row < p.n_out ? row : p.n_out - 1;
  uint32_t s_bits[kBlocksPerUnit];
  half_t s[kBlocksPerUnit], z[kBlocksPerUnit];
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) {
    z[i] = (half_t)0.0f;
    if constexpr (QOP == MGEMV_PER_COLUMN_SCALE_ONLY) {
      s[i] = p.scale[row_c];
    } else {
      Problem geo{};
      geo.k = p.k;
      geo.group_size = p.group_size;
      const int idx = group_of(geo, k_run + i * G::kChunkK) * p.n_out + row_c;
      s[i] = p.scale[idx];
      if constexpr (kHasZero) z[i] = p.zero_add[idx];
    }
    s_bits[i] = (uint32_t)__builtin_bit_cast(uint16_t, s[i]);
  }
  const bool take_short = (BITS == 4 || ACT == kActBf16) && (p.flags & kExactIntegerFormOnly) == 0 &&
                          wave_scales_permit_short_form<ACT>(s_bits);
#pragma unroll
  for (int i = 0; i < kBlocksPerUnit; ++i) {
    const int k0 = k_run + i * G::kChunkK;
    const u32x4 w = *reinterpret_cast<const u32x4*>(base + i * kBlockBytes);
    const half2_t s2 = splat(s[i]), z2 = splat(z[i]);
    if (row >= p.n_out || k0 >= p.k) continue;
    half_t* dst = out + (size_t)row * (size_t)p.k + k0;
    if constexpr (ACT == kActBf16) {
      constexpr int kPairs = BITS == 4 ? 4 : 2;
      const uint32_t z_bits = (uint32_t)__builtin_bit_cast(uint16_t, z[i]);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t d[kPairs];
        if (take_short) {
          const Bf16Scale bs = make_bf16_scale<BITS, true>(s_bits[i], z_bits);
          if constexpr (BITS == 4) dequant_int4_word_bf16<kHasZero, true>(w[j], c, bs, d);
          else dequant_int8_word_bf16<kHasZero, true>(w[j], bs, d);
        } else {
          const Bf16Scale bs = make_bf16_scale<BITS, false>(s_bits[i], z_bits);
          if constexpr (BITS == 4) dequant_int4_word_bf16<kHasZero, false>(w[j], c, bs, d);
          else dequant_int8_word_bf16<kHasZero, false>(w[j], bs, d);
        }
#pragma unroll
        for (int h = 0; h < kPairs; ++h) *reinterpret_cast<uint32_t*>(dst + j * 2 * kPairs + h * 2) = d[h];
      }
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (BITS == 4) {
        half2_t d[4];
        if (take_short) {
          dequant_int4_word_short<kHasZero>(w[j], c, make_short_form_scale(s2), z2, d);
        } else {
          half2_t q[4];
          convert_int4_word(w[j], c, q);
#pragma unroll
          for (int h = 0; h < 4; ++h) d[h] = dequant_pair<kHasZero>(q[h], s2, z2);
        }
#pragma unroll
        for (int h = 0; h < 4; ++h) *reinterpret_cast<half2_t*>(dst + j * 8 + h * 2) = d[h];
      } else {
        half2_t q[2];
        convert_int8_word(w[j], c, q);
#pragma unroll
        for (int h = 0; h < 2; ++h)
          *reinterpret_cast<half2_t*>(dst + j * 4 + h * 2) = dequant_pair<kHasZero>(q[h], s2, z2);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Host side: argument checks, launch geometry, dispatch
// ---------------------------------------------------------------------------------------------

std::atomic<int> g_override_split_k{0};
std::atomic<int> g_override_tiles_per_wg{0};
std::atomic<int> g_override_tiles_per_wave{0};
std::atomic<int> g_override_workgroups{0};
std::atomic<int> g_matrix_core_min_batch{0};  // m_batch from which the matrix-core kernels are used; 0 = built-in rule
std::atomic<int> g_dequant_flags{0};          // kExactIntegerFormOnly or 0
std::atomic<int> g_matrix_core_variant{MGEMV_MATRIX_CORE_AUTO};

// What steers plan_launch besides the shape: zeros mean "built-in rule".
struct PlanKnobs {
  int split_k = 0, tiles_per_wg = 0, tiles_per_wave = 0, workgroups = 0;
  int matrix_core_min_batch = 0;
  int matrix_core_variant = MGEMV_MATRIX_CORE_AUTO;
  bool wide_waves = false;  // the kernel is one of those compiled for at most 8 waves per workgroup
};

// Tuned plans by problem: (n_out, k, weight bits, group size or 0 for any, m_batch) -> knobs.
using PlanKey = std::tuple<int, int, int, int, int>;
std::mutex g_tuned_mutex;
std::map<PlanKey, PlanKnobs> g_tuned_plans;
std::atomic<int> g_tuned_count{0};  // lets the launch path skip the lock while the table is empty

// Process-wide overrides win over the table (they are what a tuner sweeps); then an entry for
// exactly this group size, then one for any group size, then the built-in rules.
PlanKnobs knobs_for(int n_out, int k, int bits, int group_size, int m_batch) {
  PlanKnobs kn;
  kn.split_k = g_override_split_k.load();
  kn.tiles_per_wg = g_override_tiles_per_wg.load();
  kn.tiles_per_wave = g_override_tiles_per_wave.load();
  kn.workgroups = g_override_workgroups.load();
  kn.matrix_core_min_batch = g_matrix_core_min_batch.load();
  kn.matrix_core_variant = g_matrix_core_variant.load();
  const bool overridden = kn.split_k || kn.tiles_per_wg || kn.tiles_per_wave || kn.workgroups ||
                          kn.matrix_core_min_batch || kn.matrix_core_variant != MGEMV_MATRIX_CORE_AUTO;
  if (overridden || g_tuned_count.load() == 0) return kn;
  std::lock_guard<std::mutex> lock(g_tuned_mutex);
  auto it = g_tuned_plans.find(PlanKey{n_out, k, bits, group_size, m_batch});
  if (it == g_tuned_plans.end() && group_size != 0) it = g_tuned_plans.find(PlanKey{n_out, k, bits, 0, m_batch});
  return it == g_tuned_plans.end() ? kn : it->second;
}

// Built-in rule, measured: up to 4 activation rows the VALU kernel wins on matrices of up to
// ~8k units (8192x8192: 12.0 us at 4 rows against 11.8 us, 10.9 against 11.9 at 3); on larger ones
// the LDS-staged matrix-core kernel already wins at 3 rows (28672x8192: 26.9 us against 31.9 us).
// From 5 rows the VALU kernel would need a second launch.
inline bool use_matrix_cores(int m_batch, long long units, int forced) {
  if (forced > 0) return m_batch >= forced;
  return m_batch >= 5 || (m_batch >= 3 && units >= 16384);
}

struct LaunchPlan {
  int split_k, tiles_per_wg, steps_per_wave, workgroups, wgs_per_xcd, threads;
  int tiles_per_wave;  // 1 on the VALU path; 1, 2 or 4 on the matrix-core path
  int tiles_in_sequence;  // VALU path: most tiles any wave walks one after the other
  int staged_rows;        // LDS-staged matrix-core kernel: 8 or 16 activation rows per stage; 0 = other kernels
  bool matrix_core;       // one of the two matrix-core kernels (else the VALU kernel)
};

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

LaunchPlan plan_launch(int n_out, int k, int bits, int m_batch, const PlanKnobs& knobs) {
  const int tiles = num_tiles(n_out), ksteps = num_ksteps(k, bits);
  const int ov_sk = knobs.split_k, ov_tw = knobs.tiles_per_wg;
  const int ov_t = knobs.tiles_per_wave;
  const bool mc = use_matrix_cores(m_batch, (long long)tiles * ksteps, knobs.matrix_core_min_batch);
  // Up to 256 tiles and 8 rows the register-operand kernel with one tile per wave wins: a lane of
  // a row past m_batch loads nothing there, and no barrier ties the waves of a workgroup together
  // (1024x2048, 5 rows: 3.6 us against 4.6 us; 4096x11008: 10.2 against 13.3; 4096x4096, 8 rows: 6.3
  // against 6.7; at 16 rows, or from 384 tiles, the LDS-staged kernel is level or ahead).
  const bool small_problem = knobs.matrix_core_variant == MGEMV_MATRIX_CORE_AUTO && tiles <= 256 && m_batch <= 8;
  if (mc && knobs.matrix_core_variant != MGEMV_MATRIX_CORE_REGISTER_OPERAND && !small_problem && tiles >= 2) {
    // LDS-staged kernel: two tiles per workgroup share the activation stage; k split as long as
    // the launch stays within 2048 waves (measured: 8192x8192 best at 4 k-split waves, 11008x4096
    // at 2 -- 11.4 us against 14.2 us at 4 with 16 rows, whose 133 KB of stages would leave one
    // workgroup per compute unit for 344 workgroups --, 28672x8192 at 1).
    LaunchPlan lp{};
    lp.matrix_core = true;
    lp.tiles_per_wg = 2;
    lp.staged_rows = m_batch <= 8 ? 8 : 16;
    lp.workgroups = ceil_div(tiles, lp.tiles_per_wg);
    int split = 1;
    while (split < 4 && split * 2 <= ksteps && (long long)lp.workgroups * lp.tiles_per_wg * split * 2 <= 2048) split *= 2;
    if (ov_sk > 0) split = ov_sk > 4 ? 4 : ov_sk;
    if (split > ksteps) split = ksteps;
    lp.steps_per_wave = ceil_div(ksteps, split);
    lp.split_k = ceil_div(ksteps, lp.steps_per_wave);
    lp.wgs_per_xcd = ceil_div(lp.workgroups, kNumXcd);
    lp.threads = kWave * lp.split_k * lp.tiles_per_wg;
    lp.tiles_per_wave = 1;
    lp.tiles_in_sequence = 1;
    return lp;
  }
  // Matrix-core path: a wave that works on T tiles fetches the activation operands of a k step
  // once for all of them.  Measured on 8192 x 8192 (512 tiles): T = 2 is 1.5-1.8x faster than
  // T = 1 at 8-16 activation rows; T = 4 leaves too few waves to cover the load latency.
  int tiles_per_wave = 1;
  if (mc) {
    tiles_per_wave = tiles >= 256 && !small_problem ? 2 : 1;
    if (ov_t == 1 || ov_t == 2 || ov_t == 4) tiles_per_wave = ov_t;
  }
  const int groups = ceil_div(tiles, tiles_per_wave);
  // Shapes that the exact-fit rule below does not take (measured on MI355X; one tile group per
  // workgroup is best throughout):
  //  * about one workgroup per compute unit or fewer (<= 384 tile groups): few, longer waves --
  //    4 k-split waves, each pipelining two or more units -- beat more, shorter ones
  //    (4096x4096: 4.08 us at 4 waves against 4.33 us at 8);
  //  * more tile groups than that: split as far as the units allow while the launch stays under
  //    ~8k waves, and fall back to two units per wave when that still leaves >= 4096 waves.
  const int max_waves = mc ? kMaxWavesPerMfmaWorkgroup
                        : m_batch >= 3 || knobs.wide_waves ? kMaxWavesPerWideWorkgroup
                                                  : kMaxWavesPerWorkgroup;
  int split_k;
  if (groups <= 384) {
    split_k = ksteps < 4 ? ksteps : 4;
    if (mc) split_k = ksteps < max_waves ? ksteps : max_waves;  // not pipelined: wants waves
  } else {
    constexpr int kWaveBudget = 8192;
    split_k = ksteps < max_waves ? ksteps : max_waves;
    while (split_k > 1 && (long long)groups * split_k > kWaveBudget) split_k = (split_k + 1) / 2;
    if (!mc && split_k > 1 && ceil_div(ksteps, split_k) < 2 &&
        (long long)groups * ((split_k + 1) / 2) >= 4096)
      split_k = (split_k + 1) / 2;
  }
  int tiles_per_wg = 1;
  int workgroup_cap = 0;
  if (!mc && tiles >= kNumCus && ksteps >= 4) {
    // "Exact fit": when the tiles divide (nearly) evenly over the compute units, one workgroup
    // of four waves per compute unit -- one wave per SIMD, all with the same amount of work --
    // beats any over-subscribed launch (8192x8192: 8.7 us against 10.2 us; 28672x8192: 2 %).
    // The four waves are tw tile sequences x 4/tw k-split waves, tw as large as still fits evenly.
    for (int tw = 4; tw >= 1; tw /= 2) {
      const int sequences = kNumCus * tw;
      if ((long long)ceil_div(tiles, sequences) * sequences * 100 <= (long long)tiles * 103) {
        tiles_per_wg = tw;
        split_k = 4 / tw;
        workgroup_cap = kNumCus;
        break;
      }
    }
  }
  if (ov_sk > 0) split_k = ov_sk;
  if (ov_tw > 0) tiles_per_wg = ov_tw;
  split_k = split_k > max_waves ? max_waves : split_k;
  split_k = split_k > ksteps ? ksteps : split_k;
  const int steps = ceil_div(ksteps, split_k);
  split_k = ceil_div(ksteps, steps);
  if (tiles_per_wg * split_k > max_waves) tiles_per_wg = max_waves / split_k;
  LaunchPlan lp;
  lp.split_k = split_k;
  lp.tiles_per_wg = tiles_per_wg;
  lp.steps_per_wave = steps;
  lp.workgroups = ceil_div(groups, tiles_per_wg);
  lp.tiles_in_sequence = 1;
  lp.staged_rows = 0;
  lp.matrix_core = mc;
  if (!mc) {
    // VALU path: fewer workgroups than tile groups means every wave walks several tiles.
    const int ov_wg = knobs.workgroups;
    int cap = ov_wg > 0 ? ov_wg : (workgroup_cap > 0 && ov_sk == 0 && ov_tw == 0) ? workgroup_cap : lp.workgroups;
    if (cap < lp.workgroups) lp.workgroups = cap;
    const int rows = m_batch < kMaxValuBatch ? m_batch : kMaxValuBatch;
    auto seq_tiles = [&]() { return ceil_div(tiles, lp.workgroups * tiles_per_wg); };
    // limits: a wave's weight range is addressed with 32-bit offsets; the combine parks
    // tiles x waves x rows x 64 floats in LDS
    while (lp.workgroups < ceil_div(groups, tiles_per_wg) &&
           ((long long)seq_tiles() * ksteps * kUnitBytes >= (1ll << 31) ||
            (long long)seq_tiles() * tiles_per_wg * split_k * rows * kWave * 4 > 64 * 1024))
      lp.workgroups = lp.workgroups * 2 < ceil_div(groups, tiles_per_wg) ? lp.workgroups * 2 : ceil_div(groups, tiles_per_wg);
    lp.tiles_in_sequence = seq_tiles();
  }
  lp.wgs_per_xcd = ceil_div(lp.workgroups, kNumXcd);
  lp.threads = kWave * split_k * tiles_per_wg;
  lp.tiles_per_wave = tiles_per_wave;
  return lp;
}

int check_problem(const void* weights, const void* scale, const void* zero_add, int n_out, int k, int& group_size,
                  int quant_op, int weight_bits) {
  if (quant_op != MGEMV_PER_COLUMN_SCALE_ONLY && quant_op != MGEMV_FINEGRAINED_SCALE_ONLY &&
      quant_op != MGEMV_FINEGRAINED_SCALE_AND_ZEROS)
    return MGEMV_ERR_QUANT_OP;
  if (weight_bits != 4 && weight_bits != 8) return MGEMV_ERR_QUANT_TYPE;
  if (n_out <= 0 || k <= 0) return MGEMV_ERR_SIZE;
  if (n_out % 4) return MGEMV_ERR_ROWS;
  if (k % chunk_k(weight_bits)) return MGEMV_ERR_COLS;
  if (quant_op == MGEMV_PER_COLUMN_SCALE_ONLY) {
    group_size = k;  // mixed_gemv_test.cu:142-143
  } else {
    if (group_size < 64) return MGEMV_ERR_GROUP_SIZE;  // gemv/device/gemv_adaptor.h:199-203
    if (group_size % 32 || k % group_size) return MGEMV_ERR_GROUP_SIZE;
  }
  if (weights == nullptr || scale == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (quant_op == MGEMV_FINEGRAINED_SCALE_AND_ZEROS && zero_add == nullptr) return MGEMV_ERR_NULL_POINTER;
  // 32-bit index arithmetic inside the kernels
  const long long groups = k / group_size;
  if (groups * (long long)n_out >= (1ll << 30)) return MGEMV_ERR_SIZE;
  if (num_ksteps(k, weight_bits) > 0xffff || group_size >= (1 << 24)) return MGEMV_ERR_SIZE;
  if ((long long)k * 2 * MGEMV_MAX_M_BATCH >= (1ll << 31)) return MGEMV_ERR_SIZE;
  if (reinterpret_cast<uintptr_t>(weights) % 16) return MGEMV_ERR_ALIGNMENT;
  if (reinterpret_cast<uintptr_t>(scale) % 2 || reinterpret_cast<uintptr_t>(zero_add) % 2) return MGEMV_ERR_ALIGNMENT;
  return MGEMV_OK;
}

// 1 or 2: the group size divides the k step ("regular" scale addressing, one or two groups per
// lane run); 4: any other legal group size ("generic", one lookup per block).
int groups_per_run(int group_size, int bits) {
  const int run = run_k(bits);
  if (step_k(bits) % group_size != 0) return 4;
  return group_size % run == 0 ? 1 : 2;
}

// Launches through hipLaunchKernel so that the status returned is this launch's own, not a
// stale sticky error left behind by some other runtime call of the process.
template <typename Kernel, typename... Args>
hipError_t launch(Kernel kernel, dim3 grid, dim3 block, size_t lds, hipStream_t stream, Args... args) {
  void* argv[] = {static_cast<void*>(&args)...};
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, argv, lds, stream);
}

// Host-side description of one GEMV launch.
struct GemvLaunch {
  const uint8_t* weights;
  const half_t* x;
  const half_t* scale;
  const half_t* zero_add;
  int n_out, k, group_size;
  LaunchPlan plan;
  GemvTail tail;
  dim3 grid, block;
  size_t lds;
  hipStream_t stream;
};

template <int BITS, int QOP, int MB, int GPR, bool MULTI, int ACT>
hipError_t launch_gemv_kernel_m(const GemvLaunch& g) {
  return launch(gemv_dpp_kernel<BITS, QOP, MB, GPR, MULTI, ACT>, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale,
                g.zero_add, g.n_out, g.k, pack_steps(num_ksteps(g.k, BITS), g.plan.steps_per_wave), g.plan.workgroups,
                g.tail.num_groups, pack_group(g.group_size, g.plan.tiles_per_wg), g.tail);
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

hipError_t launch_gemv(const GemvLaunch& g, int bits, int qop, int mb, int gpr, int act) {
  return act == kActBf16 ? launch_gemv_act<kActBf16>(g, bits, qop, mb, gpr)
                         : launch_gemv_act<kActF16>(g, bits, qop, mb, gpr);
}

template <int BITS, int QOP, int GPR, int T>
hipError_t launch_mfma_kernel_t(const GemvLaunch& g) {
  return launch(gemv_mfma_kernel<BITS, QOP, GPR, T>, g.grid, g.block, g.lds, g.stream, g.weights, g.x, g.scale,
                g.zero_add, g.n_out, g.k, pack_steps(num_ksteps(g.k, BITS), g.plan.steps_per_wave), g.plan.workgroups,
                g.plan.wgs_per_xcd, pack_group(g.group_size, g.plan.tiles_per_wg), g.tail);
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
template <int BITS, int QOP, int GPR, int ROUNDS, int ACT>
hipError_t launch_mfma_lds_kernel_r(const GemvLaunch& g) {
  const auto kernel = gemv_mfma_lds_kernel<BITS, QOP, GPR, ROUNDS, ACT>;
  if (g.lds > 48 * 1024) {
    // More than 48 KiB of dynamic LDS has to be granted per kernel and device; remember the
    // largest grant so that only the first such launch pays for the call.
    constexpr int kMaxDevices = 64;
    static std::atomic<int> granted[kMaxDevices];
    static std::mutex grant_mutex;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return hipErrorInvalidDevice;
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
                pack_group(g.group_size, g.plan.tiles_per_wg), g.tail);
}

template <int BITS, int QOP, int GPR, int ACT>
hipError_t launch_mfma_lds_kernel(const GemvLaunch& g, int rounds) {
  return rounds == 4 ? launch_mfma_lds_kernel_r<BITS, QOP, GPR, 4, ACT>(g)
                     : launch_mfma_lds_kernel_r<BITS, QOP, GPR, 8, ACT>(g);
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

hipError_t launch_mfma_lds(const GemvLaunch& g, int bits, int qop, int gpr, int rounds, int act) {
  return act == kActBf16 ? launch_mfma_lds_act<kActBf16>(g, bits, qop, gpr, rounds)
                         : launch_mfma_lds_act<kActF16>(g, bits, qop, gpr, rounds);
}

template <int BITS, int ACT>
hipError_t launch_dequant(const DequantParams& p, int qop, half_t* out, hipStream_t stream) {
  const long long units = (long long)p.tiles * p.ksteps;
  const dim3 block(256), grid((unsigned)((units + 3) / 4));
  switch (qop) {
    case 1: return launch(dequantize_kernel<BITS, 1, ACT>, grid, block, 0, stream, p, out);
    case 2: return launch(dequantize_kernel<BITS, 2, ACT>, grid, block, 0, stream, p, out);
    default: return launch(dequantize_kernel<BITS, 3, ACT>, grid, block, 0, stream, p, out);
  }
}

// act: kActF16 or kActBf16, the type behind every 16-bit operand.
int gemv_any(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
             const uint16_t* bias, uint16_t* y, int batch_count, int n_out, int m_batch, int k, int group_size,
             int quant_op, int weight_bits, int64_t stride_weights, int64_t stride_x, int64_t stride_scale,
             int64_t stride_bias, int64_t stride_y, void* stream, int act) {
  if (batch_count < 1 || batch_count > 65535) return MGEMV_ERR_BATCH;
  if (m_batch < 1 || m_batch > MGEMV_MAX_M_BATCH) return MGEMV_ERR_BATCH;
  if (const int st = check_problem(weights, scale, zero_add, n_out, k, group_size, quant_op, weight_bits)) return st;
  if (x == nullptr || y == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(y) % 2 ||
      reinterpret_cast<uintptr_t>(bias) % 2)
    return MGEMV_ERR_ALIGNMENT;
  if (stride_weights % 16 || stride_x % 8) return MGEMV_ERR_ALIGNMENT;

  GemvLaunch g{};
  g.weights = static_cast<const uint8_t*>(weights);
  g.scale = reinterpret_cast<const half_t*>(scale);
  g.zero_add = quant_op == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? reinterpret_cast<const half_t*>(zero_add) : nullptr;
  g.n_out = n_out;
  g.k = k;
  g.group_size = group_size;
  PlanKnobs knobs = knobs_for(n_out, k, weight_bits, group_size, m_batch);
  if (act == kActBf16) {
    // bf16: of the matrix-core kernels only the LDS-staged one (needs two tiles); the VALU kernel's
    // fp32 dequantiser wants the registers of 8-wave workgroups
    if (num_tiles(n_out) < 2) knobs.matrix_core_min_batch = MGEMV_MAX_M_BATCH + 1;
    knobs.matrix_core_variant = MGEMV_MATRIX_CORE_LDS_STAGED;
    knobs.wide_waves = true;
  }
  g.plan = plan_launch(n_out, k, weight_bits, m_batch, knobs);
  g.tail.bias = reinterpret_cast<const half_t*>(bias);
  g.tail.split_k = g.plan.split_k;
  g.tail.num_groups = k / group_size;
  g.tail.flags = g_dequant_flags.load();
  {
    const int sequences = g.plan.workgroups * g.plan.tiles_per_wg;
    g.tail.seq_base = num_tiles(n_out) / sequences;
    g.tail.seq_rem = num_tiles(n_out) % sequences;
  }
  g.tail.stride_weights = stride_weights;
  g.tail.stride_x = stride_x;
  g.tail.stride_scale = stride_scale;
  g.tail.stride_bias = stride_bias;
  g.tail.stride_y = stride_y;
  g.grid = dim3((unsigned)(g.plan.wgs_per_xcd * kNumXcd), 1, (unsigned)batch_count);
  g.block = dim3((unsigned)(kWave * g.plan.split_k), (unsigned)g.plan.tiles_per_wg, 1);
  g.stream = static_cast<hipStream_t>(stream);
  const int gpr = groups_per_run(group_size, weight_bits);

  if (g.plan.matrix_core) {
    g.x = reinterpret_cast<const half_t*>(x);
    g.tail.y = reinterpret_cast<half_t*>(y);
    g.tail.m_batch = m_batch;
    if (g.plan.staged_rows != 0) {
      const int row_stride = step_k(weight_bits) * 2 + 16;
      g.lds = (size_t)g.plan.split_k * 2 * g.plan.staged_rows * row_stride +
              (g.plan.split_k > 1 ? (size_t)g.plan.tiles_per_wg * g.plan.split_k * kWave * 4 * sizeof(float) : 0);
      return launch_mfma_lds(g, weight_bits, quant_op, gpr, g.plan.staged_rows / g.plan.tiles_per_wg, act) == hipSuccess
                 ? MGEMV_OK
                 : MGEMV_ERR_LAUNCH;
    }
    g.lds = g.plan.split_k == 1 ? 0
                                : (size_t)g.plan.tiles_per_wg * g.plan.split_k * g.plan.tiles_per_wave * kWave * 4 * sizeof(float);
    return launch_mfma(g, weight_bits, quant_op, gpr) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
  }
  // VALU path: activation rows are processed kMaxValuBatch at a time.
  for (int m0 = 0; m0 < m_batch; m0 += kMaxValuBatch) {
    const int mb = m_batch - m0 < kMaxValuBatch ? m_batch - m0 : kMaxValuBatch;
    g.x = reinterpret_cast<const half_t*>(x) + (size_t)m0 * (size_t)k;
    g.tail.y = reinterpret_cast<half_t*>(y) + (size_t)m0 * (size_t)n_out;
    g.lds = (size_t)g.plan.tiles_in_sequence * g.plan.tiles_per_wg * g.plan.split_k * mb * kWave * sizeof(float);
    if (launch_gemv(g, weight_bits, quant_op, mb, gpr, act) != hipSuccess) return MGEMV_ERR_LAUNCH;
  }
  return MGEMV_OK;
}

int dequantize_any(const void* weights, const uint16_t* scale, const uint16_t* zero_add, uint16_t* out, int n_out,
                   int k, int group_size, int quant_op, int weight_bits, void* stream, int act) {
  if (const int st = check_problem(weights, scale, zero_add, n_out, k, group_size, quant_op, weight_bits)) return st;
  if (out == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(out) % 4) return MGEMV_ERR_ALIGNMENT;
  DequantParams p{};
  p.weights = static_cast<const uint8_t*>(weights);
  p.scale = reinterpret_cast<const half_t*>(scale);
  p.zero_add = quant_op == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? reinterpret_cast<const half_t*>(zero_add) : nullptr;
  p.n_out = n_out;
  p.k = k;
  p.group_size = group_size;
  p.tiles = num_tiles(n_out);
  p.ksteps = num_ksteps(k, weight_bits);
  p.flags = g_dequant_flags.load();
  half_t* const o = reinterpret_cast<half_t*>(out);
  hipStream_t const st = static_cast<hipStream_t>(stream);
  hipError_t e;
  if (act == kActBf16)
    e = weight_bits == 4 ? launch_dequant<4, kActBf16>(p, quant_op, o, st) : launch_dequant<8, kActBf16>(p, quant_op, o, st);
  else
    e = weight_bits == 4 ? launch_dequant<4, kActF16>(p, quant_op, o, st) : launch_dequant<8, kActF16>(p, quant_op, o, st);
  return e == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
}

}  // namespace mgemv

extern "C" {

int mgemv_gemv_batched(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
                       const uint16_t* bias, uint16_t* y, int batch_count, int n_out, int m_batch, int k,
                       int group_size, int quant_op, int weight_bits, int64_t stride_weights, int64_t stride_x,
                       int64_t stride_scale, int64_t stride_bias, int64_t stride_y, void* stream) {
  return mgemv::gemv_any(weights, x, scale, zero_add, bias, y, batch_count, n_out, m_batch, k, group_size, quant_op,
                         weight_bits, stride_weights, stride_x, stride_scale, stride_bias, stride_y, stream,
                         mgemv::kActF16);
}

int mgemv_gemv_batched_bf16(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
                            const uint16_t* bias, uint16_t* y, int batch_count, int n_out, int m_batch, int k,
                            int group_size, int quant_op, int weight_bits, int64_t stride_weights, int64_t stride_x,
                            int64_t stride_scale, int64_t stride_bias, int64_t stride_y, void* stream) {
  return mgemv::gemv_any(weights, x, scale, zero_add, bias, y, batch_count, n_out, m_batch, k, group_size, quant_op,
                         weight_bits, stride_weights, stride_x, stride_scale, stride_bias, stride_y, stream,
                         mgemv::kActBf16);
}

int mgemv_gemv_bf16(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
                    const uint16_t* bias, uint16_t* y, int n_out, int m_batch, int k, int group_size, int quant_op,
                    int weight_bits, void* stream) {
  return mgemv_gemv_batched_bf16(weights, x, scale, zero_add, bias, y, 1, n_out, m_batch, k, group_size, quant_op,
                                 weight_bits, 0, 0, 0, 0, 0, stream);
}

int mgemv_dequantize_bf16(const void* weights, const uint16_t* scale, const uint16_t* zero_add, uint16_t* out, int n_out,
                          int k, int group_size, int quant_op, int weight_bits, void* stream) {
  return mgemv::dequantize_any(weights, scale, zero_add, out, n_out, k, group_size, quant_op, weight_bits, stream,
                               mgemv::kActBf16);
}

int mgemv_gemv(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
               const uint16_t* bias, uint16_t* y, int n_out, int m_batch, int k, int group_size, int quant_op,
               int weight_bits, void* stream) {
  return mgemv_gemv_batched(weights, x, scale, zero_add, bias, y, 1, n_out, m_batch, k, group_size, quant_op,
                            weight_bits, 0, 0, 0, 0, 0, stream);
}

int mgemv_dequantize(const void* weights, const uint16_t* scale, const uint16_t* zero_add, uint16_t* out, int n_out,
                     int k, int group_size, int quant_op, int weight_bits, void* stream) {
  return mgemv::dequantize_any(weights, scale, zero_add, out, n_out, k, group_size, quant_op, weight_bits, stream,
                               mgemv::kActF16);
}

int mgemv_set_launch_override(int split_k_waves, int tiles_per_workgroup, int tiles_per_wave, int max_workgroups) {
  if (split_k_waves < 0 || tiles_per_workgroup < 0 || tiles_per_wave < 0 || max_workgroups < 0) return MGEMV_ERR_SIZE;
  if (tiles_per_wave != 0 && tiles_per_wave != 1 && tiles_per_wave != 2 && tiles_per_wave != 4) return MGEMV_ERR_SIZE;
  mgemv::g_override_split_k.store(split_k_waves);
  mgemv::g_override_tiles_per_wg.store(tiles_per_workgroup);
  mgemv::g_override_tiles_per_wave.store(tiles_per_wave);
  mgemv::g_override_workgroups.store(max_workgroups);
  return MGEMV_OK;
}

int mgemv_set_matrix_core_threshold(int min_m_batch) {
  if (min_m_batch < 0 || min_m_batch > MGEMV_MAX_M_BATCH + 1) return MGEMV_ERR_BATCH;
  mgemv::g_matrix_core_min_batch.store(min_m_batch);
  return MGEMV_OK;
}

int mgemv_set_matrix_core_variant(int variant) {
  if (variant != MGEMV_MATRIX_CORE_AUTO && variant != MGEMV_MATRIX_CORE_REGISTER_OPERAND &&
      variant != MGEMV_MATRIX_CORE_LDS_STAGED)
    return MGEMV_ERR_SIZE;
  mgemv::g_matrix_core_variant.store(variant);
  return MGEMV_OK;
}

int mgemv_set_dequant_form(int form) {
  if (form != MGEMV_DEQUANT_AUTO && form != MGEMV_DEQUANT_EXACT_INTEGER) return MGEMV_ERR_SIZE;
  mgemv::g_dequant_flags.store(form == MGEMV_DEQUANT_EXACT_INTEGER ? mgemv::kExactIntegerFormOnly : 0);
  return MGEMV_OK;
}

namespace {
int check_tuned_key(int n_out, int k, int weight_bits, int group_size, int m_batch) {
  if (weight_bits != 4 && weight_bits != 8) return MGEMV_ERR_QUANT_TYPE;
  if (n_out <= 0 || k <= 0) return MGEMV_ERR_SIZE;
  if (group_size < 0) return MGEMV_ERR_GROUP_SIZE;
  if (m_batch < 1 || m_batch > MGEMV_MAX_M_BATCH) return MGEMV_ERR_BATCH;
  return MGEMV_OK;
}
}  // namespace

int mgemv_tuned_plan_set(const mgemv_tuned_plan* plan) {
  if (plan == nullptr) return MGEMV_ERR_NULL_POINTER;
  const int st = check_tuned_key(plan->n_out, plan->k, plan->weight_bits, plan->group_size, plan->m_batch);
  if (st != MGEMV_OK) return st;
  if (plan->split_k_waves < 0 || plan->tiles_per_workgroup < 0 || plan->max_workgroups < 0) return MGEMV_ERR_SIZE;
  const int t = plan->tiles_per_wave;
  if (t != 0 && t != 1 && t != 2 && t != 4) return MGEMV_ERR_SIZE;
  mgemv::PlanKnobs kn;
  kn.split_k = plan->split_k_waves;
  kn.tiles_per_wg = plan->tiles_per_workgroup;
  kn.tiles_per_wave = t;
  kn.workgroups = plan->max_workgroups;
  switch (plan->kernel) {
    case MGEMV_KERNEL_AUTO: break;
    case MGEMV_KERNEL_VALU: kn.matrix_core_min_batch = MGEMV_MAX_M_BATCH + 1; break;
    case MGEMV_KERNEL_MATRIX_CORE_REGISTER_OPERAND:
      kn.matrix_core_min_batch = 1;
      kn.matrix_core_variant = MGEMV_MATRIX_CORE_REGISTER_OPERAND;
      break;
    case MGEMV_KERNEL_MATRIX_CORE_LDS_STAGED:
      kn.matrix_core_min_batch = 1;
      kn.matrix_core_variant = MGEMV_MATRIX_CORE_LDS_STAGED;
      break;
    default: return MGEMV_ERR_SIZE;
  }
  std::lock_guard<std::mutex> lock(mgemv::g_tuned_mutex);
  mgemv::g_tuned_plans[mgemv::PlanKey{plan->n_out, plan->k, plan->weight_bits, plan->group_size, plan->m_batch}] = kn;
  mgemv::g_tuned_count.store((int)mgemv::g_tuned_plans.size());
  return MGEMV_OK;
}

int mgemv_tuned_plan_clear(void) {
  std::lock_guard<std::mutex> lock(mgemv::g_tuned_mutex);
  mgemv::g_tuned_plans.clear();
  mgemv::g_tuned_count.store(0);
  return MGEMV_OK;
}

int mgemv_tuned_plan_count(void) { return mgemv::g_tuned_count.load(); }

int mgemv_query_launch(int n_out, int m_batch, int k, int weight_bits, int group_size, int out[8]) {
  if (out == nullptr) return MGEMV_ERR_NULL_POINTER;
  const int st = check_tuned_key(n_out, k, weight_bits, group_size, m_batch);
  if (st != MGEMV_OK) return st;
  const mgemv::LaunchPlan lp = mgemv::plan_launch(n_out, k, weight_bits, m_batch,
                                                  mgemv::knobs_for(n_out, k, weight_bits, group_size, m_batch));
  out[0] = lp.wgs_per_xcd * mgemv::kNumXcd;
  out[1] = lp.threads;
  out[2] = lp.split_k;
  out[3] = lp.tiles_per_wg;
  out[4] = lp.steps_per_wave;
  out[5] = !lp.matrix_core ? 0 : lp.staged_rows != 0 ? 2 : 1;
  out[6] = lp.tiles_per_wave;
  out[7] = lp.tiles_in_sequence;
  return MGEMV_OK;
}

}  // extern "C"
