// C-ABI entry points of the device side: argument checks, launch geometry, tuned plans, and the
// dequantise kernel.  The GEMV kernels live in gemv_dpp_kernel.h (VALU) and launch_mfma.hip
// (matrix cores).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "kernel_common.h"

namespace mgemv {

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
        if (k0 + j * G::kWordK >= p.k) continue;  // k is a multiple of 8: whole words
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
      if (k0 + j * G::kWordK >= p.k) continue;  // k is a multiple of 8: whole words
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
std::atomic<int> g_override_stages{0};        // 0 = built-in (2), 1 or 2
std::atomic<int> g_matrix_core_variant{MGEMV_MATRIX_CORE_AUTO};

// What steers plan_launch besides the shape: zeros mean "built-in rule".
struct PlanKnobs {
  int split_k = 0, tiles_per_wg = 0, tiles_per_wave = 0, workgroups = 0;
  int matrix_core_min_batch = 0;
  int matrix_core_variant = MGEMV_MATRIX_CORE_AUTO;
  bool wide_waves = false;  // the kernel is one of those compiled for at most 8 waves per workgroup
  int stages = 0;           // VALU kernel: 0 = built-in rule (2: the next unit in flight while one is computed), 1, 2
  int num_cus = kNumCus;    // compute units of the device the launch goes to (256 on an unpartitioned MI355X)
  bool generic_groups = false;  // the group size does not divide the k step: one scale / zero lookup per block of a unit
};

// Tuned plans by problem: (n_out, k, weight bits, group size or 0 for any, m_batch) -> knobs.
using PlanKey = std::tuple<int, int, int, int, int, int>;  // n_out, k, bits, group size, rows, element
std::mutex g_tuned_mutex;
std::map<PlanKey, PlanKnobs> g_tuned_plans;
std::atomic<int> g_tuned_count{0};  // lets the launch path skip the lock while the table is empty

// Built-in table: plans measured on an unpartitioned MI355X that the rules below do not produce,
// kept as data (mixed_gemv_amd/default_plans.json, compiled in by the build) instead of as one
// more shape threshold in plan_launch.  Consulted after the caller's table, for launches on a
// device of kDefaultPlanCus compute units only.
const mgemv_tuned_plan kDefaultPlans[] = {
#include "default_plans.inc"
    {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}  // terminator (n_out = 0)
};
constexpr int kDefaultPlanCus = 256;
std::atomic<int> g_default_plans_enabled{1};

int default_plan_count() {
  int n = 0;
  while (kDefaultPlans[n].n_out != 0) ++n;
  return n;
}

PlanKnobs knobs_of_plan(const mgemv_tuned_plan& plan) {
  PlanKnobs kn;
  kn.split_k = plan.split_k_waves;
  kn.tiles_per_wg = plan.tiles_per_workgroup;
  kn.tiles_per_wave = plan.tiles_per_wave;
  kn.workgroups = plan.max_workgroups;
  kn.stages = plan.stages;
  switch (plan.kernel) {
    case MGEMV_KERNEL_VALU: kn.matrix_core_min_batch = MGEMV_MAX_M_BATCH + 1; break;
    case MGEMV_KERNEL_MATRIX_CORE_REGISTER_OPERAND:
      kn.matrix_core_min_batch = 1;
      kn.matrix_core_variant = MGEMV_MATRIX_CORE_REGISTER_OPERAND;
      break;
    case MGEMV_KERNEL_MATRIX_CORE_LDS_STAGED:
      kn.matrix_core_min_batch = 1;
      kn.matrix_core_variant = MGEMV_MATRIX_CORE_LDS_STAGED;
      break;
    case MGEMV_KERNEL_MATRIX_CORE_K_STATIONARY:
      kn.matrix_core_min_batch = 1;
      kn.matrix_core_variant = MGEMV_MATRIX_CORE_K_STATIONARY;
      break;
    default: break;
  }
  return kn;
}

// Process-wide overrides win over the tables (they are what a tuner sweeps); then the caller's
// entry for exactly this group size, then its entry for any group size, then the built-in table,
// then the built-in rules.
PlanKnobs knobs_for(int n_out, int k, int bits, int group_size, int m_batch, int act, int num_cus) {
  PlanKnobs kn;
  kn.split_k = g_override_split_k.load();
  kn.tiles_per_wg = g_override_tiles_per_wg.load();
  kn.tiles_per_wave = g_override_tiles_per_wave.load();
  kn.workgroups = g_override_workgroups.load();
  kn.matrix_core_min_batch = g_matrix_core_min_batch.load();
  kn.matrix_core_variant = g_matrix_core_variant.load();
  kn.stages = g_override_stages.load();
  const bool overridden = kn.split_k || kn.tiles_per_wg || kn.tiles_per_wave || kn.workgroups || kn.stages ||
                          kn.matrix_core_min_batch || kn.matrix_core_variant != MGEMV_MATRIX_CORE_AUTO;
  if (overridden) return kn;
  const int element = act == kActBf16 ? MGEMV_ELEMENT_BF16 : MGEMV_ELEMENT_F16;
  if (g_tuned_count.load() != 0) {
    std::lock_guard<std::mutex> lock(g_tuned_mutex);
    auto it = g_tuned_plans.find(PlanKey{n_out, k, bits, group_size, m_batch, element});
    if (it == g_tuned_plans.end() && group_size != 0) it = g_tuned_plans.find(PlanKey{n_out, k, bits, 0, m_batch, element});
    if (it != g_tuned_plans.end()) return it->second;
  }
  if (num_cus == kDefaultPlanCus && g_default_plans_enabled.load() != 0) {
    for (const mgemv_tuned_plan* p = kDefaultPlans; p->n_out != 0; ++p)
      if (p->n_out == n_out && p->k == k && p->weight_bits == bits && p->m_batch == m_batch && p->element == element &&
          (p->group_size == group_size || p->group_size == 0))
        return knobs_of_plan(*p);
  }
  return kn;
}

// Which row counts go to the matrix cores.  From 5 rows the VALU kernel would need a second pass
// over the weights (4096x4096: 8.8 us against 5.5).  The VALU kernel pays per row, the matrix-core kernels
// (almost) not, but the VALU kernel is at its best with at most one workgroup per compute unit:
// measured over 21 shapes, 3 and 4 rows are faster on the matrix cores whenever there are more
// than 256 tiles (5120x4096, 3 rows: 6.45 us against 6.74; 14336x4096, 4 rows: 9.2 against 11.4;
// the one exception found, 11008x4096 at 3 rows, loses 5 %) and on the VALU kernel below that
// (4096x14336, 4 rows: 10.6 against 11.3); 2 rows only from about 1536 tiles (32000x4096: 15.1
// against 16.4; 28672x8192: 25.9 against 27.3; 10240x8192: 14.2 against 12.7 the other way), and
// with fewer than 8 k steps only when one-unit VALU waves would not fit the machine (50304x2048,
// 12576 units: 15.2 against 12.8 the other way; 151936x2048, 37984 units: 33.1 against 35.1).
// cus: compute units of the device; the tile and unit counts the rules were measured at (on 256
// compute units) scale with it.
inline bool use_matrix_cores(int m_batch, int tiles, int ksteps, int forced, bool bf16, int bits, int cus) {
  if (forced > 0) return m_batch >= forced;
  // int8 weights: twice the bytes per VALU instruction, so the VALU kernel holds out longer --
  // ahead at 2-4 rows on every shape measured (8192x8192, 3 rows: 13.0 us against 14.8; 4096x11008,
  // 4 rows: 10.4 against 11.5) except the largest (28672x8192, 3 rows: 41.4 against 39.7).
  if (bits == 8) return m_batch >= 5 || (m_batch >= 3 && tiles >= 6 * cus);
  const long long units = (long long)tiles * ksteps;
  // 4 rows on up to 256 tiles: the barrier-free one-tile matrix-core launch is ahead from 16 k steps
  // (4096x8192: 6.9 us against 7.4; 4096x14336: 9.7 against 10.7; 3584x18944: 12.3 against 13.8)
  // and level below (4096x4096: 5.07 against 5.00); 2 and 3 rows stay on the VALU kernel there.
  return m_batch >= 5 || (m_batch >= 3 && tiles > cus && units >= 8ll * cus) ||
         (m_batch >= 4 && tiles >= 2 && ksteps >= 16) ||  // also on few tiles: 1536x8960 7.4 / 8.2; 1024x14336 9.0 / 10.2; 512x16384 9.9 / 10.9
         (m_batch >= 2 && !bf16 && tiles >= 6 * cus && (ksteps >= 8 || units > 64ll * cus));  // bf16, 28672x8192, 2 rows: 40.6 us against 37.8
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tiles per workgroup of the LDS-staged matrix-core kernel (= waves that share one activation stage): as few as
// bring the launch down to one workgroup per compute unit or fewer, at most 8 and at most a quarter of the staged
// rows.  Measured, 16 rows: 4096x4096 (256 tiles) 6.3 us at 1 tile against 7.2 at 2; 8192x8192 (512)
// 13.4 at 2 against 17.8 at 4; 11008x4096 (688) 10.1 at 4 against 11.3 at 2 and 14.2 at 8;
// 28672x8192 (1792) 28.3 at 8 against 30.6 at 4 and 32.8 at 2.  8 rows: 4096x4096 5.4 at 1
// against 6.4 at 2; 5120x5120 (320) 7.7 at 2 against 9.3 at 1; 10240x8192 (640) 14.7 at 4
// against 15.5 at 2; 11008x4096 9.0 at 4 against 9.7 at 2; 28672x8192 27.6 at 4 against 29.5 at 2.
// Still more workgroups than compute units: a count just above a multiple of 256 leaves most
// of the last round idle, and halving the tiles per workgroup evens that out (18944x3584,
// 8 rows: 296 workgroups of 4 tiles 12.8 us, 592 of 2 tiles 11.8; 22016x4096: 14.4 / 13.3):
// the largest count whose last round is at least three quarters full.
inline int lds_staged_tiles_per_wg(int tiles, int staged_rows, int cus) {
  int tw = 1;
  while (ceil_div(tiles, tw) > cus && tw * 2 <= 8 && tw * 4 <= staged_rows) tw *= 2;
  if (ceil_div(tiles, tw) > cus) {
    for (int t = tw; t >= 1; t /= 2) {
      const int wgs = ceil_div(tiles, t);
      if (wgs * 4 >= ceil_div(wgs, cus) * cus * 3) return t;
    }
  }
  return tw;
}

// Where the k-stationary matrix-core kernel (one wave per k step, one workgroup per compute unit walking
// ceil(tiles / cus) tiles) is ahead of the others; fp16, 4 to 16 k steps, 2 to 16 rows (int4 unless noted).  Its waves hold
// their activation operand in registers, so its loop has neither barriers nor LDS reads and costs the same at 1 to
// 8 rows; what it pays is a fixed start (operand through LDS, 0.8-1.6 us) and end (one barrier, one combine), and a
// tail: when the weight stream ends, every wave of a SIMD still has a unit to compute.  Measured against the
// built-in choice otherwise (us, k-stationary first):
//   up to 8 k steps (at most 2 waves per SIMD), 3-8 rows, more tiles than compute units (4-5 k steps: 1.5 times
//     as many; 2 rows: 8 k steps and 2.5 times as many): 4608x4096 4 rows 5.60 / 6.41; 5120x3072 5.52 / 6.82; 8192x4096 6.06 / 6.88;
//     10240x4096 7.25 / 8.77, 8 rows 7.66 / 8.89; 11008x4096 3 rows 7.29 / 8.80; 22016x4096 2 rows 11.43 / 12.77;
//     28672x4096 8 rows 13.92 / 15.50; 8192x2048 7 rows 4.75 / 5.17; 50304x2048 4 rows 13.98 / 15.61; 128256x4096
//     4 rows 46.3 / 50.2; but 4608x2048 4 rows 4.58 / 4.49, and with 1-2 k steps there are 1-2 waves per compute
//     unit (32768x1024 10.4 / 7.2);
//   9-16 k steps: wherever its one-workgroup-per-compute-unit walks fill the machine better than the LDS-staged
//     kernel's workgroups of 1-4 tiles do -- 9216x8192 4 rows 12.48 / 14.18; 10240x8192 12.65 / 14.14, 8 rows 13.37
//     / 14.49; 12288x8192 3 rows 12.94 / 14.42; 18432x8192 17.73 / 22.40; 20480x8192 18.23 / 22.61; 28672x8192 2 /
//     4 / 8 rows 22.3 / 22.5 / 23.4 against 24.7 / 24.9 / 26.2 -- and, where the two fill it alike: at 3-4 rows with
//     walks of up to 3 tiles or tiles that divide evenly (5120x5120 6.82 / 7.62; 8192x7168 8.79 / 10.03; 8192x8192
//     10.34 / 10.37; 16384x8192 14.79 / 15.36; but 13312x8192 14.99 / 14.63, 13824x5120 10.97 / 10.60), at 5-8 rows
//     only up to 12 k steps with walks of 2 (8192x6144 7.80 / 8.64; but 8192x8192 11.01 / 10.50, 16384x8192 16.42 /
//     15.95, 14336x8192 16.0 / 15.3), at 2 rows from walks of 3 (12288x8192 12.74 / 13.28; 8192x8192 9.93 / 9.05);
//   1 row: never by this rule -- the single-row path is the VALU kernel by design.  Forced (threshold 1, this
//     variant) it is ahead only with 9-16 k steps and even walks of 7 tiles or more: 28672x8192 22.2 / 22.5 (three
//     leases: 1.9, 1.8, 0.5 % ahead), 32768x8192 25.5 / 26.9, 57344x8192 40.0 / 43.9; below that the VALU kernel's
//     finer pipeline wins (16384x8192 14.9 / 13.1; 128256x4096, 8 waves, 47.8 / 45.7);
//   int8 weights (a k step is 256 long, the operand 32 registers): ahead on every shape tried at 3-8 rows, 16 waves
//     and walks of 2 included -- 8192x4096 3 / 8 rows 7.68 / 8.12, 8.18 / 9.02; 11008x4096 8 rows 10.02 / 11.76;
//     14336x2048 4 rows 7.49 / 8.58; 16384x4096 6 rows 12.87 / 14.34; 28672x4096 8 rows 20.69 / 21.57 -- so the
//     rule of up to 8 k steps serves 8-16 there (78 launches on 19 further shapes: median +7.9 %; with 4-6 k steps
//     it is 5-7 % behind);
//   9-16 rows: the operand takes two rounds through LDS and twice the registers' worth of L2 traffic per wave, and
//     the LDS-staged kernel shares a stage between up to 8 tiles there.  Ahead where that kernel's workgroups fill
//     the machine worse by a tenth or more -- 11008x4096 16 rows 8.99 / 9.92; 10240x4096 8.68 / 9.87; 17408x4096
//     12.59 / 14.40; 12288x8192 12 rows 15.04 / 16.31; 18432x8192 16 rows 20.56 / 25.39; 20480x8192 20.99 / 25.48;
//     28672x8192 12 / 16 rows 25.75 / 27.08, 26.32 / 27.73 -- except on long walks of 8-wave workgroups (28672x4096
//     12 rows 15.34 / 14.87; 22016x4096, walks of 6, 13.68 / 13.98 still ahead); level or behind where the two fill
//     it alike (8192x6144 16 rows 10.44 / 9.90; 14336x8192 18.1 / 17.0; 14336x4096 12 rows 10.18 / 10.16) or where
//     the partial sums of a walk do not fit the LDS and the workgroups double (32768x8192 35.1 / 30.0).
//   * group sizes that do not divide the k step (one scale / zero lookup per block: PlanKnobs::generic_groups) stay
//     with the other kernels, the caller sees to that: 11008x3072 g96 at 4 rows 10.98 / 9.61; 14336x4608 g96 16.0 /
//     13.95; 28672x8064 g96 36.45 / 33.08; 8192x6144 g192 12.34 / 10.83; 20480x5120 g160 19.9 / 19.9.
inline bool use_k_stationary(int m_batch, int tiles, int ksteps, int bits, int cus) {
  if (m_batch == 1 || ksteps < 4) return false;  // a single row stays on the VALU kernel, whatever was measured (above)
  const int walk = ceil_div(tiles, cus);
  const long long slots = (long long)walk * cus;  // tiles the launch has room for
  if (m_batch > 8) {
    // 9-16 rows: only where it fills the machine better than the LDS-staged kernel's workgroups of up to 8 tiles,
    // the partial sums of a whole walk fit the LDS, and -- with up to 8 k steps, 2 waves per SIMD -- walks stay short
    const int tw16 = lds_staged_tiles_per_wg(tiles, 16, cus);
    const long long lds_slots16 = (long long)ceil_div(ceil_div(tiles, tw16), cus) * cus * tw16;
    const long long park = (long long)walk * kKSlices * m_batch * kKStationaryParkSlots * 16;
    // int8 weights: the operand is half as many registers and the stage half as long, and the kernel is ahead by
    // 4-37 % on all 52 launches tried at 10-16 rows with 4-16 k steps and more tiles than compute units, as long as
    // the partial sums of a walk fit the LDS (11008x4096 at 16 rows 10.74 us / 12.94; 18944x3584 14.80 / 19.09;
    // 9216x3072 at 12 rows 7.80 / 10.67; 22016x2048 10.98 / 12.17; 11008x1024 5.78 / 6.14; where the workgroups double
    // for the LDS it loses: 32000x4096 at 16 rows 25.66 / 24.19, 50304x2048 22.62 / 21.19)
    if (bits == 8) return tiles > cus && park <= kMaxKStationaryLds;
    // a tile count that leaves the LDS-staged kernel only pairs of tiles on a large matrix: ahead even where the partial
    // sums of a walk need twice the workgroups (36400x5376 at 12 / 16 rows 23.1 / 29.3 us against 33.5 / 35.0)
    if (tw16 <= 2 && tiles > 4 * cus) return true;
    // up to 12 rows on walks of 2: 5120x5120 7.86 / 8.89; 7792x6016 8.98 / 9.83; 6144x4096 6.95 / 7.32; 8192x8192 level
    if (m_batch <= 12 && walk == 2 && park <= kMaxKStationaryLds) return true;
    return lds_slots16 * 10 >= slots * 11 && park <= kMaxKStationaryLds && (ksteps > 8 || walk <= 6);
  }
  if (tiles <= cus) {
    // At most one tile per compute unit, so no walk: still ahead of the VALU kernel's chunks of rows and of the
    // LDS-staged kernel at 3-7 rows with 9-14 k steps (4096x4608 4 rows 5.38 / 6.53; 2048x5120 5.10 / 6.44; 3072x6144
    // 5.43 / 6.29; 4096x6656 6.39 / 7.19; 3584x7168 6.31 / 7.14; 6 rows 4-7 % -- but 4096x7680, 15 k steps, 6 rows 7.72 /
    // 6.92 and 4096x8192, 16 waves, 3 / 4 / 8 rows 7.44 / 6.70, 7.70 / 6.98, 8.38 / 7.21) and at 4-7 rows with 5-8
    // (2560x2560 4 rows 4.35 / 4.74; 4096x3072 4.70 / 4.94; 4096x4096 6 rows 4.85 / 5.13; 3 rows lose 4-7 %; 8 rows
    // level).  Measured from 128 tiles up, int4.
    if (bits == 8 || tiles * 2 < cus || m_batch > 7) return false;
    if (ksteps <= 8) return ksteps >= 5 && m_batch >= 4;
    return m_batch >= 3 && (ksteps <= 14 || (ksteps == 15 && m_batch <= 4));
  }
  // tile counts that leave the LDS-staged kernel without a tidy grouping (it falls back to a workgroup per tile, no
  // stage shared): 16880x5376 at 3 / 5 / 8 rows 12.6 / 12.9 / 14.0 us against 17.4 / 17.7 / 17.8; 17408x8192 17.2 / 17.6 /
  // 18.4 against 24.1 / 24.1 / 24.3; int8 17728x1792 at 6 rows 7.9 / 10.2
  const int tw = lds_staged_tiles_per_wg(tiles, 8, cus);
  if (tw == 1 && tiles > 2 * cus && m_batch >= 3) return true;
  if (bits == 8 && ksteps < 7) return false;  // 8192x1024 int8, 3 rows: 4.9 us against 4.6; 32768x1536: 10.9 / 10.3 (but 11264x1792, 7 k steps, 4 rows: 5.9 / 7.0)
  if (ksteps <= 8 || bits == 8) {
    // the VALU kernel's two rows are cheap (8192x4096 5.90 / 5.95; 6144x3072 5.46 / 5.19; 12288x2560, 5 k steps, 6.71 /
    // 5.57): from 6 k steps and 2.5 tiles per compute unit (10240x3584 7.01 / 7.27; 12288x3072 6.84 / 7.30; 18944x3584
    // 9.88 / 10.47; 22016x3072 10.17 / 11.44; 37888x3584 15.89 / 17.87; 50304x3072 18.79 / 20.75)
    if (m_batch == 2) return (bits == 8 ? ksteps == 8 : ksteps >= 6) && tiles * 2 >= cus * 5;
    // five waves on four SIMDs: one SIMD carries two of them through every tile, and on longer walks the LDS-staged
    // kernel is ahead (26208x2176 at 3 rows 10.1 us / 11.3; 30112x2176 10.3 / 12.1; 14240x2560 at 8 rows 7.3 / 7.8)
    if (ksteps == 5 && walk >= 4) return false;
    return ksteps <= 5 ? tiles * 2 >= cus * 3 : tiles > cus;
  }
  const long long lds_slots = (long long)ceil_div(ceil_div(tiles, tw), cus) * cus * tw;
  if (lds_slots * 10 >= slots * 11) return m_batch >= 3 || walk >= 3;  // fills the machine better by a tenth or more
  // two rows: from walks of 3 tiles, evenly filled or not (21024x7808, walks of 6 at 85 %, 19.1 us / 21.8; 22016x8192 20.1 /
  // 22.2; 30064x6144 19.2 / 20.5; 14336x8192 and 16336x5632 level; 13824x5120, whose whole-k VALU waves fit well, 10.9 / 10.55)
  if (m_batch == 2) return walk >= 3;
  // walks of 4 up to 5 rows and 15 k steps: 13584x5632 11.1-11.2 / 12.0; 15360x6144 11.6-11.7 / 12.4-12.5; 12480x7424
  // 13.6-14.1 / 14.7; 16384x6144 at 5 rows 12.0 / 12.8 (13824x5120 10.9 / 10.7; with 16 k steps 13312x8192 15.1 / 14.7)
  if (m_batch <= 5 && walk == 4 && ksteps <= 15) return true;
  // ... and up to 8 rows with 9-11 k steps (12480x5632 at 6 rows 10.8 / 11.9; 13584x5632 at 8 rows 11.4 / 12.2; with 12-16
  // k steps 6-8 rows lose 3-5 %: 15360x6144, 14336x8192)
  if (walk == 4 && ksteps <= 11) return true;
  if (m_batch <= 4) return walk == 2 || walk == 3 || walk >= 5 || slots == tiles;  // (walks of 5 and more: 22944x7680 at 4 rows 19.7 / 22.4)
  // 5-8 rows: walks of 2 up to 12 k steps, and walks of 5 or more (22144x7936 at 6 rows 20.9 us / 23.8; 20672x8064 at 8
  // rows 20.3 / 23.1; 23104x7680 at 5 rows 20.8 / 23.1; 29024x5760 19.3 / 21.2); walks of 4 lose 3-5 % at 6-8 rows
  return (walk == 2 && ksteps <= 12) || walk >= 5;
}

LaunchPlan plan_launch(int n_out, int k, int bits, int m_batch, const PlanKnobs& knobs) {
  const int tiles = num_tiles(n_out), ksteps = num_ksteps(k, bits);
  const int cus = knobs.num_cus > 0 ? knobs.num_cus : kNumCus;  // the thresholds below were measured on 256 and scale with it
  const int ov_sk = knobs.split_k, ov_tw = knobs.tiles_per_wg;
  const int ov_t = knobs.tiles_per_wave;
  const bool mc = use_matrix_cores(m_batch, tiles, ksteps, knobs.matrix_core_min_batch, knobs.wide_waves, bits, cus);
  // K-stationary kernel: one wave per k step (so at most 16 k steps), one workgroup per compute unit
  // or fewer, each walking a contiguous run of tiles; more workgroups only where a walk's partial
  // sums would not fit the LDS or its weights not a 32-bit offset.
  // fp16 only: the bf16 dequantiser does not fit 128 registers beside the operand (with spills: 28672x8192 40.2 us against 35.1)
  const bool kstat_exists = ksteps <= kMaxWavesPerWorkgroup && !knobs.wide_waves;
  const bool kstat_asked = mc && knobs.matrix_core_variant == MGEMV_MATRIX_CORE_K_STATIONARY;
  const bool kstat_by_rule = knobs.matrix_core_variant == MGEMV_MATRIX_CORE_AUTO && knobs.matrix_core_min_batch == 0 &&
                             ov_sk == 0 && ov_tw == 0 && ov_t == 0 && !knobs.generic_groups &&
                             use_k_stationary(m_batch, tiles, ksteps, bits, cus);
  if (kstat_exists && (kstat_asked || kstat_by_rule)) {
    LaunchPlan lp{};
    lp.matrix_core = true;
    lp.k_stationary = true;
    lp.split_k = ksteps;
    lp.steps_per_wave = 1;
    lp.tiles_per_wg = 1;
    lp.tiles_per_wave = 1;
    lp.stages = 2;
    lp.workgroups = knobs.workgroups > 0 ? knobs.workgroups : cus;
    if (lp.workgroups > tiles) lp.workgroups = tiles;
    auto walk = [&]() { return ceil_div(tiles, lp.workgroups); };
    const long long park_bytes = (long long)kKSlices * m_batch * kKStationaryParkSlots * 16;  // per tile of a walk
    while (lp.workgroups < tiles &&
           ((long long)(walk() + 2) * ksteps * kUnitBytes >= (1ll << 31) ||  // (the loop requests up to two tiles past the walk)
            walk() * park_bytes > kMaxKStationaryLds))
      lp.workgroups = lp.workgroups * 2 < tiles ? lp.workgroups * 2 : tiles;
    lp.tiles_in_sequence = walk();
    lp.wgs_per_xcd = ceil_div(lp.workgroups, kNumXcd);
    lp.threads = kWave * lp.split_k;
    return lp;
  }
  // The LDS-staged kernel serves every matrix-core launch of two or more tiles.  (While its loop
  // still had a workgroup barrier per k step, the register-operand kernel was ahead on problems of
  // up to 256 tiles with up to 5 rows or up to 4 k steps; without the barrier the LDS-staged kernel
  // with one tile per workgroup wins there too -- 4096x4096, 5 rows: 4.98 us against 5.34;
  // 2048x8192, 5 rows: 6.5 against 7.5; 2048x2048, 8 rows: 3.68 against 3.91 -- or is level,
  // 2048x2048, 5 rows: 3.62 against 3.57.)
  if (mc && knobs.matrix_core_variant != MGEMV_MATRIX_CORE_REGISTER_OPERAND && tiles >= 2) {
    // LDS-staged kernel: the tiles of a workgroup share the activation stage; k split as long as
    // the launch stays within 2048 waves (measured: 8192x8192 best at 4 k-split waves, 11008x4096
    // at 2, 28672x8192 at 1).
    LaunchPlan lp{};
    lp.matrix_core = true;
    lp.staged_rows = m_batch <= 8 ? 8 : 16;
    lp.tiles_per_wg = lds_staged_tiles_per_wg(tiles, lp.staged_rows, cus);
    // Long reductions on many tiles (more than 16 k steps, more than 4 tiles per compute unit; the k-stationary kernel
    // does not reach these) want about two workgroups per compute unit, of few waves that walk the whole reduction:
    // 2 tiles per workgroup, or 4 where that still leaves more than 2.75 workgroups per compute unit; up to 8 rows,
    // workgroups of 2 tiles split k in two.  Against what the rules above give (us): 34576x8576 at 12 rows 40.9 / 47.7;
    // 33664x8832 at 16 rows 43.8 / 52.0; 19056x10112 at 3 / 12 rows 24.7 / 27.8, 32.8 / 38.1; 16400x9216 at 16 rows
    // 29.4 / 35.0; 28672x8704 at 5 / 16 rows 29.0 / 32.2, 33.0 / 36.2; 22016x11008 at 8 rows 30.4 / 33.6.
    const bool long_reduction = ksteps > 16 && tiles > 4 * cus;
    // (Up to 8 rows, 4 tiles only where their workgroups fill the last round to three quarters -- 28672x8704 and int8
    // 27216x4224 do, 23648x11392 and int8 33616x4352 do not: 4-12 % either way.)
    if (long_reduction) {
      const int wgs4 = ceil_div(tiles, 4);
      const bool four = lp.staged_rows == 16 ? ceil_div(tiles, 2) * 4 > cus * 11 : wgs4 * 4 >= ceil_div(wgs4, cus) * cus * 3;
      lp.tiles_per_wg = four ? 4 : 2;
    }
    // the kernel exists for 2, 4, 8 or 16 staged rows per wave of a k range
    if (ov_tw > 0 && ov_tw <= 8 && lp.staged_rows % ov_tw == 0 && lp.staged_rows / ov_tw >= 2) lp.tiles_per_wg = ov_tw;
    lp.workgroups = ceil_div(tiles, lp.tiles_per_wg);
    const int max_split = kMaxWavesPerMfmaWorkgroup / lp.tiles_per_wg < 4 ? kMaxWavesPerMfmaWorkgroup / lp.tiles_per_wg : 4;
    int split = 1;
    // (a tile count that left every tile a workgroup of its own, on a large matrix: single-wave workgroups are the worst
    // of all -- 16880x5376 bf16 at 5 rows 28.7 us against 22.6 with four k-split waves -- so those may use twice the waves)
    const int lds_wave_budget = (lp.tiles_per_wg == 1 && tiles > 2 * cus ? 20 : 8) * cus;
    while (split < max_split && split * 2 <= ksteps && (long long)lp.workgroups * lp.tiles_per_wg * split * 2 <= lds_wave_budget) split *= 2;
    if (long_reduction) split = lp.staged_rows == 8 && lp.tiles_per_wg == 2 ? 2 : 1;
    // three k steps: a wave each instead of 2 + 1 (2048x1408, 8 / 16 rows: 3.52 / 3.96 us against 4.11 / 4.69)
    if (ksteps == 3 && split == 2 && max_split >= 3 && (long long)lp.workgroups * lp.tiles_per_wg * 3 <= 8 * cus) split = 3;
    // A split that leaves the last wave nearly idle (10 k steps over 4 waves: 3, 3, 3, 1) loses
    // to half as many evenly loaded waves, as long as the workgroup keeps four (5120x5120, 8 rows,
    // 2 tiles: 7.6 us at 2 waves per tile against 8.1 at 4; 6912x5120, 16 rows: 9.0 against 9.6;
    // but 4096x6656, 8 rows, 1 tile: 9.1 at 2 against 7.8 at 4).
    auto padded_steps = [&](int s) { const int st = ceil_div(ksteps, s); return st * ceil_div(ksteps, st); };
    if (lp.tiles_per_wg * split >= 8 && padded_steps(split) * 100 > ksteps * 115 &&
        padded_steps(split / 2) < padded_steps(split))
      split /= 2;
    if (ov_sk > 0) split = ov_sk > max_split ? max_split : ov_sk;
    if (split > ksteps) split = ksteps;
    lp.steps_per_wave = ceil_div(ksteps, split);
    lp.split_k = ceil_div(ksteps, lp.steps_per_wave);
    lp.wgs_per_xcd = ceil_div(lp.workgroups, kNumXcd);
    lp.threads = kWave * lp.split_k * lp.tiles_per_wg;
    lp.tiles_per_wave = 1;
    lp.tiles_in_sequence = 1;
    lp.stages = 2;
    return lp;
  }
  // Matrix-core path: a wave that works on T tiles fetches the activation operands of a k step
  // once for all of them.  Measured on 8192 x 8192 (512 tiles): T = 2 is 1.5-1.8x faster than
  // T = 1 at 8-16 activation rows; T = 4 leaves too few waves to cover the load latency.
  int tiles_per_wave = 1;
  if (mc) {
    tiles_per_wave = tiles >= cus ? 2 : 1;
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
  // 288-512 tiles and a longer reduction: two tiles per workgroup, two k-split waves each (four
  // up to 384 tiles from 20 k steps) -- at most one workgroup per compute unit and one wave per
  // SIMD, the exact fit below without its divisibility -- beat one tile per workgroup with four
  // waves (5120x5120: 5.8 us against 6.2; 6144x8192: 7.7 against 8.3; 5120x14336: 11.0 against
  // 11.5) and one-unit or two-unit waves (7168x8192: 7.8 against 8.7; 6656x11008: 9.9 against
  // 11.3; 7168x14336: 11.8 against 15.3); at 260 tiles they are 1-3 % behind (4160x8192).
  const bool pair_tiles = !mc && tiles * 8 >= cus * 9 && tiles <= 2 * cus && ksteps >= 9;
  if (pair_tiles) {
    split_k = tiles <= cus * 3 / 2 && ksteps >= 20 ? 4 : 2;
  } else if (groups <= cus * 3 / 2) {
    split_k = ksteps < 4 ? ksteps : 4;
    // With workgroups for at most half the compute units, one unit per wave is 4-5 % ahead up to
    // 16 k steps (1024x4096: 3.38 us against 3.54; 1024x8192: 4.54 against 4.77); with a longer
    // reduction it is not (2048x11008: 6.35 at 8 waves against 6.12).
    if (!mc && tiles <= cus / 2 && ksteps <= 16) split_k = ksteps;
    // More than one workgroup per compute unit and 5-8 k steps, one or two rows: four waves would take
    // two units each, the one length at which the two-deep pipeline overlaps nothing; one unit
    // per wave is 6-7 % ahead (4608x4096: 4.81 us against 5.13; 6144x4096: 4.98 against 5.29),
    // while at 256 tiles four waves win (4096x4096: 4.08 against 4.33).
    if (!mc && m_batch <= 2 && tiles > cus && ceil_div(ksteps, 4) == 2) split_k = ksteps;
    if (mc) split_k = ksteps < max_waves ? ksteps : max_waves;  // not pipelined: wants waves
  } else {
    // One or two rows and up to 8 k steps: workgroups of up to 8 one-unit waves stay ahead of two-unit
    // waves well past 8192 waves (22016x4096, 11008 waves: 10.9 us against 11.8; 27200x4096,
    // 13600 waves: 12.6 against 13.0; 36864x2560: 11.8 against 12.3).
    // (int8 weights: the same reductions are twice as many k steps, and with half the arithmetic per byte more,
    // shorter waves stay ahead there as well -- 22016x4096 at 1 / 2 rows 15.6 / 15.5 us with 8 waves per tile against
    // 16.6 / 17.1 with 4; 11008x4096 at 2 rows 8.93 / 9.61; 12288x4096 9.55 / 10.19; 28672x4096 19.1 / 20.2.)
    const bool short_single_row = !mc && m_batch <= 2 && ksteps <= (bits == 8 ? 16 : 8);
    const int kWaveBudget = (short_single_row ? 64 : 32) * cus;
    const int kSimds = cus * 4;
    split_k = ksteps < max_waves ? ksteps : max_waves;
    if (short_single_row && bits == 8 && split_k > 8) split_k = 8;  // 16 one-unit waves lose: 11008x4096, 2 rows, 11.0 us / 8.9
    // One wave per unit does not fit the machine at once, and one wave per tile fills at least
    // 75 % of the SIMDs of its last round: the whole-k waves win (13824x5120: 9.1 us against
    // 10.3 at 5 waves per tile; 27648x5120: 15.6 against 17.5 at 3; 14848x6144: 10.6 against 12.1
    // at 6; 13824x8192: 12.6 against 13.7 at 8).  With a worse fit they lose (17408x5120, 1088
    // tiles: 13.8 against 12.4), and the halving below stands.
    const bool whole_k_waves = !mc && !knobs.wide_waves && m_batch <= 2 && (long long)groups * split_k > kWaveBudget &&
                               (long long)tiles * 100 >= (long long)ceil_div(tiles, kSimds) * kSimds * 75;  // (12432x6144, 76 %: 10.2 us / 11.5)
    if (whole_k_waves) split_k = 1;
    while (split_k > 1 && (long long)groups * split_k > kWaveBudget) split_k = (split_k + 1) / 2;
    if (!mc && !short_single_row && split_k > 1 && ceil_div(ksteps, split_k) < 2 &&
        (long long)groups * ((split_k + 1) / 2) >= 16 * cus)
      split_k = (split_k + 1) / 2;
    // From 16 k steps four waves with longer pipelines are level with or ahead of more, shorter
    // ones (9216x14336: 16.9 us against 18.1 at 7 waves; 10240x11008: 14.8 against 15.3 at 11;
    // 10240x8192 and 11008x8192: level).
    if (!mc && !short_single_row && ksteps >= 16 && split_k > 4) split_k = 4;
    // The bfloat16 kernels are bound by their arithmetic, and two-unit waves are their worst
    // length by far (13824x5120: 18.9 us at 5 waves of 2 units against 14.0 at 2 waves of 5).
    if (knobs.wide_waves && !mc && split_k > 1 && ceil_div(ksteps, split_k) == 2) split_k = (split_k + 1) / 2;
  }
  int tiles_per_wg = pair_tiles ? 2 : 1;
  int workgroup_cap = 0;
  if (!mc && tiles >= cus && ksteps >= 5) {
    // "Exact fit": when the tiles divide (nearly) evenly over the compute units, one workgroup
    // of four waves per compute unit -- one wave per SIMD, all with the same amount of work --
    // beats any over-subscribed launch (8192x8192: 8.7 us against 10.2 us; 28672x8192: 2 %).
    // The four waves are tw tile sequences x 4/tw k-split waves, tw as large as still fits evenly.
    // Walks of more than 7 tiles lose to one tile per workgroup (128256x4096, 8 tiles per wave:
    // 51.5 us against 47.3; 151936x2048, 19 tiles: 31.9 against 29.8), so those are left out.
    // (The bfloat16 kernels want every SIMD busy more than they want equal walks: 28672x8192 takes
    // 35.5 us with one tile and four waves per workgroup against 38.4 with walks of 7 tiles.)
    const int longest_walk = knobs.wide_waves ? 1 : 7;
    for (int tw = 4; tw >= 1; tw /= 2) {
      const int sequences = cus * tw;
      if (ceil_div(tiles, sequences) > longest_walk) continue;
      // The k steps must divide evenly over the 4 / tw waves of a sequence as well, or a SIMD of every compute
      // unit idles (6 k steps on 4 waves are 2 + 2 + 2 + 0): against one workgroup per tile with a wave per k step,
      // 12288x3072 7.09 us / 5.68, 20480x3072 10.10 / 8.79, 28672x3072 12.95 / 11.05, 12288x2560 7.13 / 5.24,
      // 12288x3584 7.18 / 6.24, 12288x5120 9.39 / 8.58; with four k steps or fewer that launch is ahead on every
      // even fit (12288x2048 5.10 / 4.52; 20480x2048 6.78 / 5.93; 28672x2048 8.32 / 7.64; 16384x2048 5.42 / 5.23).
      if (ksteps % (4 / tw) != 0) continue;
      // ... and with up to 8 k steps a single tile sequence of four k-split waves (two units a wave, then the next
      // tile) is behind a workgroup of one-unit waves per tile: 12288x4096 6.6 us / 7.3; 20480x4096 9.8 / 10.4; 20048x3840
      // 10.0 / 11.0; 28672x4096 level (two or four sequences side by side stay: 16384x4096 8.0 / 9.0; 24576x3072 9.5 / 10.1)
      if (ksteps <= 8 && tw == 1) continue;
      if ((long long)ceil_div(tiles, sequences) * sequences * 100 <= (long long)tiles * 103) {
        tiles_per_wg = tw;
        split_k = 4 / tw;
        workgroup_cap = cus;
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
  LaunchPlan lp{};
  lp.split_k = split_k;
  lp.tiles_per_wg = tiles_per_wg;
  lp.steps_per_wave = steps;
  lp.workgroups = ceil_div(groups, tiles_per_wg);
  lp.tiles_in_sequence = 1;
  lp.staged_rows = 0;
  lp.matrix_core = mc;
  lp.stages = !mc && knobs.stages == 1 ? 1 : 2;
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
  if (k % 8) return MGEMV_ERR_COLS;  // utils/preprocess.h:324-327
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

// What a plan asks of the hardware: dynamic LDS of its (largest) launch, the workgroup size limit the
// kernel it picks was compiled for, and how many launches serve all activation rows.
struct LaunchResources {
  size_t lds_bytes;
  int max_threads;
  int launches;
};
LaunchResources launch_resources(const LaunchPlan& lp, int bits, int m_batch, int act) {
  LaunchResources r{};
  r.launches = 1;
  if (lp.matrix_core && lp.k_stationary) {
    r.max_threads = kWave * kMaxWavesPerWorkgroup;
    const size_t stage = (size_t)lp.split_k * 8 * (step_k(bits) * 2 + 16), park = (size_t)lp.tiles_in_sequence * kKSlices * m_batch * kKStationaryParkSlots * 16;
    // both when they fit (then no barrier stands between a wave's operand and its walk), else the larger of the two
    r.lds_bytes = stage + park <= (size_t)kMaxKStationaryLds ? stage + park : stage > park ? stage : park;
    return r;
  }
  if (lp.matrix_core) {
    r.max_threads = kWave * kMaxWavesPerMfmaWorkgroup;
    if (lp.staged_rows != 0) {
      const int row_stride = step_k(bits) * 2 + 16;
      r.lds_bytes = (size_t)lp.split_k * 2 * lp.staged_rows * row_stride +
                    (lp.split_k > 1 ? (size_t)lp.tiles_per_wg * lp.split_k * kWave * 4 * sizeof(float) : 0);
    } else {
      r.lds_bytes = lp.split_k == 1 ? 0 : (size_t)lp.tiles_per_wg * lp.split_k * lp.tiles_per_wave * kWave * 4 * sizeof(float);
    }
    return r;
  }
  const int rows = m_batch < kMaxValuBatch ? m_batch : kMaxValuBatch;
  r.launches = (m_batch + kMaxValuBatch - 1) / kMaxValuBatch;
  r.max_threads = kWave * (rows >= 3 || act == kActBf16 ? kMaxWavesPerWideWorkgroup : kMaxWavesPerWorkgroup);
  r.lds_bytes = (size_t)lp.tiles_in_sequence * lp.tiles_per_wg * lp.split_k * rows * kWave * sizeof(float);
  return r;
}

hipError_t launch_gemv(const GemvLaunch& g, int bits, int qop, int mb, int gpr, int act) {
  return act == kActBf16 ? launch_gemv_bf16(g, bits, qop, mb, gpr) : launch_gemv_f16(g, bits, qop, mb, gpr);
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

// What the launch path needs to know about a device, looked up once per device and process
// (the first launch on a device pays for one hipGetDeviceProperties call).
struct DeviceInfo {
  bool usable;   // a gfx950 device
  int num_cus;
};
constexpr int kMaxDevices = 64;
std::atomic<int> g_device_state[kMaxDevices];  // 0 unknown, else 1 + (usable ? num_cus : 0)

// The device a stream belongs to (the null stream: the calling thread's current device).
int device_of_stream(hipStream_t stream, int& device) {
  if (stream != nullptr && hipStreamGetDevice(stream, &device) == hipSuccess) return MGEMV_OK;
  return hipGetDevice(&device) == hipSuccess ? MGEMV_OK : MGEMV_ERR_NO_DEVICE;
}

int device_info(int device, DeviceInfo& info) {
  const bool tracked = device >= 0 && device < kMaxDevices;
  int state = tracked ? g_device_state[device].load(std::memory_order_relaxed) : 0;
  if (state == 0) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return MGEMV_ERR_NO_DEVICE;
    const bool usable = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    state = 1 + (usable ? prop.multiProcessorCount : 0);
    if (tracked) g_device_state[device].store(state, std::memory_order_relaxed);
  }
  info.usable = state > 1;
  info.num_cus = state - 1;
  return info.usable ? MGEMV_OK : MGEMV_ERR_NO_DEVICE;
}

// The knobs of a problem with the element type taken into account.
PlanKnobs knobs_for_element(int n_out, int k, int bits, int group_size, int m_batch, int act, int num_cus = kNumCus) {
  PlanKnobs knobs = knobs_for(n_out, k, bits, group_size, m_batch, act, num_cus);
  knobs.num_cus = num_cus;
  // (a group as long as k is the per-column mode, whose kernels look one scale up per row)
  knobs.generic_groups = group_size > 0 && group_size != k && groups_per_run(group_size, bits) == 4;
  if (act == kActBf16) {
    // bf16: of the matrix-core kernels only the LDS-staged one (needs two tiles); the VALU kernel's
    // fp32 dequantiser wants the registers of 8-wave workgroups
    if (num_tiles(n_out) < 2) knobs.matrix_core_min_batch = MGEMV_MAX_M_BATCH + 1;
    knobs.matrix_core_variant = MGEMV_MATRIX_CORE_LDS_STAGED;
    knobs.wide_waves = true;
  }
  return knobs;
}

// act: kActF16 or kActBf16, the type behind every 16-bit operand.
int gemv_any(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
             const uint16_t* bias, uint16_t* y, int batch_count, int n_out, int m_batch, int k, int group_size,
             int quant_op, int weight_bits, int64_t stride_weights, int64_t stride_x, int64_t stride_scale,
             int64_t stride_bias, int64_t stride_y, void* stream, int act, float alpha = 1.0f, float beta = 1.0f,
             int probe = kProbeNone, unsigned long long* trace = nullptr, size_t trace_capacity_waves = 0,
             bool timed_waits = false, const int32_t* route = nullptr, int route_extent = 0) {
  if (batch_count < 1 || batch_count > 65535) return MGEMV_ERR_BATCH;
  if (route != nullptr && route_extent < 1) return MGEMV_ERR_BATCH;
  if (reinterpret_cast<uintptr_t>(route) % 4) return MGEMV_ERR_ALIGNMENT;
  if (m_batch < 1 || m_batch > MGEMV_MAX_M_BATCH) return MGEMV_ERR_BATCH;
  if (const int st = check_problem(weights, scale, zero_add, n_out, k, group_size, quant_op, weight_bits)) return st;
  if (x == nullptr || y == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (reinterpret_cast<uintptr_t>(x) % 16 || reinterpret_cast<uintptr_t>(y) % 2 ||
      reinterpret_cast<uintptr_t>(bias) % 2)
    return MGEMV_ERR_ALIGNMENT;
  if (stride_weights % 16 || stride_x % 8) return MGEMV_ERR_ALIGNMENT;
  int device = 0;
  if (const int st = device_of_stream(static_cast<hipStream_t>(stream), device)) return st;
  DeviceInfo info{};
  if (const int st = device_info(device, info)) return st;

  GemvLaunch g{};
  g.device = device;
  g.weights = static_cast<const uint8_t*>(weights);
  g.scale = reinterpret_cast<const half_t*>(scale);
  g.zero_add = quant_op == MGEMV_FINEGRAINED_SCALE_AND_ZEROS ? reinterpret_cast<const half_t*>(zero_add) : nullptr;
  g.n_out = n_out;
  g.k = k;
  g.group_size = group_size;
  g.plan = plan_launch(n_out, k, weight_bits, m_batch,
                       knobs_for_element(n_out, k, weight_bits, group_size, m_batch, act, info.num_cus));
  g.tail.bias = reinterpret_cast<const half_t*>(bias);
  g.tail.split_k = g.plan.split_k;
  g.tail.num_groups = k / group_size;
  g.tail.flags = g_dequant_flags.load() | (g.plan.stages == 1 ? kSingleStage : 0) | (timed_waits ? kTimelineWaits : 0);
  g.tail.alpha = alpha;
  g.tail.beta = beta;
  g.tail.trace = trace;
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
  g.tail.route = route;
  g.tail.route_extent = route_extent;
  g.grid = dim3((unsigned)(g.plan.wgs_per_xcd * kNumXcd), 1, (unsigned)batch_count);
  g.block = dim3((unsigned)(kWave * g.plan.split_k), (unsigned)g.plan.tiles_per_wg, 1);
  g.stream = static_cast<hipStream_t>(stream);
  const int gpr = groups_per_run(group_size, weight_bits);

  if (g.plan.matrix_core) {
    g.x = reinterpret_cast<const half_t*>(x);
    g.tail.y = reinterpret_cast<half_t*>(y);
    g.tail.m_batch = m_batch;
    g.lds = launch_resources(g.plan, weight_bits, m_batch, act).lds_bytes;
    if (g.plan.k_stationary) {
      const size_t stage = (size_t)g.plan.split_k * 8 * (step_k(weight_bits) * 2 + 16);
      if (g.lds > stage && g.lds - stage >= (size_t)g.plan.tiles_in_sequence * kKSlices * m_batch * kKStationaryParkSlots * 16)
        g.tail.flags |= kParkBehindStage;
      if (probe != kProbeNone) {
        if (probe == kProbeTimeline || !mfma_kstat_probe_exists(weight_bits, quant_op, gpr, act)) return MGEMV_ERR_QUANT_OP;
        return launch_mfma_kstat_probe(g, gpr, probe) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
      }
      return launch_mfma_kstat(g, weight_bits, quant_op, gpr, act) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
    }
    if (probe != kProbeNone) {
      const int rounds = g.plan.staged_rows != 0 ? g.plan.staged_rows / g.plan.tiles_per_wg : 0;
      if (probe == kProbeTimeline || rounds == 0 ||
          !mfma_lds_probe_exists(weight_bits, quant_op, gpr, rounds, act, g.plan.tiles_per_wg))
        return MGEMV_ERR_QUANT_OP;
      return launch_mfma_lds_probe(g, gpr, rounds, probe) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
    }
    if (g.plan.staged_rows != 0) {
      return launch_mfma_lds(g, weight_bits, quant_op, gpr, g.plan.staged_rows / g.plan.tiles_per_wg, act) == hipSuccess
                 ? MGEMV_OK
                 : MGEMV_ERR_LAUNCH;
    }
    return launch_mfma(g, weight_bits, quant_op, gpr) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
  }
  if (probe != kProbeNone) {
    // measurement builds exist for the headline kernel only: int4, scale and zero, one group per run, one row, fp16
    if (weight_bits != 4 || quant_op != MGEMV_FINEGRAINED_SCALE_AND_ZEROS || gpr != 1 || m_batch != 1 || act != kActF16)
      return MGEMV_ERR_QUANT_OP;
    g.x = reinterpret_cast<const half_t*>(x);
    g.tail.y = reinterpret_cast<half_t*>(y);
    g.lds = (size_t)g.plan.tiles_in_sequence * g.plan.tiles_per_wg * g.plan.split_k * kWave * sizeof(float);
    // every launched wave writes its own row of the trace: the caller's buffer must hold them all
    if (probe == kProbeTimeline &&
        (size_t)g.grid.x * (size_t)(g.plan.split_k * g.plan.tiles_per_wg) > trace_capacity_waves)
      return MGEMV_ERR_SIZE;
    return launch_gemv_probe(g, probe) == hipSuccess ? MGEMV_OK : MGEMV_ERR_LAUNCH;
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
  int device = 0;
  if (const int st = device_of_stream(static_cast<hipStream_t>(stream), device)) return st;
  DeviceInfo info{};
  if (const int st = device_info(device, info)) return st;
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

int mgemv_gemv_routed(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
                      const uint16_t* bias, uint16_t* y, const int32_t* route, int route_extent, int batch_count,
                      int n_out, int m_batch, int k, int group_size, int quant_op, int weight_bits,
                      int64_t stride_weights, int64_t stride_x, int64_t stride_scale, int64_t stride_bias,
                      int64_t stride_y, void* stream) {
  if (route == nullptr) return MGEMV_ERR_NULL_POINTER;
  return mgemv::gemv_any(weights, x, scale, zero_add, bias, y, batch_count, n_out, m_batch, k, group_size, quant_op,
                         weight_bits, stride_weights, stride_x, stride_scale, stride_bias, stride_y, stream,
                         mgemv::kActF16, 1.0f, 1.0f, mgemv::kProbeNone, nullptr, 0, false, route, route_extent);
}

int mgemv_gemv_routed_bf16(const void* weights, const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add,
                           const uint16_t* bias, uint16_t* y, const int32_t* route, int route_extent, int batch_count,
                           int n_out, int m_batch, int k, int group_size, int quant_op, int weight_bits,
                           int64_t stride_weights, int64_t stride_x, int64_t stride_scale, int64_t stride_bias,
                           int64_t stride_y, void* stream) {
  if (route == nullptr) return MGEMV_ERR_NULL_POINTER;
  return mgemv::gemv_any(weights, x, scale, zero_add, bias, y, batch_count, n_out, m_batch, k, group_size, quant_op,
                         weight_bits, stride_weights, stride_x, stride_scale, stride_bias, stride_y, stream,
                         mgemv::kActBf16, 1.0f, 1.0f, mgemv::kProbeNone, nullptr, 0, false, route, route_extent);
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

namespace {
int probe_kind(int kind) {
  return kind == MGEMV_PROBE_LOADS_ONLY     ? mgemv::kProbeLoadsOnly
         : kind == MGEMV_PROBE_COMPUTE_ONLY ? mgemv::kProbeComputeOnly
                                            : mgemv::kProbeTimeline;   // with or without the per-unit waits
}
}  // namespace

int mgemv_probe_gemv_rows(int kind, int m_batch, const void* weights, const uint16_t* x, const uint16_t* scale,
                          const uint16_t* zero_add, uint16_t* y, int n_out, int k, int group_size, void* stream) {
  if (kind != MGEMV_PROBE_LOADS_ONLY && kind != MGEMV_PROBE_COMPUTE_ONLY) return MGEMV_ERR_SIZE;
  return mgemv::gemv_any(weights, x, scale, zero_add, nullptr, y, 1, n_out, m_batch, k, group_size,
                         MGEMV_FINEGRAINED_SCALE_AND_ZEROS, 4, 0, 0, 0, 0, 0, stream, mgemv::kActF16, 1.0f, 1.0f,
                         probe_kind(kind), nullptr);
}

int mgemv_probe_gemv(int kind, unsigned long long* trace, size_t trace_capacity_waves, const void* weights,
                     const uint16_t* x, const uint16_t* scale, const uint16_t* zero_add, uint16_t* y, int n_out, int k,
                     int group_size, void* stream) {
  if (kind != MGEMV_PROBE_LOADS_ONLY && kind != MGEMV_PROBE_TIMELINE && kind != MGEMV_PROBE_COMPUTE_ONLY &&
      kind != MGEMV_PROBE_TIMELINE_WAITS)
    return MGEMV_ERR_SIZE;
  if ((kind == MGEMV_PROBE_TIMELINE || kind == MGEMV_PROBE_TIMELINE_WAITS) && (trace == nullptr || reinterpret_cast<uintptr_t>(trace) % 8)) return MGEMV_ERR_NULL_POINTER;
  return mgemv::gemv_any(weights, x, scale, zero_add, nullptr, y, 1, n_out, 1, k, group_size,
                         MGEMV_FINEGRAINED_SCALE_AND_ZEROS, 4, 0, 0, 0, 0, 0, stream, mgemv::kActF16, 1.0f, 1.0f,
                         probe_kind(kind), trace, trace_capacity_waves, kind == MGEMV_PROBE_TIMELINE_WAITS);
}

// gemv/device/gemv_adaptor.h:114-178 as one plain struct.
int mgemv_gemv_arguments(const mgemv_arguments* a, void* stream) {
  if (a == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (a->element != MGEMV_ELEMENT_F16 && a->element != MGEMV_ELEMENT_BF16) return MGEMV_ERR_QUANT_TYPE;
  // The operands are the reference's dense ones; a leading dimension may repeat what the reference
  // passes (mixed_gemv_test.cu:136-140, 153-154) or be 0 = "dense", nothing else.
  const int64_t n = a->n_out, k = a->k;
  if (a->lda != 0 && a->lda != 4 * k && a->lda != k) return MGEMV_ERR_LEADING_DIMENSION;
  if (a->ldb != k && !(a->ldb == 0 && a->m_batch == 1)) return MGEMV_ERR_LEADING_DIMENSION;
  if (a->ld_scale != 0 && a->ld_scale != n) return MGEMV_ERR_LEADING_DIMENSION;
  if (a->ld_zero != 0 && a->ld_zero != n) return MGEMV_ERR_LEADING_DIMENSION;
  if (a->ldc != 0 && a->ldc != n) return MGEMV_ERR_LEADING_DIMENSION;
  if (a->ldd != 0 && a->ldd != n) return MGEMV_ERR_LEADING_DIMENSION;
  return mgemv::gemv_any(a->weights, a->x, a->scale, a->zero_add, a->bias, a->y, a->batch_count, a->n_out,
                         a->m_batch, a->k, a->group_size, a->quant_op, a->weight_bits, a->batch_stride_weights,
                         a->batch_stride_x, a->batch_stride_scale, a->batch_stride_bias, a->batch_stride_y, stream,
                         a->element == MGEMV_ELEMENT_BF16 ? mgemv::kActBf16 : mgemv::kActF16, a->alpha, a->beta);
}

// host/mixed_gemv.h:60-70 on the GPU: un-preprocessed weights and int8 zero points in host
// memory in, result in host memory out.  Both entry points below share everything but where their
// staging memory comes from.
namespace {

struct HostGemvLayout {
  size_t tiled_bytes, table, off_w, off_x, off_s, off_z, off_b, off_y, total;
  bool has_zero;
};

int host_gemv_layout(int batch, int n_out, int m_batch, int k, int& group_size, const void* weights, const void* x,
                     const void* scale, const void* zero_point, const void* y, bool has_bias, int quant_op, int weight_bits,
                     HostGemvLayout& l) {
  if (batch != 1) return MGEMV_ERR_BATCH;  // host/mixed_gemv.h:77-80
  if (m_batch < 1 || m_batch > MGEMV_MAX_M_BATCH) return MGEMV_ERR_BATCH;
  if (weights == nullptr || x == nullptr || scale == nullptr || y == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (quant_op != MGEMV_PER_COLUMN_SCALE_ONLY && quant_op != MGEMV_FINEGRAINED_SCALE_ONLY &&
      quant_op != MGEMV_FINEGRAINED_SCALE_AND_ZEROS)
    return MGEMV_ERR_QUANT_OP;
  if (weight_bits != 4 && weight_bits != 8) return MGEMV_ERR_QUANT_TYPE;
  l.has_zero = quant_op == MGEMV_FINEGRAINED_SCALE_AND_ZEROS;
  if (l.has_zero && zero_point == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (n_out <= 0 || k <= 0) return MGEMV_ERR_SIZE;
  if (quant_op == MGEMV_PER_COLUMN_SCALE_ONLY) group_size = k;
  if (group_size <= 0 || k % group_size) return MGEMV_ERR_GROUP_SIZE;
  if (n_out % 4) return MGEMV_ERR_ROWS;  // what the preprocessor would refuse (utils/preprocess.h:319-327),
  if (k % 8) return MGEMV_ERR_COLS;      // before any memory is touched
  l.table = (size_t)(k / group_size) * (size_t)n_out;
  const size_t shape[2] = {(size_t)k, (size_t)n_out};
  l.tiled_bytes = mgemv_preprocessed_size(shape, 2, weight_bits == 4 ? MGEMV_W4_A16 : MGEMV_W8_A16);
  // one piece of memory, 256-byte aligned parts
  auto align = [](size_t v) { return (v + 255) / 256 * 256; };
  l.off_w = 0;
  l.off_x = l.off_w + align(l.tiled_bytes);
  l.off_s = l.off_x + align((size_t)m_batch * k * 2);
  l.off_z = l.off_s + align(l.table * 2);
  l.off_b = l.off_z + align(l.has_zero ? l.table * 2 : 0);
  l.off_y = l.off_b + align(has_bias ? (size_t)n_out * 2 : 0);
  l.total = l.off_y + align((size_t)m_batch * n_out * 2);
  return MGEMV_OK;
}

// dev: device staging of l.total bytes; host_stage: host memory laid out the same way, of which the
// weight and zero parts are used.
int host_gemv_staged(const HostGemvLayout& l, uint8_t* dev, uint8_t* host_stage, int n_out, int m_batch, int k,
                     int group_size, const uint8_t* weights, const uint16_t* x, const uint16_t* scale,
                     const int8_t* zero_point, const uint16_t* bias, uint16_t* y, int quant_op, int weight_bits) {
  const size_t shape[2] = {(size_t)k, (size_t)n_out};
  const int quant_type = weight_bits == 4 ? MGEMV_W4_A16 : MGEMV_W8_A16;
  uint8_t* const tiled = host_stage + l.off_w;
  if (const int st = mgemv_preprocess_weights(tiled, weights, shape, 2, MGEMV_COLUMN_MAJOR, quant_type)) return st;
  uint16_t* const zero_add = reinterpret_cast<uint16_t*>(host_stage + l.off_z);
  if (l.has_zero) {
    if (const int st = mgemv_fold_zero_points(zero_add, scale, zero_point, l.table)) return st;  // utils/preprocess.h:94-101
  }
  int st = MGEMV_OK;
  auto up = [&](size_t off, const void* src, size_t bytes) {
    if (st == MGEMV_OK && bytes && hipMemcpy(dev + off, src, bytes, hipMemcpyHostToDevice) != hipSuccess) st = MGEMV_ERR_LAUNCH;
  };
  up(l.off_w, tiled, l.tiled_bytes);
  up(l.off_x, x, (size_t)m_batch * k * 2);
  up(l.off_s, scale, l.table * 2);
  if (l.has_zero) up(l.off_z, zero_add, l.table * 2);
  if (bias) up(l.off_b, bias, (size_t)n_out * 2);
  if (st == MGEMV_OK)
    st = mgemv_gemv(dev + l.off_w, reinterpret_cast<const uint16_t*>(dev + l.off_x),
                    reinterpret_cast<const uint16_t*>(dev + l.off_s),
                    l.has_zero ? reinterpret_cast<const uint16_t*>(dev + l.off_z) : nullptr,
                    bias ? reinterpret_cast<const uint16_t*>(dev + l.off_b) : nullptr,
                    reinterpret_cast<uint16_t*>(dev + l.off_y), n_out, m_batch, k, group_size, quant_op, weight_bits, nullptr);
  // the blocking copy on the null stream is ordered behind the kernel
  if (st == MGEMV_OK && hipMemcpy(y, dev + l.off_y, (size_t)m_batch * n_out * 2, hipMemcpyDeviceToHost) != hipSuccess)
    st = MGEMV_ERR_LAUNCH;
  return st;
}

}  // namespace

int mgemv_host_gemv(int batch, int n_out, int m_batch, int k, int group_size, const uint8_t* weights,
                    const uint16_t* x, const uint16_t* scale, const int8_t* zero_point, const uint16_t* bias,
                    uint16_t* y, int quant_op, int weight_bits) {
  HostGemvLayout l{};
  if (const int st = host_gemv_layout(batch, n_out, m_batch, k, group_size, weights, x, scale, zero_point, y,
                                      bias != nullptr, quant_op, weight_bits, l))
    return st;
  std::vector<uint8_t> host_stage(l.off_b);  // the weight and zero parts are what the host side fills
  uint8_t* dev = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&dev), l.total) != hipSuccess) return MGEMV_ERR_ALLOCATION;
  const int st = host_gemv_staged(l, dev, host_stage.data(), n_out, m_batch, k, group_size, weights, x, scale, zero_point,
                                  bias, y, quant_op, weight_bits);
  (void)hipFree(dev);
  return st;
}

// The allocation-free variant: the same staging in a static device array (one copy per GPU, at
// its own address there) and a static host array.  The array's name is a host-side handle, not a
// device address: host code only ever uses the pointer hipGetSymbolAddress returned for the
// device at hand.
static __device__ __align__(256) unsigned char scratch[MGEMV_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxScratchDevices = 64;
alignas(256) unsigned char g_static_host_stage[MGEMV_STATIC_SCRATCH_BYTES];
unsigned char* g_scratch_of_device[kMaxScratchDevices];  // what hipGetSymbolAddress gave, per device
std::mutex g_static_mutex;                               // one call at a time: the arrays are shared

// The address of `scratch` on the current device (looked up once per device, with it current).
int static_scratch_of_current_device(unsigned char*& ptr) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return MGEMV_ERR_NO_DEVICE;
  if (device < 0 || device >= kMaxScratchDevices) return MGEMV_ERR_NO_DEVICE;
  if (g_scratch_of_device[device] == nullptr) {
    mgemv::DeviceInfo info{};
    if (const int st = mgemv::device_info(device, info)) return st;  // gfx950 only: other devices hold no copy of the array
    unsigned char* p = nullptr;
    if (hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr)
      return MGEMV_ERR_NO_DEVICE;
    g_scratch_of_device[device] = p;
  }
  ptr = g_scratch_of_device[device];
  return MGEMV_OK;
}
}  // namespace

size_t mgemv_static_scratch_bytes_needed(int n_out, int m_batch, int k, int group_size, int quant_op, int weight_bits,
                                         int has_bias) {
  HostGemvLayout l{};
  static const int dummy = 0;  // the layout only asks whether the pointers are there
  if (host_gemv_layout(1, n_out, m_batch, k, group_size, &dummy, &dummy, &dummy, &dummy, &dummy, has_bias != 0, quant_op,
                       weight_bits, l))
    return 0;
  return l.total;
}

int mgemv_host_gemv_static(int batch, int n_out, int m_batch, int k, int group_size, const uint8_t* weights,
                           const uint16_t* x, const uint16_t* scale, const int8_t* zero_point, const uint16_t* bias,
                           uint16_t* y, int quant_op, int weight_bits) {
  HostGemvLayout l{};
  if (const int st = host_gemv_layout(batch, n_out, m_batch, k, group_size, weights, x, scale, zero_point, y,
                                      bias != nullptr, quant_op, weight_bits, l))
    return st;
  if (l.total > MGEMV_STATIC_SCRATCH_BYTES) return MGEMV_ERR_SCRATCH_SIZE;
  std::lock_guard<std::mutex> lock(g_static_mutex);
  unsigned char* dev = nullptr;
  if (const int st = static_scratch_of_current_device(dev)) return st;
  return host_gemv_staged(l, dev, g_static_host_stage, n_out, m_batch, k, group_size, weights, x, scale, zero_point, bias, y,
                          quant_op, weight_bits);
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
      variant != MGEMV_MATRIX_CORE_LDS_STAGED && variant != MGEMV_MATRIX_CORE_K_STATIONARY)
    return MGEMV_ERR_SIZE;
  mgemv::g_matrix_core_variant.store(variant);
  return MGEMV_OK;
}

int mgemv_set_prefetch_stages(int stages) {
  if (stages < 0 || stages > 2) return MGEMV_ERR_SIZE;
  mgemv::g_override_stages.store(stages);
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
  if (plan->stages < 0 || plan->stages > 2) return MGEMV_ERR_SIZE;
  if (plan->element != MGEMV_ELEMENT_F16 && plan->element != MGEMV_ELEMENT_BF16) return MGEMV_ERR_QUANT_TYPE;
  const int t = plan->tiles_per_wave;
  if (t != 0 && t != 1 && t != 2 && t != 4) return MGEMV_ERR_SIZE;
  if (plan->kernel < MGEMV_KERNEL_AUTO || plan->kernel > MGEMV_KERNEL_MATRIX_CORE_K_STATIONARY) return MGEMV_ERR_SIZE;
  const mgemv::PlanKnobs kn = mgemv::knobs_of_plan(*plan);
  std::lock_guard<std::mutex> lock(mgemv::g_tuned_mutex);
  mgemv::g_tuned_plans[mgemv::PlanKey{plan->n_out, plan->k, plan->weight_bits, plan->group_size, plan->m_batch,
                                      plan->element}] = kn;
  mgemv::g_tuned_count.store((int)mgemv::g_tuned_plans.size());
  return MGEMV_OK;
}

int mgemv_tuned_plan_erase(const mgemv_tuned_plan* plan) {
  if (plan == nullptr) return MGEMV_ERR_NULL_POINTER;
  std::lock_guard<std::mutex> lock(mgemv::g_tuned_mutex);
  mgemv::g_tuned_plans.erase(
      mgemv::PlanKey{plan->n_out, plan->k, plan->weight_bits, plan->group_size, plan->m_batch, plan->element});
  mgemv::g_tuned_count.store((int)mgemv::g_tuned_plans.size());
  return MGEMV_OK;
}

int mgemv_set_default_plans(int enable) {
  mgemv::g_default_plans_enabled.store(enable != 0 ? 1 : 0);
  return MGEMV_OK;
}

int mgemv_default_plan_count(void) { return mgemv::default_plan_count(); }

int mgemv_tuned_plan_clear(void) {
  std::lock_guard<std::mutex> lock(mgemv::g_tuned_mutex);
  mgemv::g_tuned_plans.clear();
  mgemv::g_tuned_count.store(0);
  return MGEMV_OK;
}

int mgemv_tuned_plan_count(void) { return mgemv::g_tuned_count.load(); }

namespace {
int query_launch_any(int n_out, int m_batch, int k, int weight_bits, int group_size, int act, int out[8],
                     int num_cus = mgemv::kNumCus);
}

int mgemv_query_launch_for(int n_out, int m_batch, int k, int weight_bits, int group_size, int element,
                           int num_compute_units, int out[12]) {
  if (element != MGEMV_ELEMENT_F16 && element != MGEMV_ELEMENT_BF16) return MGEMV_ERR_QUANT_TYPE;
  if (num_compute_units < 1 || num_compute_units > 4096) return MGEMV_ERR_SIZE;
  const int act = element == MGEMV_ELEMENT_BF16 ? mgemv::kActBf16 : mgemv::kActF16;
  if (const int st = query_launch_any(n_out, m_batch, k, weight_bits, group_size, act, out, num_compute_units)) return st;
  const mgemv::LaunchPlan lp = mgemv::plan_launch(
      n_out, k, weight_bits, m_batch, mgemv::knobs_for_element(n_out, k, weight_bits, group_size, m_batch, act, num_compute_units));
  const mgemv::LaunchResources r = mgemv::launch_resources(lp, weight_bits, m_batch, act);
  out[8] = (int)r.lds_bytes;
  out[9] = r.max_threads;
  out[10] = lp.stages;
  out[11] = r.launches;
  return MGEMV_OK;
}

int mgemv_plan_coverage(int n_out, int m_batch, int k, int weight_bits, int group_size, int element,
                        int num_compute_units, int64_t out[8]) {
  using namespace mgemv;
  if (out == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (element != MGEMV_ELEMENT_F16 && element != MGEMV_ELEMENT_BF16) return MGEMV_ERR_QUANT_TYPE;
  if (num_compute_units < 1 || num_compute_units > 4096) return MGEMV_ERR_SIZE;
  if (const int st = check_tuned_key(n_out, k, weight_bits, group_size, m_batch)) return st;
  const int act = element == MGEMV_ELEMENT_BF16 ? kActBf16 : kActF16;
  const LaunchPlan lp = plan_launch(n_out, k, weight_bits, m_batch,
                                    knobs_for_element(n_out, k, weight_bits, group_size, m_batch, act, num_compute_units));
  const LaunchResources res = launch_resources(lp, weight_bits, m_batch, act);
  const int tiles = num_tiles(n_out), ksteps = num_ksteps(k, weight_bits);
  const int grid = lp.wgs_per_xcd * kNumXcd;
  const int sequences = lp.workgroups * lp.tiles_per_wg;
  const int seq_base = tiles / sequences, seq_rem = tiles % sequences;  // as gemv_any passes them
  const bool multi = (!lp.matrix_core || lp.k_stationary) && lp.tiles_in_sequence > 1;
  const int rows = m_batch < kMaxValuBatch ? m_batch : kMaxValuBatch;
  std::vector<int> covered((size_t)tiles, 0);
  std::vector<char> block_seen((size_t)lp.workgroups, 0);
  int64_t idle_waves = 0, busy_waves = 0, max_span = 0, max_lds = 0, bad_ranges = 0, max_units = 0;
  for (int block = 0; block < grid; ++block) {
    const int wg = logical_workgroup_of(block, lp.wgs_per_xcd);
    if (wg >= lp.workgroups) continue;  // the kernels leave at this test
    if (block_seen[(size_t)wg]++) ++bad_ranges;   // two blocks with one logical id
    for (int ty = 0; ty < lp.tiles_per_wg; ++ty) {
      for (int kw = 0; kw < lp.split_k; ++kw) {
        const WaveWork w = lp.matrix_core && !lp.k_stationary
                               ? (lp.staged_rows != 0
                                      ? staged_wave_work(wg, ty, kw, lp.tiles_per_wg, tiles, lp.steps_per_wave, ksteps)
                                      : mfma_wave_work(lp.tiles_per_wave, wg, ty, kw, lp.tiles_per_wg, tiles,
                                                       lp.steps_per_wave, ksteps))
                               : valu_wave_work(multi, wg, ty, kw, lp.tiles_per_wg, seq_base, seq_rem, tiles,
                                                lp.steps_per_wave, ksteps);
        if (w.units <= 0) ++bad_ranges;  // every kernel relies on each wave along k having units
        if (w.tiles <= 0 || w.units <= 0) {
          ++idle_waves;
          continue;
        }
        ++busy_waves;
        if (w.tile_begin < 0 || w.tile_begin + w.tiles > tiles || w.ks_begin < 0 || w.ks_begin + w.units > ksteps) {
          ++bad_ranges;
          continue;
        }
        for (int t = 0; t < w.tiles; ++t) covered[(size_t)(w.tile_begin + t)] += w.units;
        // the bytes one weight descriptor spans: tiles are ksteps units apart
        const int64_t span = (int64_t)(w.tiles - 1) * ksteps * kUnitBytes + (int64_t)w.units * kUnitBytes;
        max_span = span > max_span ? span : max_span;
        const int64_t walk_units = (int64_t)w.tiles * w.units;
        max_units = walk_units > max_units ? walk_units : max_units;
        if (!lp.matrix_core) {
          // last float this wave parks for the combine (tile t of its walk at t * park_stride)
          const int64_t park_stride = (int64_t)lp.tiles_per_wg * lp.split_k * rows * kWave;
          const int64_t last = (int64_t)(multi ? w.tiles - 1 : 0) * park_stride +
                               ((int64_t)(ty * lp.split_k + kw) * rows + (rows - 1)) * kWave + (kWave - 1);
          max_lds = (last + 1) * 4 > max_lds ? (last + 1) * 4 : max_lds;
        }
      }
    }
  }
  int64_t wrong = 0;
  for (int t = 0; t < tiles; ++t) wrong += covered[(size_t)t] != ksteps;
  out[0] = wrong;                 // tiles whose k steps are not covered exactly once
  out[1] = bad_ranges;            // waves with a range outside the problem or without units, duplicate workgroup ids
  out[2] = max_span;              // most bytes behind one weight descriptor
  out[3] = max_lds;               // VALU kernel: bytes of LDS up to the last parked partial sum
  out[4] = (int64_t)res.lds_bytes;
  out[5] = busy_waves;
  out[6] = idle_waves;
  out[7] = max_units;             // most units any wave computes
  return MGEMV_OK;
}

int mgemv_query_launch(int n_out, int m_batch, int k, int weight_bits, int group_size, int out[8]) {
  return query_launch_any(n_out, m_batch, k, weight_bits, group_size, mgemv::kActF16, out);
}

int mgemv_query_launch_bf16(int n_out, int m_batch, int k, int weight_bits, int group_size, int out[8]) {
  return query_launch_any(n_out, m_batch, k, weight_bits, group_size, mgemv::kActBf16, out);
}

namespace {
int query_launch_any(int n_out, int m_batch, int k, int weight_bits, int group_size, int act, int out[8], int num_cus) {
  if (out == nullptr) return MGEMV_ERR_NULL_POINTER;
  const int st = check_tuned_key(n_out, k, weight_bits, group_size, m_batch);
  if (st != MGEMV_OK) return st;
  const mgemv::LaunchPlan lp = mgemv::plan_launch(
      n_out, k, weight_bits, m_batch, mgemv::knobs_for_element(n_out, k, weight_bits, group_size, m_batch, act, num_cus));
  out[0] = lp.wgs_per_xcd * mgemv::kNumXcd;
  out[1] = lp.threads;
  out[2] = lp.split_k;
  out[3] = lp.tiles_per_wg;
  out[4] = lp.steps_per_wave;
  out[5] = !lp.matrix_core ? 0 : lp.k_stationary ? 3 : lp.staged_rows != 0 ? 2 : 1;
  out[6] = lp.tiles_per_wave;
  out[7] = lp.tiles_in_sequence;
  return MGEMV_OK;
}
}  // namespace

}  // extern "C"
