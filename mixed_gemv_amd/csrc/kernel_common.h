// Shared by the kernels of this library and their launchers: launch constants, the kernel
// argument block, small device helpers, and the host-side description of a launch.
#ifndef MIXED_GEMV_AMD_KERNEL_COMMON_H_
#define MIXED_GEMV_AMD_KERNEL_COMMON_H_

#include <hip/hip_runtime.h>

#include "device_math.h"
#include "mixed_gemv.h"
#include "mixed_gemv_probes.h"
#include "tile_layout.h"

namespace mgemv {

constexpr int kWave = 64;
constexpr int kMaxWavesPerWorkgroup = 16;
constexpr int kMaxWavesPerWideWorkgroup = 8;  // VALU kernel with 3-4 activation rows: 256 VGPRs per wave
constexpr int kMaxWavesPerMfmaWorkgroup = 8;  // leaves each wave of the matrix-core kernel 256 VGPRs
constexpr int kNumXcd = 8;
constexpr int kNumCus = 256;
constexpr int kKStationaryParkSlots = kMaxWavesPerWorkgroup + 1;  // k-stationary matrix-core kernel: entries of 16 bytes per block of partial sums
constexpr int kMaxKStationaryLds = 128 * 1024;  // most LDS the k-stationary matrix-core kernel parks partial sums in
constexpr int kMaxValuBatch = 4;  // activation rows handled per launch by the VALU kernel
constexpr int kExactIntegerFormOnly = 1;  // GemvTail::flags: never take the short int4 dequantiser
constexpr int kSingleStage = 2;           // GemvTail::flags: no load in flight while a unit is computed (VALU kernel)
constexpr int kParkBehindStage = 16;      // GemvTail::flags, k-stationary matrix-core kernel: the partial sums have LDS of their own behind the activation stages
constexpr int kTimelineWaits = 8;         // GemvTail::flags, timeline probe: time the wait in front of every unit as well
constexpr int kTimelineWordsPerWave = MGEMV_PROBE_TIMELINE_WORDS;  // 64-bit words the timeline probe writes per wave
constexpr int kProbeNone = 0, kProbeLoadsOnly = 1, kProbeTimeline = 2, kProbeComputeOnly = 3;  // measurement builds of the VALU kernel

// Kernel arguments.  The first ten (four pointers and six 32-bit words, 14 dwords) are what a
// wave needs to address its first loads, and they are preloaded into SGPRs (build flag
// -amdgpu-kernarg-preload-count=14); everything else sits in GemvTail.
struct GemvTail {
  const half_t* bias;
  half_t* y;
  int split_k;         // waves of a workgroup that share one tile (blockDim.x / 64)
  int m_batch;         // activation rows (matrix-core kernel)
  int num_groups;      // k / group_size (1 in per-column mode): extent of the scale / zero tables
  int flags;           // kExactIntegerFormOnly | kSingleStage
  float alpha, beta;   // epilogue: y = alpha * acc + beta * bias (gemv/device/gemv_adaptor.h:123, epilogue{alpha, beta})
  int seq_base;        // VALU kernel: tiles / sequences ...
  int seq_rem;         // ... and tiles % sequences (the first seq_rem sequences get one tile more)
  long long stride_weights, stride_x, stride_scale, stride_bias, stride_y;  // per batch problem
  const int* route;    // routed launch: problem b takes weights, scales, zeros and bias of entry route[b] of the stack
  int route_extent;    // entries in the stack: a problem routed outside [0, route_extent) is left alone
  unsigned long long* trace;  // timeline probe: kTimelineWordsPerWave words per wave, else unused
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
// group size in bits 0-23, tiles per workgroup in bits 24-30, bit 31: the launch is routed (GemvTail::route)
constexpr uint32_t kRoutedLaunch = 0x80000000u;
constexpr uint32_t pack_group(int group_size, int tiles_per_wg, bool routed) {
  return (uint32_t)group_size | ((uint32_t)tiles_per_wg << 24) | (routed ? kRoutedLaunch : 0u);
}
constexpr int tiles_per_wg_of(uint32_t packed_group) { return (int)((packed_group >> 24) & 0x7fu); }

// ---------------------------------------------------------------------------------------------
// Which part of the problem a wave works on.  Plain integer functions, compiled for the device
// (the kernels call them) and for the host (which replays them over a whole grid to check that a
// launch plan covers every tile and k step exactly once).
// ---------------------------------------------------------------------------------------------

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Neighbouring tiles read
// neighbouring 32-byte pieces of the same scale/zero cache lines, so give each XCD (and its
// private L2) a contiguous range of tiles instead of every eighth one.
__host__ __device__ __forceinline__ int logical_workgroup_of(int block, int wgs_per_xcd) {
  const int xcd = block % kNumXcd;
  const int slot = block / kNumXcd;
  return xcd * wgs_per_xcd + slot;
}

struct WaveWork {
  int tile_begin, tiles;  // tiles tile_begin .. tile_begin + tiles - 1 (tiles may be 0)
  int ks_begin, units;    // k steps ks_begin .. ks_begin + units - 1 of each of them (units may be <= 0)
};

// k range of the kw-th wave along k.
__host__ __device__ __forceinline__ void wave_k_range(WaveWork& w, int kw, int steps_per_wave, int ksteps) {
  w.ks_begin = kw * steps_per_wave;
  const int end = w.ks_begin + steps_per_wave < ksteps ? w.ks_begin + steps_per_wave : ksteps;
  w.units = end - w.ks_begin;
}

// VALU kernel.  The tiles are dealt out evenly, in contiguous runs, to the (workgroups x
// tiles_per_wg) tile sequences of the launch (multi: sequence s takes seq_base tiles, the first
// seq_rem sequences one more); the split_k waves of a sequence walk its tiles together, each on
// its own part of k.  Without walks (multi false) sequence s is tile s.
__host__ __device__ __forceinline__ WaveWork valu_wave_work(bool multi, int wg, int ty, int kw, int tiles_per_wg,
                                                            int seq_base, int seq_rem, int tiles, int steps_per_wave,
                                                            int ksteps) {
  WaveWork w;
  const int seq = wg * tiles_per_wg + ty;
  w.tile_begin = multi ? seq * seq_base + (seq < seq_rem ? seq : seq_rem) : seq;
  w.tiles = multi ? seq_base + (seq < seq_rem ? 1 : 0) : (seq < tiles ? 1 : 0);
  wave_k_range(w, kw, steps_per_wave, ksteps);
  return w;
}

// Register-operand matrix-core kernel: a wave takes tiles_per_wave consecutive tiles.
__host__ __device__ __forceinline__ WaveWork mfma_wave_work(int tiles_per_wave, int wg, int ty, int kw, int tiles_per_wg,
                                                            int tiles, int steps_per_wave, int ksteps) {
  WaveWork w;
  w.tile_begin = (wg * tiles_per_wg + ty) * tiles_per_wave;
  const int left = tiles - w.tile_begin;
  w.tiles = left <= 0 ? 0 : left < tiles_per_wave ? left : tiles_per_wave;
  wave_k_range(w, kw, steps_per_wave, ksteps);
  return w;
}

// LDS-staged matrix-core kernel: one tile per wave; a wave past the last tile has no tile of
// its own (it still stages activation rows and meets the barriers).
__host__ __device__ __forceinline__ WaveWork staged_wave_work(int wg, int ty, int kw, int tiles_per_wg, int tiles,
                                                              int steps_per_wave, int ksteps) {
  WaveWork w;
  w.tile_begin = wg * tiles_per_wg + ty;
  w.tiles = w.tile_begin < tiles ? 1 : 0;
  wave_k_range(w, kw, steps_per_wave, ksteps);
  return w;
}

__device__ __forceinline__ int logical_workgroup(const Problem& p) {
  return logical_workgroup_of((int)blockIdx.x, p.wgs_per_xcd);
}

// Group index of reduction position k_index (host/mixed_gemv.h:88), clamped to the last
// group for the padded positions past k.
__device__ __forceinline__ int group_of(const Problem& p, int k_index) {
  k_index = k_index < p.k ? k_index : p.k - 1;
  const bool pow2 = (p.group_size & (p.group_size - 1)) == 0;
  return pow2 ? (k_index >> __builtin_ctz((unsigned)p.group_size)) : (k_index / p.group_size);
}

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

struct ScaleTables {
  __amdgpu_buffer_rsrc_t scale, zero;
};

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

// Epilogue value before the final rounding: alpha * acc + beta * bias in fp32, the outer
// multiply-add fused -- what the reference's LinearCombination computes (alpha * accumulator +
// source, epilogue/threadblock/epilogue.h:64, 93; one `a * b + c` per element, which nvcc
// contracts).  With alpha = beta = 1 this is the single rounded fp32 add of
// host/mixed_gemv.h:102-103, bit for bit, and without a bias it adds +0 as the reference does.
__device__ __forceinline__ float epilogue_value(const GemvTail& tail, float acc, bool has_bias, float bias) {
  return __builtin_fmaf(tail.alpha, acc, has_bias ? tail.beta * bias : 0.0f);
}

// Sum over the four k slices of a wave: lanes l, l+16, l+32, l+48 hold the same row.
// The result is valid in lanes 0..15.
__device__ __forceinline__ float reduce_k_slices(float v) {
  v += __shfl_down(v, 32);
  v += __shfl_down(v, 16);
  return v;
}

// The kernel arguments behind the preloaded ones, read where the caller stands instead of at the
// kernel's entry.  A by-value kernel argument is fetched by scalar loads that the compiler puts
// in front of everything else, and as soon as one of the registers they target is needed for
// something else the wave waits for them -- a miss of the (just invalidated) scalar cache on the way
// to the first weight loads.  Reading the words through the kernarg segment pointer behind a
// statement the compiler cannot look through keeps those loads where they are written.
// The ten arguments in front of the tail occupy 56 bytes in every kernel of this library.
constexpr int kTailKernargOffset = 56;
static_assert(alignof(GemvTail) == 8 && kTailKernargOffset % alignof(GemvTail) == 0 && sizeof(GemvTail) % 4 == 0,
              "GemvTail follows four pointers and six 32-bit words without padding");
__device__ __forceinline__ GemvTail read_tail_here() {
  typedef const __attribute__((address_space(4))) uint32_t* KernargWords;
  KernargWords words = (KernargWords)__builtin_amdgcn_kernarg_segment_ptr() + kTailKernargOffset / 4;
  asm volatile("" : "+s"(words) : : "memory");
  uint32_t raw[sizeof(GemvTail) / 4];
#pragma unroll
  for (int i = 0; i < (int)(sizeof(GemvTail) / 4); ++i) raw[i] = words[i];
  GemvTail t;
  __builtin_memcpy(&t, raw, sizeof(GemvTail));
  return t;
}

// The lane number, recomputed.  Used behind the unit loop so that the value computed in front
// of it need not stay in a register (or be spilled) across the loop.
__device__ __forceinline__ int lane_after_loop() {
  int l;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
  return l;
}

// ---------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------

struct LaunchPlan {
  int split_k, tiles_per_wg, steps_per_wave, workgroups, wgs_per_xcd, threads;
  int tiles_per_wave;  // 1 on the VALU path; 1, 2 or 4 on the matrix-core path
  int tiles_in_sequence;  // VALU path: most tiles any wave walks one after the other
  int staged_rows;        // LDS-staged matrix-core kernel: 8 or 16 activation rows per stage; 0 = other kernels
  int stages;             // VALU path: 2 = the next unit is in flight while one is computed, 1 = it is not
  bool matrix_core;       // one of the matrix-core kernels (else the VALU kernel)
  bool k_stationary;      // the matrix-core kernel whose waves keep one k step each while the workgroup walks tiles_in_sequence tiles
};

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
  int device;  // the device `stream` belongs to
};

// Dispatchers, one translation unit each (the kernels are templates on weight width, quant mode,
// activation rows, groups per run, ...; the run-time values pick the instantiation).
hipError_t launch_gemv_f16(const GemvLaunch& g, int bits, int qop, int mb, int gpr);
hipError_t launch_gemv_bf16(const GemvLaunch& g, int bits, int qop, int mb, int gpr);
hipError_t launch_mfma(const GemvLaunch& g, int bits, int qop, int gpr);
hipError_t launch_mfma_lds(const GemvLaunch& g, int bits, int qop, int gpr, int rounds, int act);
hipError_t launch_mfma_kstat(const GemvLaunch& g, int bits, int qop, int gpr, int act);
// ... and of the k-stationary matrix-core kernel (kProbeLoadsOnly / kProbeComputeOnly), where they exist.
bool mfma_kstat_probe_exists(int bits, int qop, int gpr, int act);
hipError_t launch_mfma_kstat_probe(const GemvLaunch& g, int gpr, int probe);
// Measurement builds of the single-row int4 scale-and-zero fp16 VALU kernel (probe: kProbeLoadsOnly / kProbeTimeline / kProbeComputeOnly).
hipError_t launch_gemv_probe(const GemvLaunch& g, int probe);
// ... and of the LDS-staged matrix-core kernel (kProbeLoadsOnly / kProbeComputeOnly), where they exist.
bool mfma_lds_probe_exists(int bits, int qop, int gpr, int rounds, int act, int tiles_per_wg);
hipError_t launch_mfma_lds_probe(const GemvLaunch& g, int gpr, int rounds, int probe);

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_KERNEL_COMMON_H_
