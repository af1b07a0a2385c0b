// Device-side numeric building blocks for gfx950: the biased-integer -> fp16 converters, the
// two-rounding dequantiser and the DPP-broadcast dot product.  Everything here is wave64
// VALU code; nothing in this file is shared with or derived from a CUDA path.
#ifndef MIXED_GEMV_AMD_DEVICE_MATH_H_
#define MIXED_GEMV_AMD_DEVICE_MATH_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

// The dequantiser is "fp16 multiply, then fp16 add", two separately rounded operations
// (gemv/warp/warp_dequantizer.h:52-59).  A contracted v_pk_fma_f16 rounds once and changes
// bits, so contraction is switched off for everything that includes this header (the build
// also passes -ffp-contract=off).
#pragma clang fp contract(off)

namespace mgemv {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ half2_t splat(half_t v) { return half2_t{v, v}; }

// Register-resident constants for the converters.  VOP3 encodings on this target take no
// 32-bit literal, so (w & mask) | magic only becomes a single v_and_or_b32 when mask and
// magic already sit in registers; the empty asm keeps the compiler from folding them back
// into literals (which would split the operation into v_and + v_or).
struct ConvertRegs {
  uint32_t mask_lo;   // 0x000f000f   nibble 0 of each 16-bit half
  uint32_t mask_hi;   // 0x00f000f0   nibble 1 of each 16-bit half
  uint32_t magic;     // 0x64006400   fp16 1024.0 in both halves
  uint32_t sel_lo;    // v_perm selector: bytes 0,1 of a word into the low byte of each half
  uint32_t sel_hi;    // v_perm selector: bytes 2,3
};

__device__ __forceinline__ ConvertRegs make_convert_regs() {
  ConvertRegs c;
  c.mask_lo = 0x000f000fu;
  c.mask_hi = 0x00f000f0u;
  c.magic = 0x64006400u;
  c.sel_lo = 0x04010400u;
  c.sel_hi = 0x04030402u;
  asm("" : "+s"(c.mask_lo));
  asm("" : "+s"(c.mask_hi));
  asm("" : "+v"(c.magic));
  asm("" : "+s"(c.sel_lo));
  asm("" : "+s"(c.sel_hi));
  return c;
}

// int4: one stored word (8 biased nibbles in the order of tile_layout.h) -> 8 fp16 values,
// exact integers in [-8, 7], as 4 packed pairs in ascending k.
//   (w & 0x000f000f) | 0x6400_6400  is the pair (1024 + u0, 1024 + u1);  minus 1032 -> u - 8
//   (w & 0x00f000f0) | 0x6400_6400  is the pair (1024 + 16 u2, 1024 + 16 u3);  * 1/16 - 72 -> u - 8
// and the same on w >> 8.  All four operations are exact in fp16.  This is the bit-level
// contract of gemv/interleaved_numeric_conversion.h:232-291 (lop3 / sub.f16x2 / fma.rn.f16x2)
// expressed in v_and_or_b32, v_pk_add_f16 and v_pk_fma_f16.
__device__ __forceinline__ void convert_int4_word(uint32_t w, const ConvertRegs& c, half2_t (&q)[4]) {
  const uint32_t t = w >> 8;
  const half2_t h0 = as_half2((w & c.mask_lo) | c.magic);
  const half2_t h1 = as_half2((w & c.mask_hi) | c.magic);
  const half2_t h2 = as_half2((t & c.mask_lo) | c.magic);
  const half2_t h3 = as_half2((t & c.mask_hi) | c.magic);
  const half2_t k1032 = splat((half_t)1032.0f);
  const half2_t k16th = splat((half_t)0.0625f);
  const half2_t kn72 = splat((half_t)-72.0f);
  q[0] = h0 - k1032;
  q[1] = __builtin_elementwise_fma(h1, k16th, kn72);
  q[2] = h2 - k1032;
  q[3] = __builtin_elementwise_fma(h3, k16th, kn72);
}

// int8: one stored word (4 biased bytes, natural order) -> 4 fp16 exact integers in
// [-128, 127] as 2 packed pairs.  v_perm_b32 drops each byte under a 0x64 high byte
// (1024 + u), then minus 1152 -> u - 128.  Bit-level contract of
// gemv/interleaved_numeric_conversion.h:62-81 (prmt / sub.f16x2).
__device__ __forceinline__ void convert_int8_word(uint32_t w, const ConvertRegs& c, half2_t (&q)[2]) {
  const uint32_t sixty_four = 0x64646464u;
  const half2_t h0 = as_half2(__builtin_amdgcn_perm(sixty_four, w, c.sel_lo));
  const half2_t h1 = as_half2(__builtin_amdgcn_perm(sixty_four, w, c.sel_hi));
  const half2_t k1152 = splat((half_t)1152.0f);
  q[0] = h0 - k1152;
  q[1] = h1 - k1152;
}

// Dequantise one packed pair: rn16(rn16(q * s) + z) or rn16(q * s).
// gemv/warp/warp_dequantizer.h:52-59 (with zero) and :86-92 (without).
template <bool HAS_ZERO>
__device__ __forceinline__ half2_t dequant_pair(half2_t q, half2_t s, half2_t z) {
  half2_t d = q * s;
  if (HAS_ZERO) d = d + z;
  return d;
}

// acc += d.lo * x.lo + d.hi * x.hi in fp32, where x is read from lane SRC of the caller's
// DPP row (16 lanes) instead of the caller's own register: v_dot2c_f32_f16 with a
// row_newbcast DPP control.  This replaces gemv/thread/mma.h:83-95 (one scalar fp32 FMA per
// weight) and the register broadcast of the activation fragment
// (gemv/threadblock/dq_mma_base.h:76-103).
//
// The x operand must come straight from a memory load: a VALU write followed within two
// instructions by a DPP read of the same register is a hazard the assembler does not pad.
template <int SRC>
__device__ __forceinline__ void dot2_row_bcast(float& acc, uint32_t x, half2_t d) {
  static_assert(SRC >= 0 && SRC < 16, "source lane within a 16-lane DPP row");
  asm("v_dot2c_f32_f16_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
      : "+v"(acc)
      : "v"(x), "v"(d), "n"(SRC));
}

// The compiler does not know the asm above is a dot instruction, so it cannot pad the
// "dot result read by a different instruction" hazard of this target (3 wait states).
// Call this once after the last dot of a chain, before the accumulator is consumed.
__device__ __forceinline__ void settle_dot_chain(float& acc) { asm volatile("s_nop 4" : "+v"(acc)); }

// Raw buffer descriptor: base pointer + byte count; out-of-range lanes read zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

constexpr int kCacheDefault = 0;
constexpr int kCacheStream = 2;  // "nt": weights are read once, keep them from displacing x / scales

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_DEVICE_MATH_H_
