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
  uint32_t mask7;     // 0x07800780   the 4-bit field at bits 7-10 of each 16-bit half
  uint32_t mask3;     // 0x00780078   the 4-bit field at bits 3-6 of each 16-bit half
  uint32_t magic;     // 0x64006400   fp16 1024.0 in both halves      (general form only)
  uint32_t minus136;  // 0xd840d840   fp16 -136.0 in both halves      (general form only)
  uint32_t sel_lo;    // v_perm selector: bytes 0,1 of a word into the low byte of each half
  uint32_t sel_hi;    // v_perm selector: bytes 2,3
};

__device__ __forceinline__ ConvertRegs make_convert_regs() {
  ConvertRegs c;
  c.mask7 = 0x07800780u;
  c.mask3 = 0x00780078u;
  c.magic = 0x64006400u;
  c.minus136 = 0xd840d840u;
  c.sel_lo = 0x04010400u;
  c.sel_hi = 0x04030402u;
  asm("" : "+s"(c.mask7));
  asm("" : "+s"(c.mask3));
  asm("" : "+s"(c.magic));     // parked in SGPRs; general_form_regs() moves them where they are needed
  asm("" : "+s"(c.minus136));
  asm("" : "+s"(c.sel_lo));
  asm("" : "+s"(c.sel_hi));
  return c;
}

// The general form needs its two packed constants in VGPRs (a VOP3 instruction reads at most
// one SGPR).  They are copied there at the start of each general-form unit instead of living
// in VGPRs for the whole kernel, where they would cost the short form a wave of occupancy.
__device__ __forceinline__ ConvertRegs general_form_regs(ConvertRegs c) {
  asm volatile("v_mov_b32 %0, %2\n\tv_mov_b32 %1, %3" : "=&v"(c.magic), "=v"(c.minus136) : "s"(c.magic), "s"(c.minus136));
  return c;
}

__device__ __forceinline__ uint32_t rotate_right_8(uint32_t w) { return __builtin_amdgcn_alignbit(w, w, 8); }

// int4, general form: one stored word (8 biased 4-bit fields in the order of tile_layout.h)
// -> 8 fp16 values, exact integers in [-8, 7], as 4 packed pairs in ascending k.
//   (v & 0x00780078) | 0x6400_6400  is the pair (1024 + 8 u, 1024 + 8 u');  * 1/8 - 136 -> u - 8
// for v = w >> 4, w, rotr(w, 12) and w >> 8.  Every step is exact in fp16.  This is the
// numeric contract of gemv/interleaved_numeric_conversion.h:232-291 (lop3 / sub.f16x2 /
// fma.rn.f16x2: biased nibble under a 1024.0 exponent, then an exact affine map) expressed
// in v_alignbit_b32, v_and_or_b32 and v_pk_fma_f16.  (It shares no intermediate with the
// short form below, so the compiler has nothing to hoist in front of the branch between them.)
__device__ __forceinline__ void convert_int4_word(uint32_t w, const ConvertRegs& c, half2_t (&q)[4]) {
  const half2_t h0 = as_half2(((w >> 4) & c.mask3) | c.magic);
  const half2_t h1 = as_half2((w & c.mask3) | c.magic);
  const half2_t h2 = as_half2((__builtin_amdgcn_alignbit(w, w, 12) & c.mask3) | c.magic);
  const half2_t h3 = as_half2(((w >> 8) & c.mask3) | c.magic);
  const half2_t k8th = splat((half_t)0.125f);
  const half2_t kn136 = as_half2(c.minus136);
  q[0] = __builtin_elementwise_fma(h0, k8th, kn136);
  q[1] = __builtin_elementwise_fma(h1, k8th, kn136);
  q[2] = __builtin_elementwise_fma(h2, k8th, kn136);
  q[3] = __builtin_elementwise_fma(h3, k8th, kn136);
}

// int4, short form for a positive scale s below 2^-5.  A masked half-word read as fp16 IS
// u * 2^-17 (field at bits 7-10) or u * 2^-21 (field at bits 3-6), exactly; with the scale
// pre-multiplied by 2^17 / 2^21 (exact: s * 2^21 <= 65504) a single fused multiply-add
//     fma(u * 2^-p, s * 2^p, -8 s)  =  rn16(u s - 8 s)  =  rn16((u - 8) * s)
// rounds the exact product once, which is bit for bit the rn16(q * s) of
// gemv/warp/warp_dequantizer.h:52-59; the additive zero then follows as its own rounded
// add.  8 s is exact, and for s > 0 a zero product is +0 on both routes.  Outside
// 0 < s < 2^-5 (large, zero, negative, NaN) the general form above is used instead.
struct ShortFormScale {
  half2_t s17;   // (s * 2^17, s * 2^17)
  half2_t s21;   // (s * 2^21, s * 2^21)
  half2_t m8s;   // (-8 s, -8 s)
};

// fp16 bit pattern of a scale for which the short form is exact: 0x0001 .. 0x27ff.
__device__ __forceinline__ bool short_form_ok(uint32_t scale_bits) { return ((scale_bits & 0xffffu) - 1u) < 0x27ffu; }

__device__ __forceinline__ ShortFormScale make_short_form_scale(half2_t s2) {
  ShortFormScale f;
  const half2_t a = s2 * splat((half_t)32768.0f);  // 2^17 itself is not an fp16 value
  f.s17 = a * splat((half_t)4.0f);
  f.s21 = f.s17 * splat((half_t)16.0f);
  f.m8s = s2 * splat((half_t)-8.0f);
  return f;
}

template <bool HAS_ZERO>
__device__ __forceinline__ void dequant_int4_word_short(uint32_t w, const ConvertRegs& c, const ShortFormScale& f,
                                                        half2_t z2, half2_t (&d)[4]) {
  const uint32_t t = rotate_right_8(w);
  d[0] = __builtin_elementwise_fma(as_half2(w & c.mask7), f.s17, f.m8s);
  d[1] = __builtin_elementwise_fma(as_half2(w & c.mask3), f.s21, f.m8s);
  d[2] = __builtin_elementwise_fma(as_half2(t & c.mask7), f.s17, f.m8s);
  d[3] = __builtin_elementwise_fma(as_half2(t & c.mask3), f.s21, f.m8s);
  if (HAS_ZERO) {
#pragma unroll
    for (int h = 0; h < 4; ++h) d[h] = d[h] + z2;
  }
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
// instructions by a DPP read of the same register is a hazard that neither the assembler nor
// the compiler (which sees an opaque asm statement) pads.  Nothing in the sources can stop the
// register allocator from copying x or the accumulator at a bad place, so the build checks the
// compiled code instead: isa_lint.py walks the device assembly of every kernel and fails the
// build on a VALU write within two wait states in front of a DPP read, or a read of a dot
// result by any other kind of instruction within three behind it.
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

// ---------------------------------------------------------------------------------------------
// bfloat16 activations / scales / outputs.
//
// The reference's bf16 converters (gemv/interleaved_numeric_conversion.h:130-183 for int8,
// :340-401 for int4) produce the exact integer q as a bf16, and its dequantiser
// (gemv/warp/warp_dequantizer.h:52-59) multiplies by the scale and adds the zero term, each
// rounded to bf16.  This target has no packed bf16 arithmetic, so both steps run in fp32, where
// q * s is exact (at most 8 x 8 significant bits), and v_cvt_pk_bf16_f32 rounds to nearest even;
// for the sum, rounding the fp32 sum to bf16 equals rounding the exact sum once (24 >= 2*8+2).
// Values are kept as packed pairs of bf16 bit patterns, (low, high) = ascending k.
//
// Two forms, as for fp16.  With 8u (int4) or u (int8) from v_cvt_f32_ubyteN:
//   fused    fma(8u, s/8, -8s) resp. fma(u, s, -128s): exact, hence = q*s, for 2^-100 <= s < 2^119
//            (-8s / -128s stays finite; for s > 0 a zero product is +0 on both routes).  For int4
//            the fma and the conversions around it are v_dot2_f32_bf16 instructions on packed
//            pairs (dequant_int4_word_bf16), which needs s/8 to be a normal bf16;
//   general  (8u - 64) * (s/8) resp. (u - 128) * s: exact for every finite s, with the sign of
//            a zero product as the reference's multiply gives it.
// ---------------------------------------------------------------------------------------------
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#ifndef MGEMV_BF16_DOT_DEQUANT
#define MGEMV_BF16_DOT_DEQUANT 1
#endif
constexpr bool kBf16DotDequant = MGEMV_BF16_DOT_DEQUANT != 0;  // 0: the v_cvt / v_fma route for int4 as well
constexpr int kActF16 = 0;
constexpr int kActBf16 = 1;

__device__ __forceinline__ float bf16_low_to_f32(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }
__device__ __forceinline__ float bf16_high_to_f32(uint32_t bits) { return __builtin_bit_cast(float, bits & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2_t));
}
template <int BYTE>
__device__ __forceinline__ float byte_to_f32(uint32_t v) {
  return (float)((v >> (8 * BYTE)) & 0xffu);  // v_cvt_f32_ubyteN
}

// bf16 bit pattern of a scale for which the fused form is exact (both weight widths):
// 0x0d80 .. 0x7aff, i.e. 2^-100 <= s < 2^119 -- positive, s/8 a normal bf16, -128 s finite.
__device__ __forceinline__ bool fused_form_ok_bf16(uint32_t scale_bits) { return ((scale_bits & 0xffffu) - 0x0d80u) < (0x7b00u - 0x0d80u); }

struct Bf16Scale {
  float mul;        // int4: s/8; int8: s
  float add;        // fused form: -8s resp. -128s (int4 through the dot instructions: -24s); general form: unused
  float z;          // additive zero
  uint32_t sel_lo;  // int4 fused form through the dot instructions: the bf16 pairs (s/8, 0) ...
  uint32_t sel_hi;  // ... and (0, s/8)
};

template <int BITS, bool FUSED>
__device__ __forceinline__ Bf16Scale make_bf16_scale(uint32_t s_bits, uint32_t z_bits) {
  const float s = bf16_low_to_f32(s_bits);
  Bf16Scale f;
  f.mul = BITS == 4 ? s * 0.125f : s;
  f.add = FUSED ? s * (BITS == 4 ? (kBf16DotDequant ? -24.0f : -8.0f) : -128.0f) : 0.0f;
  f.z = bf16_low_to_f32(z_bits);
  f.sel_lo = f.sel_hi = 0;
  if constexpr (BITS == 4 && FUSED && kBf16DotDequant) {
    f.sel_lo = (s_bits & 0xffffu) - 0x0180u;  // s/8: three off the exponent of a normal s (the fused range has no other)
    f.sel_hi = f.sel_lo << 16;
  }
  return f;
}

// (a, b): the integers 8u (int4) or u (int8) of a k-adjacent pair -> packed bf16 pair of
// rn(rn(q s) + z) resp. rn(q s).
template <int BITS, bool HAS_ZERO, bool FUSED>
__device__ __forceinline__ uint32_t dequant_pair_bf16(float a, float b, const Bf16Scale& f) {
  float p0, p1;
  if constexpr (FUSED) {
    p0 = __builtin_fmaf(a, f.mul, f.add);
    p1 = __builtin_fmaf(b, f.mul, f.add);
  } else {
    constexpr float kBias = BITS == 4 ? 64.0f : 128.0f;
    p0 = (a - kBias) * f.mul;
    p1 = (b - kBias) * f.mul;
  }
  uint32_t d = pack_bf16(p0, p1);
  if constexpr (HAS_ZERO) d = pack_bf16(bf16_low_to_f32(d) + f.z, bf16_high_to_f32(d) + f.z);
  return d;
}

// Eight bf16 values (four packed pairs a[0..3]) through out = rn_bf16(a * m + c), fp32 inside:
// v_dot2_f32_bf16 with the factor pair sel_lo = (m, 0) resp. sel_hi = (0, m) computes
// a.lo * m + c resp. a.hi * m + c straight from the packed pair -- fused, one rounding (checked
// exhaustively by the tests) -- and v_cvt_pk_bf16_f32 rounds to bf16.  The product with the zero
// factor vanishes as long as every a is finite, which the fused form's scale range guarantees.
// One asm block, because the compiler does not know these are dot instructions: their results
// must not be read by another kind of instruction within three issue slots, and the order
// below keeps at least three instructions between each dot and the conversion that consumes it.
__device__ __forceinline__ void dot_round_bf16x8(const uint32_t (&a)[4], uint32_t sel_lo, uint32_t sel_hi, float c,
                                                 uint32_t (&out)[4]) {
  float t0, t1, t2, t3, t4, t5, t6, t7;
  asm("v_dot2_f32_bf16 %4, %12, %16, %18\n\t"
      "v_dot2_f32_bf16 %5, %12, %17, %18\n\t"
      "v_dot2_f32_bf16 %6, %13, %16, %18\n\t"
      "v_dot2_f32_bf16 %7, %13, %17, %18\n\t"
      "v_dot2_f32_bf16 %8, %14, %16, %18\n\t"
      "v_dot2_f32_bf16 %9, %14, %17, %18\n\t"
      "v_dot2_f32_bf16 %10, %15, %16, %18\n\t"
      "v_dot2_f32_bf16 %11, %15, %17, %18\n\t"
      "v_cvt_pk_bf16_f32 %0, %4, %5\n\t"
      "v_cvt_pk_bf16_f32 %1, %6, %7\n\t"
      "v_cvt_pk_bf16_f32 %2, %8, %9\n\t"
      "v_cvt_pk_bf16_f32 %3, %10, %11"
      : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3]), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3),
        "=&v"(t4), "=&v"(t5), "=&v"(t6), "=&v"(t7)
      : "v"(a[0]), "v"(a[1]), "v"(a[2]), "v"(a[3]), "v"(sel_lo), "v"(sel_hi), "v"(c));
}

// int4: the fields of elements (2,3) sit at bits 3-6 of bytes 0 and 2, those of (6,7) at bits 3-6
// of bytes 1 and 3; (0,1) and (4,5) come to bytes 0 and 2 after a shift by 4 resp. a rotation
// by 12 (tile_layout.h).  A masked byte converts to 8u.
template <bool HAS_ZERO, bool FUSED>
__device__ __forceinline__ void dequant_int4_word_bf16(uint32_t w, const ConvertRegs& c, const Bf16Scale& f,
                                                       uint32_t (&d)[4]) {
  if constexpr (FUSED && kBf16DotDequant) {
    // A field at bits 3-6 of a half-word under the bf16 pattern 0x4300 (128.0, mantissa step 1) IS
    // the bf16 value 128 + 8u -- the route of gemv/interleaved_numeric_conversion.h:340-401 on
    // these field positions -- and (128 + 8u) * (s/8) - 24 s = (u - 8) s exactly.
    uint32_t magic;  // in a VGPR, so that mask (an SGPR) and magic fit one v_and_or_b32
    asm("v_mov_b32 %0, 0x43004300" : "=v"(magic));
    uint32_t m[4];
    m[0] = ((w >> 4) & c.mask3) | magic;
    m[1] = (w & c.mask3) | magic;
    m[2] = (__builtin_amdgcn_alignbit(w, w, 12) & c.mask3) | magic;
    m[3] = ((w >> 8) & c.mask3) | magic;
    if constexpr (HAS_ZERO) {
      uint32_t pb[4];
      dot_round_bf16x8(m, f.sel_lo, f.sel_hi, f.add, pb);
      dot_round_bf16x8(pb, 0x00003f80u, 0x3f800000u, f.z, d);   // factors (1, 0) and (0, 1)
    } else {
      dot_round_bf16x8(m, f.sel_lo, f.sel_hi, f.add, d);
    }
    return;
  }
  const uint32_t e01 = (w >> 4) & c.mask3;
  const uint32_t e23 = w & c.mask3;
  const uint32_t e45 = __builtin_amdgcn_alignbit(w, w, 12) & c.mask3;
  const uint32_t e67 = w & 0x78007800u;
  d[0] = dequant_pair_bf16<4, HAS_ZERO, FUSED>(byte_to_f32<0>(e01), byte_to_f32<2>(e01), f);
  d[1] = dequant_pair_bf16<4, HAS_ZERO, FUSED>(byte_to_f32<0>(e23), byte_to_f32<2>(e23), f);
  d[2] = dequant_pair_bf16<4, HAS_ZERO, FUSED>(byte_to_f32<0>(e45), byte_to_f32<2>(e45), f);
  d[3] = dequant_pair_bf16<4, HAS_ZERO, FUSED>(byte_to_f32<1>(e67), byte_to_f32<3>(e67), f);
}

// int8: 4 biased bytes in natural order.
template <bool HAS_ZERO, bool FUSED>
__device__ __forceinline__ void dequant_int8_word_bf16(uint32_t w, const Bf16Scale& f, uint32_t (&d)[2]) {
  d[0] = dequant_pair_bf16<8, HAS_ZERO, FUSED>(byte_to_f32<0>(w), byte_to_f32<1>(w), f);
  d[1] = dequant_pair_bf16<8, HAS_ZERO, FUSED>(byte_to_f32<2>(w), byte_to_f32<3>(w), f);
}

// bf16 counterpart of dot2_row_bcast (same hazards, same settle_dot_chain afterwards).
template <int SRC>
__device__ __forceinline__ void dot2_row_bcast_bf16(float& acc, uint32_t x, uint32_t d) {
  static_assert(SRC >= 0 && SRC < 16, "source lane within a 16-lane DPP row");
  asm("v_dot2c_f32_bf16_dpp %0, %1, %2 row_newbcast:%3 row_mask:0xf bank_mask:0xf"
      : "+v"(acc)
      : "v"(x), "v"(d), "n"(SRC));
}

// Raw buffer descriptor: base pointer + byte count; out-of-range lanes read zero.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}

constexpr int kCacheDefault = 0;
constexpr int kCacheStream = 2;  // "nt": weights are read once, keep them from displacing x / scales

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_DEVICE_MATH_H_
