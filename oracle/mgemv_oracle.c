/*
 * CPU oracle for the weight-only-quantised GEMV path of JJXiangJiaoJun/mixed_gemv.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of the
 * reference's HOST_CHECK path and of its host utilities so that the HIP kernels can be
 * checked against it.  Nothing in the shipped library links, loads or calls it; only the
 * tests, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function cites the reference file:line it follows.  All half-precision arithmetic
 * is done the way the reference's host half type does it: convert both operands to
 * binary32, do one binary32 operation, round the result to binary16 with
 * round-to-nearest-even.  For a product of two halves the binary32 result is exact
 * (22 significant bits), and for a sum the double rounding 53/24 -> 11 bits is innocuous
 * because 24 >= 2*11+2, so each such operation equals the correctly rounded IEEE-754
 * binary16 operation.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see Makefile); no -march flags so the
 * results do not depend on the host's vector extensions.
 *
 * Pinning status (what independent evidence each function is checked against is listed in
 * tests/test_oracle_*.py):
 *   orc_f16_to_f32 / orc_f32_to_f16    exhaustive against numpy.float16
 *   orc_pack_int4 / orc_unpack_int4    closed form, exhaustive over byte values
 *   orc_fold_zero_points               exhaustive z x all finite scales against numpy.float16
 *   orc_ref_preprocess_* / orc_ref_convert_*  invariant convert(preprocess(W)) == W
 *   orc_dequantize                     numpy.float16 restatement, exhaustive q x all scales
 *   orc_gemv                           numpy restatement, one-hot / all-ones closed forms,
 *                                      float64 bound
 *   orc_fill_*                         definitional (they are the generator); statistics only
 *   orc_bf16_to_f32 / orc_f32_to_bf16  exhaustive / 4 M random floats against torch.bfloat16; ties
 *   orc_bf16_mul / orc_bf16_add        exact rational arithmetic (fractions) on random and edge pairs
 *   orc_dequantize_bf16 / orc_gemv_bf16 / orc_fold_zero_points_bf16
 *                                      the same loops as the fp16 functions with the element
 *                                      arithmetic swapped; torch.bfloat16 restatements, one-hot and
 *                                      unit-weight closed forms.  The reference holds no bf16 test or
 *                                      vector (its bf16 instantiation does not compile,
 *                                      gemv/threadblock/default_dq_mma_simt.h:133-134), so these are
 *                                      pinned by the mathematics alone.
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------ */
/* binary16 <-> binary32, software, IEEE-754 round-to-nearest-even                       */
/* ------------------------------------------------------------------------------------ */

ORC_API float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

ORC_API uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((absx >> 13) & 0x3ffu));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* <= 2^-25 rounds to zero (tie at 2^-25 goes to even = 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                      /* bits to drop */
  uint32_t hexp;
  if (e < -14) { /* result subnormal */
    shift = 13 + (-14 - e);
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t kept = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) kept += 1;
  uint32_t out;
  if (hexp == 0) {
    out = kept; /* may carry into exponent 1: still the right encoding */
  } else {
    out = ((hexp - 1) << 10) + kept; /* kept has the implicit bit at position 10 */
  }
  return (uint16_t)(sign | out);
}

static inline uint16_t h_mul(uint16_t a, uint16_t b) {
  return orc_f32_to_f16(orc_f16_to_f32(a) * orc_f16_to_f32(b));
}
static inline uint16_t h_add(uint16_t a, uint16_t b) {
  return orc_f32_to_f16(orc_f16_to_f32(a) + orc_f16_to_f32(b));
}
static inline uint16_t h_neg(uint16_t a) { return (uint16_t)(a ^ 0x8000u); }
static inline uint16_t h_from_int(int v) { return orc_f32_to_f16((float)v); }

ORC_API uint16_t orc_h_mul(uint16_t a, uint16_t b) { return h_mul(a, b); }
ORC_API uint16_t orc_h_add(uint16_t a, uint16_t b) { return h_add(a, b); }

/* bfloat16 = the upper 16 bits of a binary32; conversion from binary32 rounds to nearest even
 * (cutlass::bfloat16_t's conversion, which the reference's element types would use).  A product
 * of two bfloat16 values is exact in binary32 (16 significant bits) and for a sum the double
 * rounding 24 -> 8 bits is innocuous (24 >= 2*8+2), so one binary32 operation followed by this
 * rounding is the correctly rounded bfloat16 operation. */
ORC_API float orc_bf16_to_f32(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
ORC_API uint16_t orc_f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u); /* quiet NaN */
  uint32_t kept = x >> 16, rem = x & 0xffffu;
  if (rem > 0x8000u || (rem == 0x8000u && (kept & 1u))) kept += 1; /* carries into the exponent / to inf correctly */
  return (uint16_t)kept;
}
static inline uint16_t b_mul(uint16_t a, uint16_t b) { return orc_f32_to_bf16(orc_bf16_to_f32(a) * orc_bf16_to_f32(b)); }
static inline uint16_t b_add(uint16_t a, uint16_t b) { return orc_f32_to_bf16(orc_bf16_to_f32(a) + orc_bf16_to_f32(b)); }
ORC_API uint16_t orc_bf16_mul(uint16_t a, uint16_t b) { return b_mul(a, b); }
ORC_API uint16_t orc_bf16_add(uint16_t a, uint16_t b) { return b_add(a, b); }

/* Element type of activations / scales / zeros / outputs: the reference's ElementB = ElementScale =
 * ElementOutput template arguments (host/mixed_gemv.h:24-31). */
enum { ORC_ELEM_F16 = 0, ORC_ELEM_BF16 = 1 };
static inline uint16_t e_mul(int elem, uint16_t a, uint16_t b) { return elem == ORC_ELEM_BF16 ? b_mul(a, b) : h_mul(a, b); }
static inline uint16_t e_add(int elem, uint16_t a, uint16_t b) { return elem == ORC_ELEM_BF16 ? b_add(a, b) : h_add(a, b); }
static inline uint16_t e_from_int(int elem, int v) { /* |v| <= 128: exact in either type */
  return elem == ORC_ELEM_BF16 ? orc_f32_to_bf16((float)v) : orc_f32_to_f16((float)v);
}
static inline float e_to_f32(int elem, uint16_t a) { return elem == ORC_ELEM_BF16 ? orc_bf16_to_f32(a) : orc_f16_to_f32(a); }
static inline uint16_t e_from_f32(int elem, float f) { return elem == ORC_ELEM_BF16 ? orc_f32_to_bf16(f) : orc_f32_to_f16(f); }
/* Correctly rounded fused multiply-add on binary16, by exact integer arithmetic: every
 * finite half is an integer multiple of 2^-24, so a*b + c is an integer multiple of 2^-48
 * that fits in 128 bits.  Used for the reference converter's fma.rn.f16x2 and by tests
 * that show a fused dequantisation would differ from multiply-then-add. */
static int64_t h_to_fixed24(uint16_t h) { /* value * 2^24, finite inputs only */
  int64_t man = h & 0x3ff;
  int exp = (h >> 10) & 0x1f;
  int64_t v = exp == 0 ? man : ((man | 0x400) << (exp - 1));
  return (h & 0x8000) ? -v : v;
}

ORC_API uint16_t orc_h_fma(uint16_t a, uint16_t b, uint16_t c) {
  if ((a & 0x7c00) == 0x7c00 || (b & 0x7c00) == 0x7c00 || (c & 0x7c00) == 0x7c00) {
    /* inf / nan operands: no rounding question arises */
    double r = (double)orc_f16_to_f32(a) * (double)orc_f16_to_f32(b) + (double)orc_f16_to_f32(c);
    return orc_f32_to_f16((float)r);
  }
  __int128 v = (__int128)h_to_fixed24(a) * (__int128)h_to_fixed24(b) + ((__int128)h_to_fixed24(c) << 24);
  if (v == 0) {
    /* IEEE: exact zero sum is +0 unless both addends are -0 */
    int prod_neg = ((a ^ b) & 0x8000) != 0;
    int c_neg = (c & 0x8000) != 0;
    return (prod_neg && c_neg) ? 0x8000 : 0x0000;
  }
  uint16_t sign = 0;
  if (v < 0) {
    sign = 0x8000;
    v = -v;
  }
  unsigned __int128 m = (unsigned __int128)v; /* value = m * 2^-48 */
  int top = 127;
  while (!((m >> top) & 1)) --top;            /* value in [2^(top-48), 2^(top-47)) */
  int e = top - 48;                            /* unbiased exponent */
  int lsb_exp = e < -14 ? -24 : e - 10;        /* weight of the kept lsb */
  int shift = lsb_exp + 48;                    /* bits of m below the kept lsb */
  unsigned __int128 kept;
  if (shift <= 0) {
    kept = m << (-shift);
  } else {
    kept = m >> shift;
    unsigned __int128 rem = m & ((((unsigned __int128)1) << shift) - 1);
    unsigned __int128 half = ((unsigned __int128)1) << (shift - 1);
    if (rem > half || (rem == half && (kept & 1))) kept += 1;
  }
  uint32_t out;
  if (e < -14) {
    out = (uint32_t)kept; /* subnormal, a carry lands on exponent 1 */
  } else {
    out = ((uint32_t)(e + 15 - 1) << 10) + (uint32_t)kept;
  }
  if (out >= 0x7c00) out = 0x7c00; /* overflow to infinity */
  return (uint16_t)(sign | out);
}

/* array forms of the scalar helpers, for vectorised checks in the tests */
ORC_API void orc_f16_to_f32_n(float *out, const uint16_t *in, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_f16_to_f32(in[i]);
}
ORC_API void orc_f32_to_f16_n(uint16_t *out, const float *in, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_f16(in[i]);
}
ORC_API void orc_h_mul_n(uint16_t *out, const uint16_t *a, const uint16_t *b, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = h_mul(a[i], b[i]);
}
ORC_API void orc_h_add_n(uint16_t *out, const uint16_t *a, const uint16_t *b, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = h_add(a[i], b[i]);
}
ORC_API void orc_bf16_to_f32_n(float *out, const uint16_t *in, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_bf16_to_f32(in[i]);
}
ORC_API void orc_f32_to_bf16_n(uint16_t *out, const float *in, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(in[i]);
}
ORC_API void orc_bf16_mul_n(uint16_t *out, const uint16_t *a, const uint16_t *b, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = b_mul(a[i], b[i]);
}
ORC_API void orc_bf16_add_n(uint16_t *out, const uint16_t *a, const uint16_t *b, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = b_add(a[i], b[i]);
}
ORC_API void orc_h_fma_n(uint16_t *out, const uint16_t *a, const uint16_t *b, const uint16_t *c, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_h_fma(a[i], b[i], c[i]);
}

/* ------------------------------------------------------------------------------------ */
/* int4 packing: utils/preprocess.h:41-84, utils/vector_subbyte.h:55-67,150-156           */
/* element 2i -> bits 0..3 of byte i, element 2i+1 -> bits 4..7                           */
/* ------------------------------------------------------------------------------------ */

ORC_API void orc_pack_int4(uint8_t *packed, const int8_t *unpacked, size_t n_unpacked) {
  size_t nb = n_unpacked / 2; /* preprocess.h:62 */
  for (size_t i = 0; i < nb; ++i) {
    uint8_t lo = (uint8_t)unpacked[2 * i] & 0x0fu;          /* preprocess.h:79 */
    uint8_t hi = (uint8_t)((uint8_t)unpacked[2 * i + 1] << 4); /* preprocess.h:80 */
    packed[i] = (uint8_t)(lo | hi);
  }
}

ORC_API void orc_unpack_int4(int8_t *unpacked, const uint8_t *packed, size_t n_packed) {
  for (size_t i = 0; i < n_packed; ++i) {
    int8_t b = (int8_t)packed[i];
    unpacked[2 * i] = (int8_t)((int8_t)(b << 4) >> 4); /* preprocess.h:47 sign extension */
    unpacked[2 * i + 1] = (int8_t)(b >> 4);            /* preprocess.h:48 arithmetic shift */
  }
}

/* signed value of element idx of a packed int4 array (vector_subbyte.h:63-67,150-156) */
static inline int get_int4(const uint8_t *packed, size_t idx) {
  uint8_t b = packed[idx >> 1];
  int v = (idx & 1) ? (b >> 4) : (b & 0x0f);
  return v >= 8 ? v - 16 : v;
}

/* ------------------------------------------------------------------------------------ */
/* zero fold: utils/preprocess.h:94-101   out = half(-z) * s  (one fp16 multiply)         */
/* ------------------------------------------------------------------------------------ */

ORC_API void orc_fold_zero_points(uint16_t *out, const uint16_t *scales, const int8_t *zeros, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    out[i] = h_mul(h_from_int(-(int)zeros[i]), scales[i]); /* preprocess.h:99 */
  }
}
ORC_API void orc_fold_zero_points_bf16(uint16_t *out, const uint16_t *scales, const int8_t *zeros, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    out[i] = b_mul(e_from_int(ORC_ELEM_BF16, -(int)zeros[i]), scales[i]); /* preprocess.h:99 with bfloat16_t */
  }
}

/* ------------------------------------------------------------------------------------ */
/* the reference's own device layout and converter, restated only to document and pin    */
/* them (utils/preprocess.h:292-348, 365-455; gemv/interleaved_numeric_conversion.h)      */
/* ------------------------------------------------------------------------------------ */

/* src: [rows][cols] packed int4 row-major (cols/2 bytes per row). dst same size.
 * step 1 (preprocess.h:338-346) 4-row interleave of 32-bit words,
 * step 2 (preprocess.h:399-420) +8 on every nibble,
 * step 3 (preprocess.h:436-454) nibble permutation inside each 32-bit word.
 * returns 0, or -1 when rows%4 / cols%8 is violated (preprocess.h:319-327). */
ORC_API int orc_ref_preprocess_int4(uint8_t *dst, const uint8_t *src, size_t rows, size_t cols) {
  if (rows % 4 || cols % 8) return -1;
  size_t C = cols / 8;
  const uint32_t *in = (const uint32_t *)src;
  uint32_t *out = (uint32_t *)dst;
  for (size_t r = 0; r < rows; ++r) {
    for (size_t c = 0; c < C; ++c) {
      uint32_t w;
      memcpy(&w, &in[r * C + c], 4);
      /* +8 per nibble == xor 0x8 in two's complement nibble arithmetic */
      uint32_t biased = 0;
      for (int n = 0; n < 8; ++n) {
        int v = (int)((w >> (4 * n)) & 0xf);
        v = v >= 8 ? v - 16 : v;
        biased |= (uint32_t)((v + 8) & 0xf) << (4 * n);
      }
      uint32_t perm = 0;
      for (int d = 0; d < 8; ++d) {
        int s = d < 4 ? 2 * d : 2 * (d - 4) + 1; /* preprocess.h:446 */
        perm |= ((biased >> (4 * s)) & 0xfu) << (4 * d);
      }
      size_t o = (r / 4) * (C * 4) + c * 4 + (r % 4); /* preprocess.h:341-343 */
      memcpy(&out[o], &perm, 4);
    }
  }
  return 0;
}

/* bit-level simulation of interleaved_numeric_conversion.h:232-291 on one 32-bit word.
 * out[0..7] are fp16 bit patterns in the original element order. */
ORC_API void orc_ref_convert_u4x8(uint16_t out[8], uint32_t w) {
  const uint32_t MAGIC = 0x64006400u;
  uint32_t top = w >> 8;                       /* :252 */
  uint32_t h0 = (w & 0x000f000fu) | MAGIC;     /* :254-256 */
  uint32_t h1 = (w & 0x00f000f0u) | MAGIC;     /* :258-260 */
  uint32_t h2 = (top & 0x000f000fu) | MAGIC;   /* :262-264 */
  uint32_t h3 = (top & 0x00f000f0u) | MAGIC;   /* :266-268 */
  const uint16_t k1032 = 0x6408, k16th = 0x2c00, kn72 = 0xd480;
  uint32_t hs[4] = {h0, h1, h2, h3};
  for (int j = 0; j < 4; ++j) {
    for (int p = 0; p < 2; ++p) {
      uint16_t v = (uint16_t)(hs[j] >> (16 * p));
      uint16_t r;
      if ((j & 1) == 0) {
        r = h_add(v, h_neg(k1032));            /* sub.f16x2 :282,286 */
      } else {
        r = orc_h_fma(v, k16th, kn72);         /* fma.rn.f16x2 :284,288 */
      }
      out[2 * j + p] = r;
    }
  }
}

/* interleaved_numeric_conversion.h:62-81 for 4 biased bytes [e3 e1 e2 e0] */
ORC_API void orc_ref_convert_u8x4(uint16_t out[4], uint32_t w) {
  /* prmt selectors 0x5250 / 0x5351: result half p of h[0] = 0x64 : byte(p*2... ) */
  uint8_t b[4] = {(uint8_t)w, (uint8_t)(w >> 8), (uint8_t)(w >> 16), (uint8_t)(w >> 24)};
  /* h[0] = {0x64,b2 | 0x64,b0} -> halves (b0, b2); h[1] -> halves (b1, b3) (:69-73) */
  uint16_t pre[4] = {(uint16_t)(0x6400u | b[0]), (uint16_t)(0x6400u | b[2]),
                     (uint16_t)(0x6400u | b[1]), (uint16_t)(0x6400u | b[3])};
  for (int i = 0; i < 4; ++i) out[i] = h_add(pre[i], h_neg(0x6480)); /* :76-78 */
}

/* ------------------------------------------------------------------------------------ */
/* dequantisation of one weight                                                          */
/*   device convention  gemv/warp/warp_dequantizer.h:52-59 (scale then add) / :86-92      */
/*   host convention    host/mixed_gemv.h:92-96                                           */
/* ------------------------------------------------------------------------------------ */

enum { ORC_ZERO_NONE = 0, ORC_ZERO_INT8 = 1, ORC_ZERO_FOLDED_F16 = 2 };
enum { ORC_PER_COLUMN_SCALE_ONLY = 1, ORC_FINEGRAINED_SCALE_ONLY = 2, ORC_FINEGRAINED_SCALE_AND_ZEROS = 3 };

static inline uint16_t dequant_one(int elem, int q, uint16_t s, int zero_kind, const void *zero, size_t zi) {
  uint16_t p = e_mul(elem, e_from_int(elem, q), s); /* host/mixed_gemv.h:95-96 first product */
  if (zero_kind == ORC_ZERO_INT8) {
    /* host/mixed_gemv.h:92-93: scale_x_zero = -(s * half(z)) */
    uint16_t sz = h_neg(e_mul(elem, s, e_from_int(elem, (int)((const int8_t *)zero)[zi])));
    return e_add(elem, p, sz);
  } else if (zero_kind == ORC_ZERO_FOLDED_F16) {
    /* warp_dequantizer.h:57: plus(mul(q, s), zadd) */
    return e_add(elem, p, ((const uint16_t *)zero)[zi]);
  }
  return p; /* warp_dequantizer.h:90 */
}

static inline int get_q(const void *w, int bits, size_t idx) {
  return bits == 4 ? get_int4((const uint8_t *)w, idx) : (int)((const int8_t *)w)[idx];
}

/* W: un-preprocessed weights, [n_out][k] row-major, int4 packed two per byte or int8.
 * scale: [k/g][n_out] (n_out contiguous), per-column: [n_out].  zero: same shape, int8 or
 * fp16 according to zero_kind.  out: [n_out][k] fp16 bit patterns. */
static int dequantize_impl(int elem, uint16_t *out, const void *W, const uint16_t *scale, const void *zero,
                           int zero_kind, int n_out, int k, int group_size, int quant_op, int bits) {
  if (bits != 4 && bits != 8) return -1;
  if (quant_op == ORC_PER_COLUMN_SCALE_ONLY) group_size = k; /* mixed_gemv_test.cu:142-143 */
  if (quant_op != ORC_FINEGRAINED_SCALE_AND_ZEROS) zero_kind = ORC_ZERO_NONE; /* :145-147 */
  if (group_size <= 0) return -1;
#pragma omp parallel for schedule(static)
  for (int n = 0; n < n_out; ++n) {
    for (int kk = 0; kk < k; ++kk) {
      int g = kk / group_size; /* host/mixed_gemv.h:88 */
      size_t si = (size_t)g * (size_t)n_out + (size_t)n;
      int q = get_q(W, bits, (size_t)n * (size_t)k + (size_t)kk);
      out[(size_t)n * (size_t)k + kk] = dequant_one(elem, q, scale[si], zero_kind, zero, si);
    }
  }
  return 0;
}

ORC_API int orc_dequantize(uint16_t *out, const void *W, const uint16_t *scale, const void *zero,
                           int zero_kind, int n_out, int k, int group_size, int quant_op, int bits) {
  return dequantize_impl(ORC_ELEM_F16, out, W, scale, zero, zero_kind, n_out, k, group_size, quant_op, bits);
}
/* The same with bfloat16 scales / zeros / results (ORC_ZERO_FOLDED_F16 then means folded bf16). */
ORC_API int orc_dequantize_bf16(uint16_t *out, const void *W, const uint16_t *scale, const void *zero,
                                int zero_kind, int n_out, int k, int group_size, int quant_op, int bits) {
  return dequantize_impl(ORC_ELEM_BF16, out, W, scale, zero, zero_kind, n_out, k, group_size, quant_op, bits);
}

/* ------------------------------------------------------------------------------------ */
/* the HOST_CHECK GEMV: host/mixed_gemv.h:82-104, generalised to int8 weights, the three  */
/* quant modes, either zero convention, and m_batch activation rows (row b of x produces  */
/* y[b*n_out .. b*n_out+n_out), the column-major D with ldd = n_out of                    */
/* mixed_gemv_test.cu:140).  threads <= 1 runs the reference's single-threaded loop.      */
/* ------------------------------------------------------------------------------------ */

static void gemv_rows(int elem, uint16_t *y, const void *W, const uint16_t *x, const uint16_t *scale,
                      const void *zero, const uint16_t *bias, int zero_kind, int n_out,
                      int m_batch, int k, int group_size, int bits, int n_begin, int n_end) {
  for (int b = 0; b < m_batch; ++b) {
    const uint16_t *xb = x + (size_t)b * (size_t)k;
    for (int n = n_begin; n < n_end; ++n) {
      float acc = 0.0f; /* host/mixed_gemv.h:84 */
      for (int kk = 0; kk < k; ++kk) {
        int g = kk / group_size; /* :88 */
        size_t si = (size_t)g * (size_t)n_out + (size_t)n;
        int q = get_q(W, bits, (size_t)n * (size_t)k + (size_t)kk);
        float dq = e_to_f32(elem, dequant_one(elem, q, scale[si], zero_kind, zero, si)); /* :92-96 */
        acc += e_to_f32(elem, xb[kk]) * dq; /* :98 */
      }
      float bias_val = bias ? e_to_f32(elem, bias[n]) : 0.0f; /* :102 */
      y[(size_t)b * (size_t)n_out + n] = e_from_f32(elem, acc + bias_val); /* :103, Identity activation */
    }
  }
}

static int gemv_impl(int elem, uint16_t *y, const void *W, const uint16_t *x, const uint16_t *scale,
                     const void *zero, const uint16_t *bias, int zero_kind, int n_out, int m_batch,
                     int k, int group_size, int quant_op, int bits, int threads) {
  if (bits != 4 && bits != 8) return -1;
  if (quant_op < 1 || quant_op > 3) return -1;
  if (quant_op == ORC_PER_COLUMN_SCALE_ONLY) group_size = k;
  if (quant_op != ORC_FINEGRAINED_SCALE_AND_ZEROS) zero_kind = ORC_ZERO_NONE;
  if (group_size <= 0) return -1;
  if (threads <= 1) {
    gemv_rows(elem, y, W, x, scale, zero, bias, zero_kind, n_out, m_batch, k, group_size, bits, 0, n_out);
    return 0;
  }
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads)
#endif
  for (int n0 = 0; n0 < n_out; n0 += 16) {
    int n1 = n0 + 16 < n_out ? n0 + 16 : n_out;
    gemv_rows(elem, y, W, x, scale, zero, bias, zero_kind, n_out, m_batch, k, group_size, bits, n0, n1);
  }
  return 0;
}

ORC_API int orc_gemv(uint16_t *y, const void *W, const uint16_t *x, const uint16_t *scale,
                     const void *zero, const uint16_t *bias, int zero_kind, int n_out, int m_batch,
                     int k, int group_size, int quant_op, int bits, int threads) {
  return gemv_impl(ORC_ELEM_F16, y, W, x, scale, zero, bias, zero_kind, n_out, m_batch, k, group_size, quant_op, bits,
                   threads);
}
/* The same loop with bfloat16 as ElementB / ElementScale / ElementOutput (host/mixed_gemv.h:24-31). */
ORC_API int orc_gemv_bf16(uint16_t *y, const void *W, const uint16_t *x, const uint16_t *scale,
                          const void *zero, const uint16_t *bias, int zero_kind, int n_out, int m_batch,
                          int k, int group_size, int quant_op, int bits, int threads) {
  return gemv_impl(ORC_ELEM_BF16, y, W, x, scale, zero, bias, zero_kind, n_out, m_batch, k, group_size, quant_op, bits,
                   threads);
}

ORC_API int orc_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------------------ */
/* deterministic, counter-based input generator (the reference seeds from                */
/* std::random_device, utils/initializer.h:37-38, which cannot be reproduced).           */
/* value i of a stream depends only on (seed, i).                                        */
/* ------------------------------------------------------------------------------------ */

static inline uint64_t mix64(uint64_t z) { /* splitmix64 finaliser */
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}
static inline uint64_t draw(uint64_t seed, uint64_t i) { return mix64(mix64(seed) + i * 0x9e3779b97f4a7c15ull); }

/* uniform integers in [lo, hi] */
ORC_API void orc_fill_int8(int8_t *out, size_t n, uint64_t seed, int lo, int hi) {
  uint64_t range = (uint64_t)(hi - lo + 1);
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    uint64_t r = draw(seed, i) >> 32;
    out[i] = (int8_t)(lo + (int)((r * range) >> 32));
  }
}

/* uniform [lo, hi) drawn in binary32 then rounded to binary16 */
ORC_API void orc_fill_uniform_f16(uint16_t *out, size_t n, uint64_t seed, float lo, float hi) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float u = (float)(draw(seed, i) >> 40) * (1.0f / 16777216.0f);
    out[i] = orc_f32_to_f16(lo + (hi - lo) * u);
  }
}

/* approximately N(0,1) (sum of 12 uniforms - 6, exact in binary32 up to the final
 * roundings of the additions), clipped to [-clip, clip], rounded to binary16 */
ORC_API void orc_fill_normal_clipped_f16(uint16_t *out, size_t n, uint64_t seed, float clip) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    float s = 0.0f;
    for (int j = 0; j < 6; ++j) {
      uint64_t r = draw(seed ^ (0xa5a5a5a5ull * (uint64_t)(j + 1)), i);
      s += (float)(r >> 40) * (1.0f / 16777216.0f);
      s += (float)((r >> 16) & 0xffffffu) * (1.0f / 16777216.0f);
    }
    s -= 6.0f;
    if (s > clip) s = clip;
    if (s < -clip) s = -clip;
    out[i] = orc_f32_to_f16(s);
  }
}
