// Host-side utilities of the library: int4 packing, zero-point folding and the weight
// preprocessor that produces the gfx950 tile layout.  They stand in for
// utils/preprocess.h:41-84 (SubBytePacker), :94-101 (ZeroPointPreprocessor) and :482-522
// (MixedGemvWeightPreprocessor::run) of the reference: same inputs, same meaning, new layout.
#include <cstring>
#include <vector>

#include "mixed_gemv.h"
#include "tile_layout.h"

namespace {

// ---- binary16 helpers (host) ---------------------------------------------------------------

inline uint32_t bits_of(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float float_of(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

// Exact widening binary16 -> binary32 through a power-of-two rescale.
inline float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t body = (uint32_t)(h & 0x7fffu);
  if (body >= 0x7c00u) return float_of(sign | 0x7f800000u | ((body & 0x3ffu) << 13));
  // Place exponent+mantissa in the binary32 fields, then multiply by 2^(127-15) = 2^112:
  // exact for normals, and it normalises subnormals for free.
  const float scaled = float_of(body << 13) * float_of(0x77800000u);
  return float_of(sign | bits_of(scaled));
}

// binary32 -> binary16, round-to-nearest-even.
inline uint16_t float_to_half_bits(float f) {
  uint32_t x = bits_of(f);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x >= 0x47800000u) {  // |f| >= 65536, inf or nan
    return (uint16_t)(sign | (x > 0x7f800000u ? 0x7e00u : 0x7c00u));
  }
  if (x < 0x38800000u) {  // |f| < 2^-14: the result is subnormal (or zero)
    // Adding 0.5 shifts the value so that the binary32 unit in the last place is 2^-24,
    // the subnormal half spacing; the hardware's RNE does the rounding.
    const float shifted = float_of(x) + 0.5f;
    return (uint16_t)(sign | (bits_of(shifted) - 0x3f000000u));
  }
  const uint32_t odd = (x >> 13) & 1u;
  x += 0xc8000fffu;  // rebias exponent by (15 - 127) and add the rounding bias 0xfff
  x += odd;          // ties go to even
  return (uint16_t)(sign | (x >> 13));
}

bool shape_ok(const size_t* shape, int rank, size_t& experts, size_t& k, size_t& n_out) {
  if (shape == nullptr || (rank != 2 && rank != 3)) return false;
  experts = rank == 2 ? 1 : shape[0];
  k = rank == 2 ? shape[0] : shape[1];
  n_out = rank == 2 ? shape[1] : shape[2];
  return true;
}

int bits_of_quant_type(int quant_type) {
  if (quant_type == MGEMV_W4_A16) return 4;
  if (quant_type == MGEMV_W8_A16) return 8;
  return 0;
}

// Transpose a [k][n_out] matrix of `bits`-wide elements into [n_out][k] (both densely packed,
// low nibble = even index).  Blocked so that both sides are walked in cache-sized tiles.
void transpose_quantised(uint8_t* dst, const uint8_t* src, size_t k, size_t n_out, int bits) {
  constexpr size_t kBlock = 64;
  const long long n_blocks = (long long)((n_out + kBlock - 1) / kBlock);
  // one thread per block of 64 output rows: no two threads write the same byte (k is even)
#pragma omp parallel for schedule(static)
  for (long long nb = 0; nb < n_blocks; ++nb) {
    const size_t n0 = (size_t)nb * kBlock;
    const size_t n1 = n0 + kBlock < n_out ? n0 + kBlock : n_out;
    if (bits == 4) std::memset(dst + n0 * k / 2, 0, (n1 - n0) * k / 2);
    for (size_t k0 = 0; k0 < k; k0 += kBlock) {
      const size_t k1 = k0 + kBlock < k ? k0 + kBlock : k;
      if (bits == 8) {
        for (size_t n = n0; n < n1; ++n)
          for (size_t kk = k0; kk < k1; ++kk) dst[n * k + kk] = src[kk * n_out + n];
      } else {
        for (size_t n = n0; n < n1; ++n)
          for (size_t kk = k0; kk < k1; ++kk) {
            const size_t si = kk * n_out + n;
            const uint8_t v = (uint8_t)((src[si >> 1] >> (4 * (si & 1))) & 0xfu);
            const size_t di = n * k + kk;
            dst[di >> 1] = (uint8_t)(dst[di >> 1] | (v << (4 * (di & 1))));
          }
      }
    }
  }
}

// Walks the chunks of row n in ascending k and hands each (source byte offset inside the row,
// byte offset inside the tiled buffer, bytes of the chunk that lie inside the row -- fewer than 16
// only for the last chunk of a row whose k is not a multiple of the chunk) to `visit`; nested
// loops instead of chunk_offset() keep integer divisions out of the inner loop.
template <typename Visit>
inline void for_each_chunk_of_row(size_t n, size_t k, size_t ksteps, int bits, Visit visit) {
  const size_t ck = (size_t)mgemv::chunk_k(bits);
  const size_t tile = n / mgemv::kTileRows, r = n % mgemv::kTileRows;
  size_t k0 = 0;
  for (size_t s = 0; s < ksteps && k0 < k; ++s) {
    const size_t unit = (tile * ksteps + s) * (size_t)mgemv::kUnitBytes;
    for (size_t slice = 0; slice < (size_t)mgemv::kKSlices && k0 < k; ++slice) {
      const size_t lane_off = (slice * mgemv::kTileRows + r) * (size_t)mgemv::kChunkBytes;
      for (size_t blk = 0; blk < (size_t)mgemv::kBlocksPerUnit && k0 < k; ++blk, k0 += ck)
        visit(k0 * (size_t)bits / 8, unit + blk * (size_t)mgemv::kBlockBytes + lane_off,
              (k - k0 < ck ? k - k0 : ck) * (size_t)bits / 8);
    }
  }
}

// One matrix: rows of k elements (n_out rows) -> tile layout.
void tile_one_matrix(uint8_t* dst, const uint8_t* src, size_t n_out, size_t k, int bits) {
  const size_t ksteps = (size_t)mgemv::num_ksteps((int)k, bits);
  const size_t row_bytes = k * (size_t)bits / 8;
  // zero bytes only where the layout pads: whole rows past n_out, reduction positions past k
  if (n_out % mgemv::kTileRows != 0 || k % (size_t)mgemv::step_k(bits) != 0) {
    const size_t total = mgemv::preprocessed_bytes(n_out, k, bits), piece = (size_t)1 << 20;
#pragma omp parallel for schedule(static)
    for (long long off = 0; off < (long long)total; off += (long long)piece)
      std::memset(dst + off, 0, total - (size_t)off < piece ? total - (size_t)off : piece);
  }
#pragma omp parallel for schedule(static)
  for (long long n = 0; n < (long long)n_out; ++n) {
    const uint8_t* row = src + (size_t)n * row_bytes;
    for_each_chunk_of_row((size_t)n, k, ksteps, bits, [&](size_t src_off, size_t dst_off, size_t valid) {
      uint32_t words[4] = {0, 0, 0, 0};  // positions past k: any value, they only ever meet zero activations
      std::memcpy(words, row + src_off, valid);
      if (bits == 4) {
        for (int j = 0; j < 4; ++j) words[j] = mgemv::encode_int4_word(words[j]);
      } else {
        for (int j = 0; j < 4; ++j) words[j] = mgemv::encode_int8_word(words[j]);
      }
      std::memcpy(dst + dst_off, words, mgemv::kChunkBytes);
    });
  }
}

void untile_one_matrix(uint8_t* dst, const uint8_t* src, size_t n_out, size_t k, int bits) {
  const size_t ksteps = (size_t)mgemv::num_ksteps((int)k, bits);
  const size_t row_bytes = k * (size_t)bits / 8;
#pragma omp parallel for schedule(static)
  for (long long n = 0; n < (long long)n_out; ++n) {
    uint8_t* row = dst + (size_t)n * row_bytes;
    for_each_chunk_of_row((size_t)n, k, ksteps, bits, [&](size_t row_off, size_t tiled_off, size_t valid) {
      uint32_t words[4];
      std::memcpy(words, src + tiled_off, mgemv::kChunkBytes);
      if (bits == 4) {
        for (int j = 0; j < 4; ++j) words[j] = mgemv::decode_int4_word(words[j]);
      } else {
        for (int j = 0; j < 4; ++j) words[j] = mgemv::decode_int8_word(words[j]);
      }
      std::memcpy(row + row_off, words, valid);
    });
  }
}

int check_dims(size_t n_out, size_t k, int bits) {
  if (n_out == 0 || k == 0) return MGEMV_ERR_SIZE;
  if (n_out % 4) return MGEMV_ERR_ROWS;                          // utils/preprocess.h:319-322
  if (k % 8) return MGEMV_ERR_COLS;                              // utils/preprocess.h:324-327
  if (n_out > 0x7fffffffull || k > 0x7fffffffull) return MGEMV_ERR_SIZE;
  return MGEMV_OK;
}

}  // namespace

extern "C" {

int mgemv_pack_int4(uint8_t* packed, const int8_t* unpacked, size_t n_unpacked) {
  if (n_unpacked == 0) return MGEMV_OK;
  if (packed == nullptr || unpacked == nullptr) return MGEMV_ERR_NULL_POINTER;
  if (n_unpacked % 2) return MGEMV_ERR_SIZE;  // two elements per byte
  const size_t n_bytes = n_unpacked / 2;
  for (size_t i = 0; i < n_bytes; ++i) {
    const unsigned lo = (unsigned)unpacked[2 * i] & 0xfu;
    const unsigned hi = (unsigned)unpacked[2 * i + 1] & 0xfu;
    packed[i] = (uint8_t)(lo | (hi << 4));
  }
  return MGEMV_OK;
}

int mgemv_unpack_int4(int8_t* unpacked, const uint8_t* packed, size_t n_packed) {
  if (n_packed == 0) return MGEMV_OK;
  if (packed == nullptr || unpacked == nullptr) return MGEMV_ERR_NULL_POINTER;
  for (size_t i = 0; i < n_packed; ++i) {
    const int lo = packed[i] & 0xf, hi = packed[i] >> 4;
    unpacked[2 * i] = (int8_t)(lo >= 8 ? lo - 16 : lo);
    unpacked[2 * i + 1] = (int8_t)(hi >= 8 ? hi - 16 : hi);
  }
  return MGEMV_OK;
}

int mgemv_fold_zero_points(uint16_t* out, const uint16_t* scales, const int8_t* zeros, size_t n) {
  if (n == 0) return MGEMV_OK;
  if (out == nullptr || scales == nullptr || zeros == nullptr) return MGEMV_ERR_NULL_POINTER;
  for (size_t i = 0; i < n; ++i) {
    // -z is an integer of magnitude <= 128: exact in binary16.  The binary32 product of two
    // halves is exact, so one rounding to binary16 is the correctly rounded fp16 multiply.
    const float neg_z = (float)(-(int)zeros[i]);
    out[i] = float_to_half_bits(neg_z * half_bits_to_float(scales[i]));
  }
  return MGEMV_OK;
}

int mgemv_fold_zero_points_bf16(uint16_t* out, const uint16_t* scales, const int8_t* zeros, size_t n) {
  if (n == 0) return MGEMV_OK;
  if (out == nullptr || scales == nullptr || zeros == nullptr) return MGEMV_ERR_NULL_POINTER;
  for (size_t i = 0; i < n; ++i) {
    // -z has at most 8 significant bits: exact in bfloat16.  The binary32 product of two
    // bfloat16 values is exact, so one rounding (nearest even) is the correctly rounded multiply.
    const uint32_t s_bits = (uint32_t)scales[i] << 16;
    float s;
    std::memcpy(&s, &s_bits, 4);
    const float prod = (float)(-(int)zeros[i]) * s;
    uint32_t bits;
    std::memcpy(&bits, &prod, 4);
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
      out[i] = (uint16_t)((bits >> 16) | 0x0040u);  // NaN stays NaN
    } else {
      out[i] = (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
    }
  }
  return MGEMV_OK;
}

size_t mgemv_preprocessed_size(const size_t* shape, int rank, int quant_type) {
  size_t experts, k, n_out;
  const int bits = bits_of_quant_type(quant_type);
  if (bits == 0 || !shape_ok(shape, rank, experts, k, n_out)) return 0;
  return experts * mgemv::preprocessed_bytes(n_out, k, bits);
}

int mgemv_preprocess_weights(uint8_t* dst, const uint8_t* src, const size_t* shape, int rank, int layout,
                             int quant_type) {
  if (dst == nullptr || src == nullptr || shape == nullptr) return MGEMV_ERR_NULL_POINTER;
  size_t experts, k, n_out;
  if (!shape_ok(shape, rank, experts, k, n_out)) return MGEMV_ERR_RANK;
  const int bits = bits_of_quant_type(quant_type);
  if (bits == 0) return MGEMV_ERR_QUANT_TYPE;
  if (layout != MGEMV_ROW_MAJOR && layout != MGEMV_COLUMN_MAJOR) return MGEMV_ERR_LAYOUT;
  if (const int st = check_dims(n_out, k, bits)) return st;

  const size_t src_bytes = n_out * k * (size_t)bits / 8;
  const size_t dst_bytes = mgemv::preprocessed_bytes(n_out, k, bits);
  std::vector<uint8_t> transposed;
  if (layout == MGEMV_ROW_MAJOR) transposed.resize(src_bytes);
  for (size_t e = 0; e < experts; ++e) {
    const uint8_t* matrix = src + e * src_bytes;
    if (layout == MGEMV_ROW_MAJOR) {
      transpose_quantised(transposed.data(), matrix, k, n_out, bits);
      matrix = transposed.data();
    }
    tile_one_matrix(dst + e * dst_bytes, matrix, n_out, k, bits);
  }
  return MGEMV_OK;
}

int mgemv_unpreprocess_weights(uint8_t* dst, const uint8_t* src_preprocessed, const size_t* shape, int rank,
                               int quant_type) {
  if (dst == nullptr || src_preprocessed == nullptr || shape == nullptr) return MGEMV_ERR_NULL_POINTER;
  size_t experts, k, n_out;
  if (!shape_ok(shape, rank, experts, k, n_out)) return MGEMV_ERR_RANK;
  const int bits = bits_of_quant_type(quant_type);
  if (bits == 0) return MGEMV_ERR_QUANT_TYPE;
  if (const int st = check_dims(n_out, k, bits)) return st;
  const size_t raw_bytes = n_out * k * (size_t)bits / 8;
  const size_t tiled_bytes = mgemv::preprocessed_bytes(n_out, k, bits);
  for (size_t e = 0; e < experts; ++e)
    untile_one_matrix(dst + e * raw_bytes, src_preprocessed + e * tiled_bytes, n_out, k, bits);
  return MGEMV_OK;
}

const char* mgemv_status_string(int status) {
  switch (status) {
    case MGEMV_OK: return "ok";
    case MGEMV_ERR_NULL_POINTER: return "a required pointer is NULL";
    case MGEMV_ERR_RANK: return "weight shape must be 2-D {k, n_out} or 3-D {experts, k, n_out}";
    case MGEMV_ERR_ROWS: return "n_out must be a multiple of 4";
    case MGEMV_ERR_COLS: return "k must be a multiple of 8";
    case MGEMV_ERR_GROUP_SIZE: return "group_size must be >= 64, a multiple of 32 and divide k";
    case MGEMV_ERR_QUANT_OP: return "quant_op must be 1 (per-column scale), 2 (group scale) or 3 (group scale + zero)";
    case MGEMV_ERR_QUANT_TYPE: return "weights must be int8 (W8_A16) or int4 (W4_A16)";
    case MGEMV_ERR_BATCH: return "batch_count must be >= 1 and m_batch in [1, 16]";
    case MGEMV_ERR_LAYOUT: return "layout must be 0 (row major) or 1 (column major)";
    case MGEMV_ERR_LEADING_DIMENSION: return "a leading dimension or batch stride describes an operand this library does not take (only the reference's dense operands)";
    case MGEMV_ERR_ALLOCATION: return "device memory could not be allocated (host-pointer entry point)";
    case MGEMV_ERR_SCRATCH_SIZE: return "the problem does not fit the static scratch arrays of the allocation-free host-pointer entry point";
    case MGEMV_ERR_SIZE: return "a dimension is zero, negative or exceeds the 32-bit index range of the kernels";
    case MGEMV_ERR_LAUNCH: return "HIP launch failed";
    case MGEMV_ERR_NO_DEVICE: return "no usable gfx950 device";
    case MGEMV_ERR_ALIGNMENT: return "device pointer alignment: weights and activations 16 bytes, scales / zeros / bias / outputs 2 bytes, dequantised output 4 bytes";
    default: return "unknown status";
  }
}

int mgemv_version(void) { return 212; }  // 2xx: int4 fields at bits 7-10 / 3-6 of each half-word

}  // extern "C"
