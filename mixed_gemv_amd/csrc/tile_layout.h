// Weight tile layout for 64-lane wavefronts and 128-bit loads on gfx950.
//
// This is the layout descriptor that takes the place of the reference's
// RowMajorTileInterleave<8,4> tag (layout/tile_interleaved_layout.h:42-47) and of the
// interleave arithmetic in utils/preprocess.h:292-348, 365-455.  It is shared by the host
// preprocessor and the device kernels so that the two cannot disagree.
//
// The n_out x k weight matrix is cut into UNITS of 16 rows x kStepK reduction elements.
// A unit is 4096 contiguous bytes = 4 BLOCKS of 1024 bytes; one block is exactly what one
// wavefront fetches with a single 128-bit-per-lane load (64 lanes x 16 bytes), so every wave
// load is one contiguous KiB and a wave that walks consecutive units streams one contiguous
// range.  Units are stored tile-major: unit (t, s) of row tile t and k step s starts at byte
// (t * ksteps + s) * 4096.
//
// Inside a unit, lane l of block i holds the 16-byte CHUNK of
//     row  16 t + (l % 16)
//     k    s*kStepK + (l / 16)*kRunK + i*kChunkK ... + kChunkK
// so lane l owns one row and, over the 4 blocks, one contiguous RUN of kRunK reduction
// elements of that row (128 for int4, 64 for int8): with a group size of 128 a lane needs a
// single scale/zero pair per unit.  The 16 lanes of a DPP row own 16 different rows at the
// SAME k range, so the activations of that range are held one piece per lane and handed
// round with DPP row broadcasts instead of being loaded 16 times.  The same arrangement
// (lane % 16 = row, lane / 16 = k slice) is the operand shape of the 16x16 matrix-core
// instructions, so the small-batch path consumes the identical buffer.
//
// A chunk is four 32-bit words in ascending k.  int4: a word holds 8 consecutive elements,
// each stored biased (value + 8) as a 4-bit field whose least significant bit sits at bit
// int4_field_shift(e) of the word (the field of element 5 wraps round from bit 31 to bits 0-2):
//     e      0   1   2   3   4   5   6   7
//     bits  7-10 23-26 3-6 19-22 15-18 31,0-2 11-14 27-30
// The k-adjacent pair (2h, 2h+1) always lands at the SAME position of the two 16-bit halves,
// either at bits 7-10 or at bits 3-6 of the half, directly (h = 0, 1) or after rotating the
// word right by 8 (h = 2, 3).  Read as fp16, a half-word that is zero outside bits 0-10 has
// the value (bits) * 2^-24 -- exponent fields 0 and 1 continue each other linearly -- so one
// AND yields the packed pair (u * 2^-17, u' * 2^-17) or (u * 2^-21, u' * 2^-21) with no
// integer-to-float conversion at all; the kernels fold the missing power of two into the scale.
// int8: a word holds 4 consecutive elements in natural byte order, stored biased (value + 128).
//
// Rows are padded to a multiple of 16 and k to a multiple of kStepK with zero bytes; padded
// positions are never multiplied by a non-zero activation.
#ifndef MIXED_GEMV_AMD_TILE_LAYOUT_H_
#define MIXED_GEMV_AMD_TILE_LAYOUT_H_

#include <stddef.h>
#include <stdint.h>

#if defined(__HIPCC__)
#define MGEMV_HD __host__ __device__ inline
#else
#define MGEMV_HD inline
#endif

namespace mgemv {

constexpr int kTileRows = 16;       // rows per tile = lanes per DPP row
constexpr int kKSlices = 4;         // k slices per unit = DPP rows per wave
constexpr int kBlocksPerUnit = 4;   // wave loads per unit
constexpr int kChunkBytes = 16;     // one lane, one load
constexpr int kBlockBytes = 1024;   // one wave, one load
constexpr int kUnitBytes = kBlocksPerUnit * kBlockBytes;

template <int BITS>
struct Geometry {
  static_assert(BITS == 4 || BITS == 8, "int4 or int8 weights");
  static constexpr int kChunkK = kChunkBytes * 8 / BITS;        // 32 | 16
  static constexpr int kRunK = kBlocksPerUnit * kChunkK;        // 128 | 64
  static constexpr int kStepK = kKSlices * kRunK;               // 512 | 256
  static constexpr int kWordK = 32 / BITS;                      // 8 | 4
};

MGEMV_HD int chunk_k(int bits) { return kChunkBytes * 8 / bits; }
MGEMV_HD int run_k(int bits) { return kBlocksPerUnit * chunk_k(bits); }
MGEMV_HD int step_k(int bits) { return kKSlices * run_k(bits); }
MGEMV_HD int num_tiles(int n_out) { return (n_out + kTileRows - 1) / kTileRows; }
MGEMV_HD int num_ksteps(int k, int bits) { return (k + step_k(bits) - 1) / step_k(bits); }
MGEMV_HD size_t preprocessed_bytes(size_t n_out, size_t k, int bits) {
  size_t t = (n_out + kTileRows - 1) / kTileRows;
  size_t s = (k + (size_t)step_k(bits) - 1) / (size_t)step_k(bits);
  return t * s * (size_t)kUnitBytes;
}

// Byte offset of the chunk holding (row n, reduction index k0), k0 a multiple of kChunkK.
MGEMV_HD size_t chunk_offset(size_t n, size_t k0, size_t ksteps, int bits) {
  const size_t ck = (size_t)chunk_k(bits), rk = (size_t)run_k(bits), sk = (size_t)step_k(bits);
  size_t t = n / kTileRows, r = n % kTileRows;
  size_t s = k0 / sk, kk = k0 % sk;
  size_t slice = kk / rk, blk = (kk % rk) / ck;
  size_t lane = slice * kTileRows + r;
  return (t * ksteps + s) * (size_t)kUnitBytes + blk * (size_t)kBlockBytes + lane * (size_t)kChunkBytes;
}

// int4 word: natural order (element e in bits 4e..4e+3, two's complement) <-> stored order.
MGEMV_HD uint32_t rotl32(uint32_t v, int s) { return s ? (v << s) | (v >> (32 - s)) : v; }
MGEMV_HD uint32_t rotr32(uint32_t v, int s) { return s ? (v >> s) | (v << (32 - s)) : v; }
MGEMV_HD int int4_field_shift(int e) {
  return e == 0 ? 7 : e == 1 ? 23 : e == 2 ? 3 : e == 3 ? 19 : e == 4 ? 15 : e == 5 ? 31 : e == 6 ? 11 : 27;
}
// Straight-line forms of "field e moves from bit 4e to bit int4_field_shift(e)" (the host
// preprocessor spends its time here).
MGEMV_HD uint32_t encode_int4_word(uint32_t natural) {
  const uint32_t b = natural ^ 0x88888888u;  // +8 on each two's-complement nibble
  return ((b & 0x0000000fu) << 7) | ((b & 0x000000f0u) << 19) | ((b & 0x00000f00u) >> 5) | ((b & 0x0000f000u) << 7) |
         ((b & 0x000f0000u) >> 1) | rotl32(b & 0x00f00000u, 11) | ((b & 0x0f000000u) >> 13) | ((b & 0xf0000000u) >> 1);
}
MGEMV_HD uint32_t decode_int4_word(uint32_t stored) {
  const uint32_t w = stored;
  const uint32_t b = ((w >> 7) & 0x0000000fu) | ((w >> 19) & 0x000000f0u) | ((w << 5) & 0x00000f00u) |
                     ((w >> 7) & 0x0000f000u) | ((w << 1) & 0x000f0000u) | (rotr32(w, 11) & 0x00f00000u) |
                     ((w << 13) & 0x0f000000u) | ((w << 1) & 0xf0000000u);
  return b ^ 0x88888888u;
}
MGEMV_HD uint32_t encode_int8_word(uint32_t natural) { return natural ^ 0x80808080u; }
MGEMV_HD uint32_t decode_int8_word(uint32_t stored) { return stored ^ 0x80808080u; }

}  // namespace mgemv

#endif  // MIXED_GEMV_AMD_TILE_LAYOUT_H_
