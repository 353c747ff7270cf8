// Shared declarations of libentropack_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "entropack_hip.h"

namespace ep {

constexpr int kStreams = 17;          // 1 coset stream + 8 fields x 2 cosets
constexpr int kFieldStreams = 16;
constexpr int kFields = 8;
constexpr int kStatesPerTile = 32;    // interleaved rANS lanes per tile, fixed by the bitstream
constexpr uint32_t kStateMin = 1u << 15;
constexpr int kMetaWidth = 4;         // (n_symbols, sym_min, freq_offset, alphabet)

// Plan buffer: a 256-byte header of u32 words, then the tables.
constexpr uint32_t kPlanMagic = 0x45504C54u;
constexpr int kHdrMagic = 0, kHdrKind = 1, kHdrProbBits = 2, kHdrCosetFreq0 = 3, kHdrSymMin = 4, kHdrAlphabet = 21;
constexpr int kHeaderWords = 64;
constexpr size_t kHeaderBytes = kHeaderWords * 4;

// LDS_BYTE entry: freq[0:12) | (slot - cdf)[12:23) | value as a signed byte [24:32)
// LDS_WIDE entry: freq[0:11) | (slot - cdf)[11:22) | symbol[22:32)
// GLOBAL64 entry: symbol[0:16) | freq[16:32) | (slot - cdf)[32:64)

// Payload ring kept in LDS per tile by the LDS-table kernels: 2 chunks of 64 words.
constexpr int kRingWords = 192;       // a stream's LDS window: three chunks of 64 payload words
constexpr int kRingBytes = kRingWords * 2;
constexpr int kChunkWords = 64;

void set_runtime_error(hipError_t e);
// Address of the current device's static accumulator (ep_hip_linear_fused_bf16_static), resolved on first use per device.
int static_accumulator(float** address);

#define EP_HIP_TRY(expr)                         \
  do {                                           \
    hipError_t ep_try_status_ = (expr);          \
    if (ep_try_status_ != hipSuccess) {          \
      ::ep::set_runtime_error(ep_try_status_);   \
      return EP_HIP_ERUNTIME;                    \
    }                                            \
  } while (0)

inline int tile_vectors_of(int tile_elements) {
  const int v = tile_elements / 9;
  return v > 32 ? v : 32;
}
// Largest tile the LDS-table kernels take (plans for larger tiles use the global tables).
constexpr int kMaxLdsTileVectors = 1 << 18;

// LDS_RANK plan layout after the header: FB u32[P] | VAL i16[P] | RS {u32 bits, u32 count}[16][2^pb / 32], each part
// starting on a multiple of 16 bytes and RS on a multiple of one stream's RS size (its base is OR-ed with word offsets).
inline size_t rank_fb_bytes(int present) { return (static_cast<size_t>(present) * 4 + 15) / 16 * 16; }
inline size_t rank_val_bytes(int present) { return (static_cast<size_t>(present) * 2 + 15) / 16 * 16; }
inline size_t rank_rs_stream_bytes(int prob_bits) { return (size_t{1} << prob_bits) / 32 * 8; }
inline size_t rank_rs_offset(int present, int prob_bits) {
  const size_t unit = rank_rs_stream_bytes(prob_bits);
  return (rank_fb_bytes(present) + rank_val_bytes(present) + unit - 1) / unit * unit;
}
inline size_t rank_table_bytes(int present, int prob_bits) {
  return rank_rs_offset(present, prob_bits) + kFieldStreams * rank_rs_stream_bytes(prob_bits);
}

// LDS_SYM section, staged at LDS offset 0: FB u64[16][256], indexed by value + 128, then SLOT u8[16][2048] = value + 128
// (the first 2^pb slots of each are used). An FB entry is
//   word 0: freq | 0x3C000000 when the value is odd  (the multiply takes the low 24 bits; the high halves of seven such
//           words XOR to the parity of z0..z6 as a half-precision 0.0 or 1.0)
//   word 1: (cdf + 2048 * coset) | half(coordinate) << 16  (the decode step forms slot | 2048 * coset, both as the slot
//           table's address and as the number the low half is subtracted from; the high half is the lattice coordinate
//           value + coset / 2 (for the last field, whose coordinate is 2 m + parity + coset / 2: m + coset / 4), which a
//           mixed-precision multiply-add takes without a conversion).
// A field's two cosets lie 2048 bytes apart in both parts, so one per-lane offset serves both lookups.
constexpr int kSymFbStreamBytes = 256 * 8;
constexpr int kSymFbBytes = kFieldStreams * kSymFbStreamBytes;
constexpr int kSymSlotStreamBytes = 2048;
static_assert(kSymSlotStreamBytes == kSymFbStreamBytes, "one coset offset addresses both parts");
constexpr int sym_table_bytes(int /*prob_bits*/) { return kSymFbBytes + kFieldStreams * kSymSlotStreamBytes; }
inline int lds_sym_decode_bytes(int prob_bits, int waves) { return sym_table_bytes(prob_bits) + waves * 2 * kRingBytes + 256; }

// LDS bytes the LDS-table decode kernel needs for `waves` wavefronts each carrying `ilp` tile pairs.
inline int lds_decode_bytes(int prob_bits, int waves, int ilp) {
  return (kFieldStreams << prob_bits) * 4 + waves * ilp * 2 * kRingBytes + 256;
}
inline int lds_rank_decode_bytes_of(int table_bytes, int waves) {
  return (table_bytes + 255) / 256 * 256 + waves * 2 * kRingBytes + 256;
}
inline int lds_rank_decode_bytes(int present, int prob_bits, int waves) {
  return lds_rank_decode_bytes_of(static_cast<int>(rank_table_bytes(present, prob_bits)), waves);
}

}  // namespace ep
