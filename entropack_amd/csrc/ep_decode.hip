// lattice_rans decode kernels for gfx950: 32-way interleaved rANS entropy decode fused with E8 reconstruction,
// row rescale and the container cast. A tile owns 32 rANS lanes, so one wave64 carries two tiles, one per
// 32-lane half; every ballot/prefix-count is taken per half.
//
//   decode_global64_kernel   any container: u64 slot table read from global memory, payload words read from
//                            global memory with a bounds check on every renormalisation.
//   decode_lds_kernel        prob_bits <= 11: u32 slot table staged in LDS (one gather per symbol), the tile's
//                            payload streamed through a 128-word LDS ring refilled by 64-word prefetches, row
//                            pointers kept in scalar registers, one or two tile pairs interleaved per wave.
//
// Both compute, per vector: coset c from stream 0, fields f = 0..7 from stream 1 + 2f + c, z7 = 2 m + parity,
// w_j = f32_mul(float(z_j) + c / 2, scale[row]) and the container cast of w_j; the result is bit-identical for
// every table representation.
#include <type_traits>

#include "ep_common.hpp"

namespace ep {

struct DecodeArgs {
  const uint16_t* payload;
  uint64_t payload_words;
  const uint32_t* offsets;
  const uint32_t* states;
  const float* scales;
  const uint32_t* plan;     // header + tables
  void* out;
  int store_kind;
  int vecs_per_row;
  uint32_t row_magic;       // row = vecs_per_row == 1 ? v : umulhi(v, row_magic) >> row_shift
  int row_shift;
  int64_t num_vectors;
  int tile_vectors;
  int num_tiles;
  int* error;
};

__device__ __forceinline__ void flag_error(int* error, int code) { atomicCAS(error, 0, code); }

// ---- container casts (format.py:153-168 / lattice_rans.cu:560-653 of the reference) -----------------------

__device__ __forceinline__ uint32_t bf16_bits_rne(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16;      // finite input
}

__device__ __forceinline__ float clamp_bf16(float v) {
  return __builtin_fminf(__builtin_fmaxf(v, -3.3895313892515355e38f), 3.3895313892515355e38f);
}

__device__ __forceinline__ uint32_t f16_bits(float v) {
  const _Float16 h = static_cast<_Float16>(__builtin_fminf(__builtin_fmaxf(v, -65504.0f), 65504.0f));
  return __builtin_bit_cast(unsigned short, h);
}

// Round-to-nearest-even float -> OCP fp8 after saturating to the largest finite value.
template <int MBITS, int BIAS>
__device__ __forceinline__ uint32_t fp8_bits(float v, float limit) {
  const uint32_t sign = (__float_as_uint(v) >> 24) & 0x80u;
  float a = __builtin_fminf(__builtin_fabsf(v), limit);
  const float min_normal = __uint_as_float(static_cast<uint32_t>(127 + 1 - BIAS) << 23);
  if (!(a >= min_normal)) {
    const float quantum = __uint_as_float(static_cast<uint32_t>(127 + 1 - BIAS - MBITS) << 23);
    return sign | static_cast<uint32_t>(__builtin_rintf(a / quantum));
  }
  const uint32_t bits = __float_as_uint(a);
  const int exponent = static_cast<int>(bits >> 23) - 127 + BIAS;
  constexpr int kShift = 23 - MBITS;
  const uint32_t mant = bits & 0x7FFFFFu;
  uint32_t r = mant >> kShift;
  const uint32_t rest = mant & ((1u << kShift) - 1u);
  constexpr uint32_t kHalf = 1u << (kShift - 1);
  r += (rest > kHalf) || (rest == kHalf && (r & 1u));
  return sign | ((static_cast<uint32_t>(exponent) << MBITS) + r);
}

template <typename T>
__device__ __forceinline__ T snap_integer(float v, float low, float high_exclusive) {
  const float high = __uint_as_float(__float_as_uint(high_exclusive) - 1u);   // nextafter(high_exclusive, 0)
  return static_cast<T>(__builtin_fminf(__builtin_fmaxf(__builtin_rintf(v), low), high));
}

// Writes the eight values of vector `vector` in any container kind.
__device__ __forceinline__ void store_vector(void* out, int kind, int64_t vector, const float (&w)[8]) {
  switch (kind) {
    case EP_STORE_BF16: {
      uint32_t p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = bf16_bits_rne(clamp_bf16(w[2 * i])) | (bf16_bits_rne(clamp_bf16(w[2 * i + 1])) << 16);
      reinterpret_cast<uint4*>(out)[vector] = make_uint4(p[0], p[1], p[2], p[3]);
      break;
    }
    case EP_STORE_F16: {
      uint32_t p[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = f16_bits(w[2 * i]) | (f16_bits(w[2 * i + 1]) << 16);
      reinterpret_cast<uint4*>(out)[vector] = make_uint4(p[0], p[1], p[2], p[3]);
      break;
    }
    case EP_STORE_F32: {
      float4* dst = reinterpret_cast<float4*>(out) + vector * 2;
      dst[0] = make_float4(w[0], w[1], w[2], w[3]);
      dst[1] = make_float4(w[4], w[5], w[6], w[7]);
      break;
    }
    case EP_STORE_F8E4M3FN:
    case EP_STORE_F8E5M2:
    case EP_STORE_I8:
    case EP_STORE_U8:
    case EP_STORE_BOOL: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (kind == EP_STORE_F8E4M3FN) b[i] = fp8_bits<3, 7>(w[i], 448.0f);
        else if (kind == EP_STORE_F8E5M2) b[i] = fp8_bits<2, 15>(w[i], 57344.0f);
        else if (kind == EP_STORE_I8) b[i] = static_cast<uint8_t>(snap_integer<int8_t>(w[i], -128.0f, 128.0f));
        else if (kind == EP_STORE_U8) b[i] = snap_integer<uint8_t>(w[i], 0.0f, 256.0f);
        else b[i] = __builtin_rintf(w[i]) != 0.0f;
      }
      reinterpret_cast<uint2*>(out)[vector] =
          make_uint2(b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24), b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
      break;
    }
    case EP_STORE_I16:
    case EP_STORE_U16: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        b[i] = kind == EP_STORE_I16 ? static_cast<uint16_t>(snap_integer<int16_t>(w[i], -32768.0f, 32768.0f))
                                    : snap_integer<uint16_t>(w[i], 0.0f, 65536.0f);
      }
      reinterpret_cast<uint4*>(out)[vector] =
          make_uint4(b[0] | (b[1] << 16), b[2] | (b[3] << 16), b[4] | (b[5] << 16), b[6] | (b[7] << 16));
      break;
    }
    case EP_STORE_I32:
    case EP_STORE_U32: {
      uint32_t b[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        b[i] = kind == EP_STORE_I32 ? static_cast<uint32_t>(snap_integer<int32_t>(w[i], -2147483648.0f, 2147483648.0f))
                                    : snap_integer<uint32_t>(w[i], 0.0f, 4294967296.0f);
      }
      uint4* dst = reinterpret_cast<uint4*>(out) + vector * 2;
      dst[0] = make_uint4(b[0], b[1], b[2], b[3]);
      dst[1] = make_uint4(b[4], b[5], b[6], b[7]);
      break;
    }
    default: {   // EP_STORE_I64 / EP_STORE_U64
      uint64_t* dst = reinterpret_cast<uint64_t*>(out) + vector * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        dst[i] = kind == EP_STORE_I64
                     ? static_cast<uint64_t>(snap_integer<int64_t>(w[i], -9223372036854775808.0f, 9223372036854775808.0f))
                     : snap_integer<uint64_t>(w[i], 0.0f, 18446744073709551616.0f);
      }
      break;
    }
  }
}

__device__ __forceinline__ uint32_t row_of(const DecodeArgs& a, uint32_t vector) {
  return a.vecs_per_row == 1 ? vector : (__umulhi(vector, a.row_magic) >> a.row_shift);
}

// ---- any container: tables and payload in global memory ----------------------------------------------------

__global__ __launch_bounds__(256) void decode_global64_kernel(DecodeArgs a) {
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t tile = 2 * (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) + half;
  const int pb = static_cast<int>(a.plan[kHdrProbBits]);
  const uint32_t slot_mask = (1u << pb) - 1u;
  const uint64_t* lut = reinterpret_cast<const uint64_t*>(reinterpret_cast<const uint8_t*>(a.plan) + kHeaderBytes);
  const int32_t* sym_min = reinterpret_cast<const int32_t*>(a.plan) + kHdrSymMin;

  int64_t word_begin = 0, pointer = 0;
  int count = 0;
  uint32_t x = kStateMin;
  const int64_t vector_begin = tile * a.tile_vectors;
  if (tile < a.num_tiles) {
    word_begin = a.offsets[tile];
    pointer = a.offsets[tile + 1];
    const int64_t left = a.num_vectors - vector_begin;
    count = static_cast<int>(left < a.tile_vectors ? left : a.tile_vectors);
    if (word_begin > pointer || static_cast<uint64_t>(pointer) > a.payload_words) {
      flag_error(a.error, EP_DECODE_BAD_OFFSETS);
      count = 0;
    } else {
      x = a.states[tile * kStatesPerTile + l32];
    }
  }
  const bool checked_tile = count > 0;
  const int groups = (count + 31) >> 5;
  const int rem = count & 31;
  const int other = __shfl_xor(groups, 32);
  const int rounds = groups > other ? groups : other;

  auto renormalise = [&](bool valid) {
    const bool read = valid && x < kStateMin;
    const uint64_t vote = __ballot(read);
    const uint32_t mine = half ? static_cast<uint32_t>(vote >> 32) : static_cast<uint32_t>(vote);
    if (read) {
      const int64_t at = pointer - __popc(mine >> l32);    // readers at or above this lane, itself included
      uint32_t word = 0;
      if (at >= word_begin) word = a.payload[at];
      else flag_error(a.error, EP_DECODE_OVERREAD);
      x = (x << 16) | word;
    }
    pointer -= __popc(mine);
  };

  for (int round = 0; round < rounds; ++round) {
    const bool active = round < groups;
    const int offset = (groups - 1 - round) << 5;
    const int lanes = (round == 0 && rem != 0) ? rem : 32;
    const bool valid = active && l32 < lanes;
    int c = 0;
    int value[8];
    if (valid) {
      const uint32_t slot = x & slot_mask;
      const uint64_t entry = lut[slot];
      c = static_cast<int>(entry & 1u);
      x = (static_cast<uint32_t>(entry >> 16) & 0xFFFFu) * (x >> pb) + static_cast<uint32_t>(entry >> 32);
    }
    renormalise(valid);
#pragma unroll
    for (int f = 0; f < kFields; ++f) {
      if (valid) {
        const int table = 1 + 2 * f + c;
        const uint32_t slot = x & slot_mask;
        const uint64_t entry = lut[(static_cast<size_t>(table) << pb) + slot];
        value[f] = static_cast<int>(entry & 0xFFFFu) + sym_min[table];
        x = (static_cast<uint32_t>(entry >> 16) & 0xFFFFu) * (x >> pb) + static_cast<uint32_t>(entry >> 32);
      }
      renormalise(valid);
    }
    if (valid) {
      int parity = 0;
#pragma unroll
      for (int f = 0; f < 7; ++f) parity += value[f];
      value[7] = 2 * value[7] + (parity & 1);
      const int64_t vector = vector_begin + offset + l32;
      const float scale = a.scales[vector / a.vecs_per_row];
      const float shift = c ? 0.5f : 0.0f;
      float w[8];
#pragma unroll
      for (int f = 0; f < 8; ++f) w[f] = __fmul_rn(__fadd_rn(static_cast<float>(value[f]), shift), scale);
      store_vector(a.out, a.store_kind, vector, w);
    }
  }
  if (checked_tile && (pointer != word_begin || x != kStateMin)) flag_error(a.error, EP_DECODE_NOT_CONSUMED);
}

// ---- prob_bits <= 11: LDS-resident u32 tables, LDS payload ring ----------------------------------------------

template <int PB, bool WIDE>
struct Entry {
  static constexpr int kFreqBits = WIDE ? 11 : 12;
  static constexpr int kDeltaBits = 11;
  static constexpr int kSymShift = WIDE ? 22 : 24;
  __device__ static __forceinline__ uint32_t freq(uint32_t e) { return e & ((1u << kFreqBits) - 1u); }
  __device__ static __forceinline__ uint32_t delta(uint32_t e) { return (e >> kFreqBits) & ((1u << kDeltaBits) - 1u); }
};

// Per-wave state of one tile pair (lower half = tile 2p, upper half = tile 2p + 1). Members named *A / *B are
// wave-uniform (kept in scalar registers); the rest are per lane.
struct PairState {
  uint32_t x;          // rANS state of this lane
  uint32_t prefetch;   // next 64-word payload chunk, one dword (2 words) per lane
  int32_t fetch_dword; // absolute dword index `prefetch` was loaded from
  uint32_t ring;       // LDS byte offset of this half's ring
  uint32_t ring_write; // LDS byte offset where `prefetch` goes on the next refill
  uint32_t vector0;    // first vector of this lane's tile
  int count;           // vectors in this lane's tile
  int ptrA, ptrB;      // payload positions (words, relative to a 64-word aligned base below the tile)
  int limA, limB;      // refill when ptr <= lim
  int beginA, beginB;  // position of the tile's first word
};

template <int PB, bool WIDE, int ILP, int KIND>
__global__ __launch_bounds__(1024) void decode_lds_kernel(DecodeArgs a, int num_pairs) {
  extern __shared__ __align__(16) uint8_t smem[];
  constexpr uint32_t kTable = 1u << PB;
  constexpr uint32_t kLutBytes = (kFieldStreams << PB) * 4;
  using E = Entry<PB, WIDE>;

  const int waves = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6;
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const uint32_t rings0 = kLutBytes;
  const uint32_t minima0 = rings0 + static_cast<uint32_t>(waves) * ILP * 2 * kRingBytes;

  {
    const uint4* src = reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.plan) + kHeaderBytes);
    uint4* dst = reinterpret_cast<uint4*>(smem);
    for (uint32_t i = threadIdx.x; i < kLutBytes / 16; i += blockDim.x) dst[i] = src[i];
    if (threadIdx.x < kStreams) {
      reinterpret_cast<int32_t*>(smem + minima0)[threadIdx.x] = static_cast<int32_t>(a.plan[kHdrSymMin + threadIdx.x]);
    }
  }
  __syncthreads();

  const uint32_t freq0 = a.plan[kHdrCosetFreq0];
  const uint32_t half_shift = half ? 16u : 0u;
  const uint32_t* payload32 = reinterpret_cast<const uint32_t*>(a.payload);

  auto lds_u16 = [&](uint32_t at) -> uint32_t { return *reinterpret_cast<const uint16_t*>(smem + at); };
  auto lds_u32 = [&](uint32_t at) -> uint32_t { return *reinterpret_cast<const uint32_t*>(smem + at); };

  const int stride = gridDim.x * waves * ILP;
  for (int first_pair = (blockIdx.x * waves + wave) * ILP; first_pair < num_pairs; first_pair += stride) {
    PairState st[ILP];
    bool uniform = true;

    // ---- set up each tile: pointers, initial states, first two ring chunks, first prefetch -------------------
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      PairState& s = st[j];
      const int64_t tile = 2 * static_cast<int64_t>(first_pair + j) + half;
      s.ring = rings0 + static_cast<uint32_t>((wave * ILP + j) * 2 + half) * kRingBytes;
      uint32_t word_begin = 0, word_end = 0;
      s.count = 0;
      s.x = kStateMin;
      s.vector0 = 0;
      if (first_pair + j < num_pairs && tile < a.num_tiles) {
        word_begin = a.offsets[tile];
        word_end = a.offsets[tile + 1];
        const int64_t v0 = tile * a.tile_vectors;
        const int64_t left = a.num_vectors - v0;
        s.vector0 = static_cast<uint32_t>(v0);
        s.count = static_cast<int>(left < a.tile_vectors ? left : a.tile_vectors);
        if (word_begin > word_end || word_end > a.payload_words) {
          flag_error(a.error, EP_DECODE_BAD_OFFSETS);
          s.count = 0;
          word_begin = word_end = 0;
        } else {
          s.x = a.states[tile * kStatesPerTile + l32];
        }
      }
      uniform = uniform && s.count == a.tile_vectors;
      const uint32_t base = word_begin & ~63u;               // absolute index of relative position 0
      const int begin = static_cast<int>(word_begin - base);
      const int ptr = static_cast<int>(word_end - base);
      const int low = (((ptr - 1) & ~63)) - 64;              // ring holds relative [low, low + 128)
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int chunk = low + 64 * k;
        const int64_t at = static_cast<int64_t>(base) + chunk + 2 * l32;
        uint32_t lo = 0, hi = 0;
        if (at >= 0 && static_cast<uint64_t>(at) < a.payload_words) lo = a.payload[at];
        if (at + 1 >= 0 && static_cast<uint64_t>(at + 1) < a.payload_words) hi = a.payload[at + 1];
        *reinterpret_cast<uint32_t*>(smem + s.ring + static_cast<uint32_t>(((chunk & 127) + 2 * l32) * 2)) = lo | (hi << 16);
      }
      s.fetch_dword = static_cast<int32_t>((static_cast<int64_t>(base) + low - 64) >> 1) + l32;
      s.prefetch = s.fetch_dword >= 0 ? payload32[s.fetch_dword] : 0u;
      s.ring_write = s.ring + static_cast<uint32_t>((((low - 64) & 127) + 2 * l32) * 2);
      s.ptrA = __builtin_amdgcn_readlane(ptr, 0);
      s.ptrB = __builtin_amdgcn_readlane(ptr, 32);
      s.beginA = __builtin_amdgcn_readlane(begin, 0);
      s.beginB = __builtin_amdgcn_readlane(begin, 32);
      s.limA = __builtin_amdgcn_readlane(low, 0) + 64;
      s.limB = __builtin_amdgcn_readlane(low, 32) + 64;
    }
    const bool all_uniform = __builtin_amdgcn_readfirstlane(__all(uniform) ? 1 : 0) != 0;

    // Shared renormalisation of every interleaved pair: lanes below 2^15 take one word each, in ascending lane
    // order, from just below their half's pointer. Straight-line code (the ring read is unconditional and
    // selected afterwards) so that the interleaved pairs' LDS reads overlap.
    auto renormalise = [&](const bool (&valid)[ILP]) {
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        PairState& s = st[j];
        const bool read = valid[j] && s.x < kStateMin;
        const uint64_t vote = __builtin_amdgcn_ballot_w64(read);
        const uint32_t vote_lo = static_cast<uint32_t>(vote), vote_hi = static_cast<uint32_t>(vote >> 32);
        const int taken_lo = __popc(vote_lo);
        s.ptrA -= taken_lo;
        s.ptrB -= __popc(vote_hi);
        const uint32_t packed = (static_cast<uint32_t>(s.ptrA) & 127u) | ((static_cast<uint32_t>(s.ptrB - taken_lo) & 127u) << 16);
        const uint32_t rank = __builtin_amdgcn_mbcnt_hi(vote_hi, __builtin_amdgcn_mbcnt_lo(vote_lo, packed >> half_shift));
        uint32_t word = lds_u16(s.ring + ((rank & 127u) << 1));
        asm volatile("" : "+v"(word));     // keep the ring read unconditional: no branch around it
        s.x = read ? ((s.x << 16) | word) : s.x;
      }
      // Top the rings up once a pointer has left its upper chunk: the prefetched 64 words go where that chunk
      // was, and the next chunk down is requested. One uniform test per step for all pairs.
      bool any = false;
#pragma unroll
      for (int j = 0; j < ILP; ++j) any = any || st[j].ptrA <= st[j].limA || st[j].ptrB <= st[j].limB;
      if (any) {
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
          PairState& s = st[j];
          const bool needA = s.ptrA <= s.limA, needB = s.ptrB <= s.limB;
          if (half ? needB : needA) {
            *reinterpret_cast<uint32_t*>(smem + s.ring_write) = s.prefetch;
            s.ring_write ^= 128u;
            s.fetch_dword -= 32;
            s.prefetch = s.fetch_dword >= 0 ? payload32[s.fetch_dword] : 0u;
          }
          s.limA -= needA ? 64 : 0;
          s.limB -= needB ? 64 : 0;
        }
      }
    };

    // One group of 32 vectors per half for every interleaved pair. `offset` is the group's first vector within
    // the tile; with MASKED it and `valid` are per lane, otherwise wave-uniform.
    auto decode_group = [&](auto masked_tag, const int (&offset)[ILP], const bool (&valid)[ILP]) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      uint32_t coset_base[ILP];   // byte offset of this lane's coset inside a field's table pair
      uint32_t e[ILP][8];
      bool c[ILP];
      float scale[ILP];
      uint32_t vector[ILP];
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        PairState& s = st[j];
        vector[j] = s.vector0 + static_cast<uint32_t>(offset[j]) + l32;
        const bool ok = !MASKED || valid[j];
        scale[j] = ok ? a.scales[row_of(a, vector[j])] : 0.0f;
        const uint32_t slot = s.x & (kTable - 1u);
        c[j] = ok && slot >= freq0;
        const uint32_t begin = c[j] ? freq0 : 0u;
        const uint32_t freq = c[j] ? kTable - freq0 : freq0;
        const uint32_t next = __umul24(freq, s.x >> PB) + (slot - begin);
        s.x = ok ? next : s.x;
        coset_base[j] = c[j] ? kTable * 4u : 0u;       // tables start at LDS offset 0, each 4 << PB bytes
      }
      renormalise(valid);
#pragma unroll
      for (int f = 0; f < kFields; ++f) {
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
          PairState& s = st[j];
          const uint32_t entry = lds_u32((((s.x << 2) & (kTable * 4u - 4u)) | coset_base[j]) + static_cast<uint32_t>(f) * (kTable * 8u));
          e[j][f] = entry;
          const uint32_t next = __umul24(E::freq(entry), s.x >> PB) + E::delta(entry);
          s.x = (!MASKED || valid[j]) ? next : s.x;
        }
        renormalise(valid);
      }
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        if (MASKED && !valid[j]) continue;
        float p[8];
        if constexpr (!WIDE) {
          // Top byte = value + 128. 7 * 128 is even, so the parity of z0..z6 is the parity of the biased bytes.
          const uint32_t folded = e[j][0] ^ e[j][1] ^ e[j][2] ^ e[j][3] ^ e[j][4] ^ e[j][5] ^ e[j][6];
          const float parity = static_cast<float>((folded >> 24) & 1u);
          const float bias = c[j] ? -127.5f : -128.0f;
#pragma unroll
          for (int f = 0; f < 7; ++f) p[f] = __fadd_rn(static_cast<float>(e[j][f] >> 24), bias);
          p[7] = __fadd_rn(__fmaf_rn(static_cast<float>(e[j][7] >> 24), 2.0f, parity), c[j] ? -255.5f : -256.0f);
        } else {
          const int32_t* minima = reinterpret_cast<const int32_t*>(smem + minima0) + 1 + (c[j] ? 1 : 0);
          int z[8];
#pragma unroll
          for (int f = 0; f < 8; ++f) z[f] = static_cast<int>(e[j][f] >> E::kSymShift) + minima[2 * f];
          const int parity = (z[0] + z[1] + z[2] + z[3] + z[4] + z[5] + z[6]) & 1;
          z[7] = 2 * z[7] + parity;
          const float shift = c[j] ? 0.5f : 0.0f;
#pragma unroll
          for (int f = 0; f < 8; ++f) p[f] = __fadd_rn(static_cast<float>(z[f]), shift);
        }
        float w[8];
#pragma unroll
        for (int f = 0; f < 8; ++f) w[f] = __fmul_rn(p[f], scale[j]);
        if constexpr (KIND == EP_STORE_BF16) {
          // |w| can pass the largest finite bf16 only for scales beyond 1e30; the reference's CPU lane saturates.
          if (__builtin_fabsf(scale[j]) > 1.0e30f) {
#pragma unroll
            for (int f = 0; f < 8; ++f) w[f] = clamp_bf16(w[f]);
          }
          uint32_t packed[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            typedef float float2v __attribute__((ext_vector_type(2)));
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            const float2v pair = {w[2 * i], w[2 * i + 1]};
            packed[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
          }
          reinterpret_cast<uint4*>(a.out)[vector[j]] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        } else {
          store_vector(a.out, a.store_kind, vector[j], w);
        }
      }
    };

    using Masked = std::integral_constant<bool, true>;
    using Unmasked = std::integral_constant<bool, false>;

    if (all_uniform) {
      // Every tile here is full: the schedule is the same for both halves of every pair.
      const int rem = a.tile_vectors & 31;
      int group_offset = a.tile_vectors - rem;
      if (rem != 0) {
        int offset[ILP];
        bool valid[ILP];
#pragma unroll
        for (int j = 0; j < ILP; ++j) { offset[j] = group_offset; valid[j] = l32 < rem; }
        decode_group(Masked{}, offset, valid);
      }
      while (group_offset > 0) {
        group_offset -= 32;
        int offset[ILP];
        bool valid[ILP];
#pragma unroll
        for (int j = 0; j < ILP; ++j) { offset[j] = group_offset; valid[j] = true; }
        decode_group(Unmasked{}, offset, valid);
      }
    } else {
      int groups[ILP];
      int rounds = 0;
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        groups[j] = (st[j].count + 31) >> 5;
        const int other = __shfl_xor(groups[j], 32);
        const int most = groups[j] > other ? groups[j] : other;
        rounds = rounds > most ? rounds : most;
      }
      rounds = __builtin_amdgcn_readfirstlane(rounds);
#pragma unroll 1
      for (int round = 0; round < rounds; ++round) {
        int offset[ILP];
        bool valid[ILP];
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
          const int rem = st[j].count & 31;
          const int lanes = (round == 0 && rem != 0) ? rem : 32;
          offset[j] = (groups[j] - 1 - round) << 5;
          valid[j] = round < groups[j] && l32 < lanes;
        }
        decode_group(Masked{}, offset, valid);
      }
    }

    // A valid tile ends with every word consumed and every lane back at the encoder's initial state.
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      const PairState& s = st[j];
      const uint64_t stale = __ballot(s.count > 0 && s.x != kStateMin);
      const uint64_t live = __ballot(s.count > 0);
      const bool liveA = (live & 1u) != 0, liveB = ((live >> 32) & 1u) != 0;
      const bool badA = liveA && (s.ptrA != s.beginA || static_cast<uint32_t>(stale) != 0);
      const bool badB = liveB && (s.ptrB != s.beginB || static_cast<uint32_t>(stale >> 32) != 0);
      if ((badA || badB) && lane == 0) {
        const bool over = (liveA && s.ptrA < s.beginA) || (liveB && s.ptrB < s.beginB);
        flag_error(a.error, over ? EP_DECODE_OVERREAD : EP_DECODE_NOT_CONSUMED);
      }
    }
  }
}

// ---- host side --------------------------------------------------------------------------------------------------

template <int PB, bool WIDE, int ILP, int KIND>
static int launch_lds(const DecodeArgs& args, int num_pairs, int blocks, int threads, hipStream_t stream) {
  auto kernel = decode_lds_kernel<PB, WIDE, ILP, KIND>;
  const int lds = lds_decode_bytes(PB, threads / 64, ILP);
  static thread_local int configured_for = -1;     // per instantiation: raise the dynamic LDS cap once per device
  int device = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  if (configured_for != device) {
    EP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    configured_for = device;
  }
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, stream, args, num_pairs);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}

template <int PB, bool WIDE>
static int launch_lds_pb(const DecodeArgs& args, int num_pairs, int blocks, int threads, int ilp, hipStream_t stream) {
  const bool bf16 = args.store_kind == EP_STORE_BF16;
  if (ilp == 2) {
    return bf16 ? launch_lds<PB, WIDE, 2, EP_STORE_BF16>(args, num_pairs, blocks, threads, stream)
                : launch_lds<PB, WIDE, 2, -1>(args, num_pairs, blocks, threads, stream);
  }
  return bf16 ? launch_lds<PB, WIDE, 1, EP_STORE_BF16>(args, num_pairs, blocks, threads, stream)
              : launch_lds<PB, WIDE, 1, -1>(args, num_pairs, blocks, threads, stream);
}

}  // namespace ep

extern "C" int ep_hip_decode_lattice(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                                     const uint32_t* states_dev, const float* scales_dev, const void* tables_dev,
                                     const ep_hip_plan_desc* desc, void* out_dev, int store_kind, int64_t rows,
                                     int64_t cols_padded, int tile_elements, int32_t* error_dev, void* stream) {
  using namespace ep;
  if (offsets_dev == nullptr || states_dev == nullptr || scales_dev == nullptr || tables_dev == nullptr ||
      desc == nullptr || out_dev == nullptr || error_dev == nullptr) return EP_HIP_EINVAL;
  if (payload_dev == nullptr && payload_words != 0) return EP_HIP_EINVAL;
  if (rows <= 0 || cols_padded <= 0 || cols_padded % 8 != 0 || tile_elements <= 0) return EP_HIP_EINVAL;
  if (store_kind < EP_STORE_F32 || store_kind > EP_STORE_BF16) return EP_HIP_EINVAL;
  if (desc->prob_bits < 9 || desc->prob_bits > 15) return EP_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(payload_dev) % 4 != 0 || reinterpret_cast<uintptr_t>(out_dev) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(tables_dev) % 256 != 0) return EP_HIP_EINVAL;
  if (payload_words > 0xFFFFFFFFull) return EP_HIP_EINVAL;           // offsets are 32-bit
  const int64_t vecs_per_row = cols_padded / 8;
  if (vecs_per_row > 0x7FFFFFFF) return EP_HIP_EINVAL;
  const int64_t vectors = rows * vecs_per_row;
  const int tv = tile_vectors_of(tile_elements);
  const int64_t tiles = (vectors + tv - 1) / tv;
  if (vectors >= (int64_t{1} << 31) || tiles >= (int64_t{1} << 30)) return EP_HIP_EUNSUPPORTED;

  DecodeArgs args;
  args.payload = payload_dev;
  args.payload_words = payload_words;
  args.offsets = offsets_dev;
  args.states = states_dev;
  args.scales = scales_dev;
  args.plan = static_cast<const uint32_t*>(tables_dev);
  args.out = out_dev;
  args.store_kind = store_kind;
  args.vecs_per_row = static_cast<int>(vecs_per_row);
  args.num_vectors = vectors;
  args.tile_vectors = tv;
  args.num_tiles = static_cast<int>(tiles);
  args.error = error_dev;
  // row = floor(v / d) for v < 2^31 as umulhi(v, ceil(2^p / d)) >> (p - 32), p = 31 + ceil(log2 d), d >= 2.
  args.row_magic = 0;
  args.row_shift = 0;
  if (vecs_per_row > 1) {
    int log2_ceil = 0;
    while ((int64_t{1} << log2_ceil) < vecs_per_row) ++log2_ceil;
    const int p = 31 + log2_ceil;
    const unsigned __int128 power = static_cast<unsigned __int128>(1) << p;
    args.row_magic = static_cast<uint32_t>((power + vecs_per_row - 1) / vecs_per_row);
    args.row_shift = p - 32;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int pairs = static_cast<int>((tiles + 1) / 2);

  if (desc->table_kind == EP_TABLE_GLOBAL64) {
    const int waves_per_block = 4;
    const int blocks = (pairs + waves_per_block - 1) / waves_per_block;
    hipLaunchKernelGGL(decode_global64_kernel, dim3(blocks), dim3(waves_per_block * 64), 0, s, args);
    EP_HIP_TRY(hipGetLastError());
    return EP_HIP_OK;
  }
  if (desc->table_kind != EP_TABLE_LDS_BYTE && desc->table_kind != EP_TABLE_LDS_WIDE) return EP_HIP_EINVAL;
  if (desc->prob_bits > 11) return EP_HIP_EINVAL;

  int device = 0, cus = 0;
  EP_HIP_TRY(hipGetDevice(&device));
  EP_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  if (cus <= 0) cus = 256;
  // One resident block per CU (the table fills most of its LDS). Two interleaved pairs per wave once there is
  // enough work to fill 16 waves on every CU; otherwise spread the pairs over as many CUs as possible.
  const int ilp = pairs >= cus * 16 * 2 ? 2 : 1;
  int waves = (pairs + cus * ilp - 1) / (cus * ilp);
  waves = waves < 1 ? 1 : (waves > 16 ? 16 : waves);
  int blocks = (pairs + waves * ilp - 1) / (waves * ilp);
  blocks = blocks > cus ? cus : blocks;
  const bool wide = desc->table_kind == EP_TABLE_LDS_WIDE;
  const int threads = waves * 64;
  switch (desc->prob_bits) {
    case 9: return wide ? launch_lds_pb<9, true>(args, pairs, blocks, threads, ilp, s) : launch_lds_pb<9, false>(args, pairs, blocks, threads, ilp, s);
    case 10: return wide ? launch_lds_pb<10, true>(args, pairs, blocks, threads, ilp, s) : launch_lds_pb<10, false>(args, pairs, blocks, threads, ilp, s);
    default: return wide ? launch_lds_pb<11, true>(args, pairs, blocks, threads, ilp, s) : launch_lds_pb<11, false>(args, pairs, blocks, threads, ilp, s);
  }
}
