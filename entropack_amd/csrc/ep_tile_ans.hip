// Lossless tile_ans decode for gfx950: byte lanes, each raw or 32-way interleaved rANS over a 256-symbol table.
//
// Container: entropack/schemes/tile_ans/format.py:53-59 of the reference; decode semantics: eager.py:231-307,
// tile_ans.cu:175-470. Stream (lane b, tile t) holds byte b of elements [t * tile_elements, ...); streams are
// lane-major. A coded stream is decoded exactly like a lattice_rans tile with one symbol per group: tail group first,
// then whole groups of 32 downwards; after each symbol the states below 2^15 read one word each, the i-th reader in
// ascending lane order taking words[ptr - n + i]. Table entry: cdf << 20 | freq << 8 | symbol, freq 4096 stored as 0.
//
//   tile_ans_stream_kernel   any container: one stream per 32-lane half, table and words read from global memory
//                            (L2-resident), every renormalisation read bounds-checked, bytes stored one by one.
//   tile_ans_tile_kernel     containers with exactly one coded lane (bf16 / f16: raw low byte + coded high byte,
//                            f32: three raw + one coded, 1-byte types): one tile per 32-lane half, the lane's table
//                            in LDS, the words through the LDS windows and the scalar vote of the lattice decoder,
//                            raw bytes fetched one group ahead, whole elements stored.
#include "ep_decode_lds.hpp"

namespace ep {

constexpr int kMaxByteLanes = 8;

struct TileAnsArgs {
  const uint16_t* payload;
  uint64_t payload_words;
  const uint32_t* offsets;
  const uint32_t* states;
  const uint32_t* tables;
  uint8_t* out;
  int64_t tile_elements;
  int64_t elements;
  int64_t tiles;
  int prob_bits;
  int lanes;
  int coded_lane;                        // tile kernel: the one coded lane
  int wide_stores;                       // tile kernel: `out` is 16-byte aligned
  int* error;
  uint8_t raw[kMaxByteLanes];            // 1 = raw lane
  int coded_before[kMaxByteLanes];       // coded lanes before lane b (row block of `states`)
};

__device__ __forceinline__ void tile_ans_flag(int* error, int code) { atomicCAS(error, 0, code); }

// One stream per 32-lane half; both halves of a wave call this together (the votes are wave-wide).
__device__ __forceinline__ void decode_stream(const TileAnsArgs& a, int64_t stream, bool live, int half, int l32) {
  const int byte_lane = live ? static_cast<int>(stream / a.tiles) : 0;
  const int64_t tile = live ? stream % a.tiles : 0;
  const int64_t first = tile * a.tile_elements;
  const int64_t left = a.elements - first;
  int64_t count = live ? (left < a.tile_elements ? left : a.tile_elements) : 0;
  int64_t word_begin = 0, pointer = 0;
  if (live) {
    word_begin = a.offsets[stream];
    pointer = a.offsets[stream + 1];
    if (word_begin > pointer || static_cast<uint64_t>(pointer) > a.payload_words) {
      if (l32 == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
      count = 0;
    }
  }
  uint8_t* dst = a.out + first * a.lanes + byte_lane;
  const bool raw = live && a.raw[byte_lane] != 0;
  if (raw && count > 0) {
    if (pointer - word_begin != (count + 1) / 2) {
      if (l32 == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
    } else {
      for (int64_t e = l32; e < count; e += 32) {
        const uint32_t word = a.payload[word_begin + (e >> 1)];
        dst[e * a.lanes] = static_cast<uint8_t>((e & 1) ? word >> 8 : word);
      }
    }
  }

  // Coded streams. Both halves run the same number of rounds (the votes are wave-wide); a raw or idle half has none.
  const bool coded = live && !raw && count > 0;
  const int pb = a.prob_bits;
  const uint32_t slot_mask = (1u << pb) - 1u;
  const uint32_t* table = a.tables + (static_cast<size_t>(byte_lane) << pb);
  uint32_t x = kStateMin;
  if (coded) x = a.states[(static_cast<int64_t>(a.coded_before[byte_lane]) * a.tiles + tile) * kStatesPerTile + l32];
  const int64_t groups = coded ? (count + 31) >> 5 : 0;
  const int rem = static_cast<int>(count & 31);
  const int64_t other = __shfl_xor(groups, 32);
  const int64_t rounds = groups > other ? groups : other;
  for (int64_t round = 0; round < rounds; ++round) {
    const bool active = round < groups;
    const int64_t at = (groups - 1 - round) << 5;
    const int lanes_now = (round == 0 && rem != 0) ? rem : 32;
    const bool valid = active && l32 < lanes_now;
    if (valid) {
      const uint32_t slot = x & slot_mask;
      const uint32_t entry = table[slot];
      uint32_t freq = (entry >> 8) & 0xFFFu;
      if (freq == 0) freq = 1u << pb;
      dst[(at + l32) * a.lanes] = static_cast<uint8_t>(entry);
      x = freq * (x >> pb) + slot - (entry >> 20);
    }
    const bool read = valid && x < kStateMin;
    const uint64_t vote = __ballot(read);
    const uint32_t mine = half ? static_cast<uint32_t>(vote >> 32) : static_cast<uint32_t>(vote);
    if (read) {
      const int64_t from = pointer - __popc(mine >> l32);      // readers at or above this lane, itself included
      uint32_t word = 0;
      if (from >= word_begin) word = a.payload[from];
      else tile_ans_flag(a.error, EP_DECODE_OVERREAD);
      x = (x << 16) | word;
    }
    pointer -= __popc(mine);
  }
  if (coded && pointer != word_begin && l32 == 0) tile_ans_flag(a.error, pointer < word_begin ? EP_DECODE_OVERREAD : EP_DECODE_NOT_CONSUMED);
}

__global__ __launch_bounds__(256) void tile_ans_stream_kernel(TileAnsArgs a) {
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int64_t stream = 2 * (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) + half;
  decode_stream(a, stream, stream < a.tiles * a.lanes, half, lane & 31);
}

// ---- one coded lane ----------------------------------------------------------------------------------------------------
//
// LDS: the coded lane's table as 2^pb entries freq[0:12) | (slot - cdf)[12:24) | symbol << 24 at offset 0 (the byte
// form of the lattice decoder, so its step applies unchanged), then one 128-word window per half. A table that
// holds a frequency of 4096 (a one-symbol lane at prob_bits 12) does not fit that entry; a workgroup that meets one
// decodes its tiles stream by stream as the general kernel does.

template <int BYTES> struct ElementWord;
template <> struct ElementWord<1> { using type = uint8_t; };
template <> struct ElementWord<2> { using type = uint16_t; };
template <> struct ElementWord<4> { using type = uint32_t; };
template <> struct ElementWord<8> { using type = uint64_t; };

template <bool MASKED>
__device__ __forceinline__ uint32_t tile_ans_step(Pair& p, uint32_t pb, uint32_t kslot, uint32_t table_at, uint32_t shv, uint64_t valid) {
  uint32_t t, h, d, e, na, nb;
  uint64_t sv;
  uint32_t pos = uniform(p.pos);
  valid = uniform(valid);
#define EP_TILE_ANS_OPERANDS                                                                                        \
  : [x0] "+v"(p.x), [pos0] "+s"(pos), [e0] "=&v"(e), [t0] "=&v"(t), [h0] "=&v"(h), [d0] "=&v"(d), [na] "=&s"(na),       \
    [nb] "=&s"(nb), [sv] "=&s"(sv)                                                                                   \
  : [cb0] "v"(table_at), [ring0] "v"(p.ring), [shv] "v"(shv), [kslot] "s"(kslot), [valid] "s"(valid), [off] "n"(0),   \
    [pb] "s"(pb), [fmask] "n"(0xFFF), [dshift] "n"(12), [dwidth] "n"(12)                                             \
  : "vcc", "scc", "memory"
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_FIELD_SINGLE_BODY EP_ASM_MASK_OFF EP_TILE_ANS_OPERANDS);
  else asm volatile(EP_FIELD_SINGLE_FAST EP_TILE_ANS_OPERANDS);
  p.pos = pos;
  return e >> 24;
}

template <int BYTES>
__global__ __launch_bounds__(1024, BYTES == 8 ? 4 : 8) void tile_ans_tile_kernel(TileAnsArgs a, int num_pairs) {
  extern __shared__ __align__(16) uint8_t smem[];
  using Word = typename ElementWord<BYTES>::type;
  constexpr int RAW = BYTES - 1;
  typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
  const uint32_t pb = uniform(static_cast<uint32_t>(a.prob_bits));
  const uint32_t table_bytes = 4u << pb;
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr)smem));
  const int coded_lane = __builtin_amdgcn_readfirstlane(a.coded_lane);

  // One word behind the windows says whether the table holds a frequency the 12-bit field cannot.
  volatile uint32_t* wide_flag = reinterpret_cast<volatile uint32_t*>(smem + table_bytes + static_cast<uint32_t>(waves) * 2 * kRingBytes);
  if (threadIdx.x == 0) *wide_flag = 0u;
  __syncthreads();
  {
    const uint32_t* table = a.tables + (static_cast<size_t>(coded_lane) << pb);
    uint32_t* dst = reinterpret_cast<uint32_t*>(smem);
    for (uint32_t slot = threadIdx.x; slot < (1u << pb); slot += blockDim.x) {
      const uint32_t entry = table[slot];
      const uint32_t freq = (entry >> 8) & 0xFFFu;
      if (freq == 0) *wide_flag = 1u;
      dst[slot] = freq | (((slot - (entry >> 20)) & 0xFFFu) << 12) | (entry << 24);
    }
  }
  __syncthreads();
  const bool wide = *wide_flag != 0u;
  if (lds0 != 0) {      // the step addresses the table from LDS offset 0
    if (threadIdx.x == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
    return;
  }
  const int stride = static_cast<int>(gridDim.x) * waves;
  if (wide) {
    for (int pair = static_cast<int>(blockIdx.x) * waves + wave; pair < num_pairs; pair += stride) {
      const int64_t tile = 2 * static_cast<int64_t>(pair) + half;
      for (int b = 0; b < BYTES; ++b) decode_stream(a, static_cast<int64_t>(b) * a.tiles + tile, tile < a.tiles, half, l32);
    }
    return;
  }

  const uint32_t kslot = table_bytes - 4u;
  uint32_t shv = half ? 16u : 0u, table_at = 0u;
  asm volatile("" : "+v"(shv), "+v"(table_at));     // the step names them as vector operands
  const uint32_t* payload32 = reinterpret_cast<const uint32_t*>(a.payload);
  const uint8_t* payload8 = reinterpret_cast<const uint8_t*>(a.payload);
  const uint32_t window_at = lds0 + table_bytes + static_cast<uint32_t>(wave * 2 + half) * kRingBytes;
  // Byte positions of the raw lanes inside an element: every lane but the coded one, ascending.
  int raw_lane[RAW > 0 ? RAW : 1];
#pragma unroll
  for (int j = 0; j < RAW; ++j) raw_lane[j] = j + (j >= coded_lane ? 1 : 0);
  const int tile_elements = static_cast<int>(a.tile_elements);
  constexpr int kChunk = 256;                     // elements a half gathers before it stores
  const uint32_t stage_at = lds0 + table_bytes + static_cast<uint32_t>(waves) * 2 * kRingBytes + 16u + static_cast<uint32_t>(wave * 2 + half) * kChunk;

  for (int pair = static_cast<int>(blockIdx.x) * waves + wave; pair < num_pairs; pair += stride) {
    Pair s;
    const int64_t tile = 2 * static_cast<int64_t>(pair) + half;
    uint32_t word_begin = 0, word_end = 0;
    int count = 0;
    uint32_t raw_at[RAW > 0 ? RAW : 1];       // a raw lane's bytes of this tile are consecutive payload bytes: this lane's first
#pragma unroll
    for (int j = 0; j < RAW; ++j) raw_at[j] = 0;
    s.x = kStateMin;
    if (tile < a.tiles) {
      const int64_t left = a.elements - tile * a.tile_elements;
      count = static_cast<int>(left < a.tile_elements ? left : a.tile_elements);
      const int64_t coded_stream = static_cast<int64_t>(coded_lane) * a.tiles + tile;
      word_begin = a.offsets[coded_stream];
      word_end = a.offsets[coded_stream + 1];
      bool good = word_begin <= word_end && word_end <= a.payload_words;
#pragma unroll
      for (int j = 0; j < RAW; ++j) {
        const int64_t raw_stream = static_cast<int64_t>(raw_lane[j]) * a.tiles + tile;
        const uint32_t from = a.offsets[raw_stream], to = a.offsets[raw_stream + 1];
        good = good && from <= to && to <= a.payload_words && to - from == static_cast<uint32_t>((count + 1) >> 1);
        raw_at[j] = 2u * from + static_cast<uint32_t>(l32);      // the launcher keeps the payload below 4 GiB
      }
      if (!good) {
        if (l32 == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
        count = 0;
        word_begin = word_end = 0;
      } else {
        s.x = a.states[tile * kStatesPerTile + l32];
      }
    }
    open_window(s, window_at, word_begin, word_end, a.payload, a.payload_words, l32);
    // Wave-uniform base, 32-bit lane offsets: the addresses cost one vector add per access.
    Word* out = reinterpret_cast<Word*>(a.out) + 2 * static_cast<int64_t>(pair) * a.tile_elements;
    const uint32_t out_lane = static_cast<uint32_t>(half * tile_elements + l32);

    auto fetch_raw = [&](int at, bool valid_lane, uint32_t (&bytes)[RAW > 0 ? RAW : 1]) {
#pragma unroll
      for (int j = 0; j < RAW; ++j) bytes[j] = valid_lane ? payload8[raw_at[j] + static_cast<uint32_t>(at)] : 0u;
    };
    auto emit = [&](int at, uint32_t symbol, const uint32_t (&bytes)[RAW > 0 ? RAW : 1]) {
      Word value = static_cast<Word>(static_cast<Word>(symbol) << (8 * coded_lane));
#pragma unroll
      for (int j = 0; j < RAW; ++j) value |= static_cast<Word>(static_cast<Word>(bytes[j]) << (8 * raw_lane[j]));
      __builtin_nontemporal_store(value, out + (out_lane + static_cast<uint32_t>(at)));
    };

    const bool full = count == tile_elements && (tile_elements % kChunk) == 0 && a.wide_stores != 0;
    const bool all_full = __builtin_amdgcn_readfirstlane(__all(full) ? 1 : 0) != 0;
    if (all_full) {
      // Chunks of eight groups. The steps leave their symbols in this half's 256 bytes of LDS; then lane l takes
      // elements 8 l .. 8 l + 7 of the chunk: their symbols from LDS, 8 bytes of each raw lane from the payload
      // (requested before the steps), and stores the 8 elements as one piece. One memory instruction per raw lane
      // and 16 bytes of output per chunk, instead of one per group: the per-CU address path is the bottleneck otherwise.
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const uint32_t mine = 8u * static_cast<uint32_t>(l32);
#pragma unroll 1
      for (int at = tile_elements - kChunk; at >= 0; at -= kChunk) {
        u32x2 raw[RAW > 0 ? RAW : 1];
#pragma unroll
        for (int j = 0; j < RAW; ++j) __builtin_memcpy(&raw[j], payload8 + (raw_at[j] - static_cast<uint32_t>(l32) + static_cast<uint32_t>(at) + mine), 8);
#pragma unroll
        for (int g = kChunk / 32 - 1; g >= 0; --g) {
          const uint32_t symbol = tile_ans_step<false>(s, pb, kslot, table_at, shv, ~0ull);
          *reinterpret_cast<__attribute__((address_space(3))) uint8_t*>(static_cast<uintptr_t>(stage_at + 32u * g + l32)) = static_cast<uint8_t>(symbol);
          if ((g & 1) == 0) slide_window(s, half, payload32);     // a step takes at most 32 words, the window holds 64
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const u32x2 symbols = *reinterpret_cast<__attribute__((address_space(3))) const u32x2*>(static_cast<uintptr_t>(stage_at + mine));
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        Word* to = out + (out_lane - static_cast<uint32_t>(l32) + static_cast<uint32_t>(at) + mine);
        if constexpr (BYTES == 1) {
          __builtin_nontemporal_store(symbols, reinterpret_cast<u32x2*>(to));
        } else if constexpr (BYTES == 2) {
          // v_perm_b32 picks bytes from {second operand: 0..3, first operand: 4..7}.
          u32x4 v;
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const uint32_t low = coded_lane == 0 ? symbols[d >> 1] : raw[0][d >> 1];
            const uint32_t high = coded_lane == 0 ? raw[0][d >> 1] : symbols[d >> 1];
            v[d] = __builtin_amdgcn_perm(high, low, (d & 1) ? 0x07030602u : 0x05010400u);
          }
          __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(to));
        } else {
          Word e[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            e[i] = static_cast<Word>(static_cast<Word>((symbols[i >> 2] >> (8 * (i & 3))) & 0xFFu) << (8 * coded_lane));
#pragma unroll
            for (int j = 0; j < RAW; ++j) e[i] |= static_cast<Word>(static_cast<Word>((raw[j][i >> 2] >> (8 * (i & 3))) & 0xFFu) << (8 * raw_lane[j]));
          }
#pragma unroll
          for (int q = 0; q < BYTES / 2; ++q) {
            u32x4 v;
            if constexpr (BYTES == 4) {
              v = u32x4{e[4 * q], e[4 * q + 1], e[4 * q + 2], e[4 * q + 3]};
            } else {
              v = u32x4{static_cast<uint32_t>(e[2 * q]), static_cast<uint32_t>(static_cast<uint64_t>(e[2 * q]) >> 32),
                        static_cast<uint32_t>(e[2 * q + 1]), static_cast<uint32_t>(static_cast<uint64_t>(e[2 * q + 1]) >> 32)};
            }
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(to) + q);
          }
        }
      }
    } else {
      const int groups = (count + 31) >> 5;
      const int other = __shfl_xor(groups, 32);
      const int rounds = __builtin_amdgcn_readfirstlane(groups > other ? groups : other);
      const int rem = count & 31;
#pragma unroll 1
      for (int round = 0; round < rounds; ++round) {
        const int lanes_now = (round == 0 && rem != 0) ? rem : 32;
        const bool valid_lane = round < groups && l32 < lanes_now;
        const int at = (groups - 1 - round) << 5;
        uint32_t now[RAW > 0 ? RAW : 1];
        fetch_raw(at, valid_lane, now);
        const uint32_t symbol = tile_ans_step<true>(s, pb, kslot, table_at, shv, __builtin_amdgcn_ballot_w64(valid_lane));
        if (valid_lane) emit(at, symbol, now);
        slide_window(s, half, payload32);
      }
    }

    // A valid stream ends with every word consumed.
    const uint64_t live = __builtin_amdgcn_ballot_w64(count > 0);
    const bool liveA = (live & 1u) != 0, liveB = ((live >> 32) & 1u) != 0;
    const int ptrA = window_pointer_a(s), ptrB = window_pointer_b(s);
    if (((liveA && ptrA != s.beginA) || (liveB && ptrB != s.beginB)) && lane == 0) {
      const bool over = (liveA && ptrA < s.beginA) || (liveB && ptrB < s.beginB);
      tile_ans_flag(a.error, over ? EP_DECODE_OVERREAD : EP_DECODE_NOT_CONSUMED);
    }
  }
}

template <int BYTES>
static hipError_t launch_tile_kernel(const TileAnsArgs& args, int compute_units, hipStream_t stream) {
  const int64_t pairs = (args.tiles + 1) / 2;
  const int64_t resident = (BYTES == 8 ? 1 : 2) * static_cast<int64_t>(compute_units);
  // A pair is one long serial chain, so the grid walks the pairs in rounds, and a round costs about as much as it
  // has waves per SIMD (the steps are issue-bound from two waves per SIMD up): take the workgroup size whose last
  // round is fullest.
  int waves = 16;
  int64_t best = INT64_MAX;
  for (int w = 16; w >= 8; --w) {
    const int64_t rounds = (pairs + resident * w - 1) / (resident * w);
    if (rounds * w < best) {
      best = rounds * w;
      waves = w;
    }
  }
  const int64_t wanted = (pairs + waves - 1) / waves;
  const unsigned blocks = static_cast<unsigned>(wanted < resident ? wanted : resident);
  const size_t lds = (size_t{4} << args.prob_bits) + static_cast<size_t>(waves) * 2 * (kRingBytes + 256) + 16;
  hipLaunchKernelGGL(tile_ans_tile_kernel<BYTES>, dim3(blocks), dim3(waves * 64), lds, stream, args, static_cast<int>(pairs));
  return hipGetLastError();
}

}  // namespace ep

extern "C" int ep_hip_decode_tile_ans(const uint16_t* payload_dev, uint64_t payload_words, const uint32_t* offsets_dev,
                                      const uint32_t* states_dev, const uint32_t* decode_tables_dev,
                                      const uint8_t* lane_modes_host, int64_t tile_elements, int prob_bits, int num_lanes,
                                      int64_t num_elements, void* out_dev, int32_t* error_dev, void* stream) {
  using namespace ep;
  if (offsets_dev == nullptr || decode_tables_dev == nullptr || lane_modes_host == nullptr || out_dev == nullptr || error_dev == nullptr)
    return EP_HIP_EINVAL;
  if (payload_dev == nullptr && payload_words != 0) return EP_HIP_EINVAL;
  if (tile_elements <= 0 || prob_bits < 9 || prob_bits > 12 || num_elements <= 0) return EP_HIP_EINVAL;
  if (num_lanes != 1 && num_lanes != 2 && num_lanes != 4 && num_lanes != 8) return EP_HIP_EINVAL;
  if (payload_words > 0xFFFFFFFFull || reinterpret_cast<uintptr_t>(payload_dev) % 2 != 0) return EP_HIP_EINVAL;
  TileAnsArgs args;
  args.payload = payload_dev;
  args.payload_words = payload_words;
  args.offsets = offsets_dev;
  args.states = states_dev;
  args.tables = decode_tables_dev;
  args.out = static_cast<uint8_t*>(out_dev);
  args.tile_elements = tile_elements;
  args.elements = num_elements;
  args.tiles = (num_elements + tile_elements - 1) / tile_elements;
  args.prob_bits = prob_bits;
  args.lanes = num_lanes;
  args.coded_lane = -1;
  args.wide_stores = reinterpret_cast<uintptr_t>(out_dev) % 16 == 0;
  args.error = error_dev;
  int coded = 0;
  for (int b = 0; b < kMaxByteLanes; ++b) {
    args.raw[b] = 0;
    args.coded_before[b] = coded;
    if (b < num_lanes) {
      if (lane_modes_host[b] > 1) return EP_HIP_EINVAL;
      args.raw[b] = lane_modes_host[b];
      if (!args.raw[b]) {
        args.coded_lane = b;
        ++coded;
      }
    }
  }
  if (coded > 0 && states_dev == nullptr) return EP_HIP_EINVAL;
  const int64_t streams = args.tiles * num_lanes;
  if (streams >= (int64_t{1} << 31)) return EP_HIP_EUNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (coded == 1 && args.tile_elements < (int64_t{1} << 28) && payload_words < (uint64_t{1} << 31)) {
    int device = 0, compute_units = 0;
    EP_HIP_TRY(hipGetDevice(&device));
    EP_HIP_TRY(hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device));
    switch (num_lanes) {
      case 1: EP_HIP_TRY(launch_tile_kernel<1>(args, compute_units, s)); break;
      case 2: EP_HIP_TRY(launch_tile_kernel<2>(args, compute_units, s)); break;
      case 4: EP_HIP_TRY(launch_tile_kernel<4>(args, compute_units, s)); break;
      default: EP_HIP_TRY(launch_tile_kernel<8>(args, compute_units, s)); break;
    }
    return EP_HIP_OK;
  }
  const int waves_per_block = 4;
  const int64_t pairs = (streams + 1) / 2;
  const int64_t blocks = (pairs + waves_per_block - 1) / waves_per_block;
  hipLaunchKernelGGL(tile_ans_stream_kernel, dim3(static_cast<unsigned>(blocks)), dim3(waves_per_block * 64), 0, s, args);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}
