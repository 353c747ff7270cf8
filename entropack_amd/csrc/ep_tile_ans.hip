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
//   tile_ans_tile_kernel     containers with at most four coded lanes (weights: bf16 / f16 raw low byte + coded high
//                            byte, f32 three raw + one coded, 1-byte types; integers with constant upper bytes; all
//                            raw): one tile per 32-lane half, the coded lanes' tables in LDS, the words through the
//                            LDS windows and the scalar vote of the lattice decoder, raw bytes fetched 256 elements
//                            ahead, whole elements stored 8 at a time.
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

// ---- tiles: every lane of a tile in one wave -------------------------------------------------------------------------------
//
// One tile per 32-lane half, all of its byte lanes together, whole elements stored. LDS: per coded lane its table as
// 2^pb entries freq[0:12) | (slot - cdf)[12:24) | symbol << 24 (the byte form of the lattice decoder, so its step
// applies unchanged; table c at offset c * 4 * 2^pb, the first at 0), then per half and coded lane one 128-word
// window and 256 bytes where the steps leave their symbols. A table that holds a frequency of 4096 (a one-symbol
// lane at prob_bits 12) does not fit that entry; a workgroup that meets one decodes its tiles stream by stream as
// the general kernel does.

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

// Two chains of one wave in lock step: both table gathers are in flight together, and each chain's vote runs while the
// other's window read returns.
template <bool MASKED>
__device__ __forceinline__ void tile_ans_step_dual(Pair& p0, Pair& p1, uint32_t pb, uint32_t kslot, uint32_t table0, uint32_t table1,
                                                   uint32_t shv, uint64_t valid, uint32_t& symbol0, uint32_t& symbol1) {
  uint32_t t0, h0, d0, e0, t1, h1, d1, e1, na, nb;
  uint64_t sv, m0;
  uint32_t pos0 = uniform(p0.pos), pos1 = uniform(p1.pos);
  valid = uniform(valid);
#define EP_TILE_ANS_DUAL_OPERANDS                                                                                    \
  : [x0] "+v"(p0.x), [x1] "+v"(p1.x), [pos0] "+s"(pos0), [pos1] "+s"(pos1), [e0] "=&v"(e0), [e1] "=&v"(e1),            \
    [t0] "=&v"(t0), [t1] "=&v"(t1), [h0] "=&v"(h0), [h1] "=&v"(h1), [d0] "=&v"(d0), [d1] "=&v"(d1), [na] "=&s"(na),      \
    [nb] "=&s"(nb), [sv] "=&s"(sv), [m0] "=&s"(m0)                                                                    \
  : [cb0] "v"(table0), [cb1] "v"(table1), [ring0] "v"(p0.ring), [ring1] "v"(p1.ring), [shv] "v"(shv), [kslot] "s"(kslot), \
    [valid] "s"(valid), [off] "n"(0), [pb] "s"(pb), [fmask] "n"(0xFFF), [dshift] "n"(12), [dwidth] "n"(12)             \
  : "vcc", "scc", "memory"
  if constexpr (MASKED) asm volatile(EP_ASM_MASK_ON EP_FIELD_DUAL_BODY EP_ASM_MASK_OFF EP_TILE_ANS_DUAL_OPERANDS);
  else asm volatile(EP_FIELD_DUAL_FAST EP_TILE_ANS_DUAL_OPERANDS);
  p0.pos = pos0;
  p1.pos = pos1;
  symbol0 = e0 >> 24;
  symbol1 = e1 >> 24;
}

constexpr int kTileChunk = 256;                      // elements a half gathers before it stores
// A wave walks its chains two at a time in lock step: the coded lanes of one tile pair (ILP = 1), or, for containers
// with a single coded lane and more tile pairs than one pass of waves holds, that lane of two tile pairs (ILP = 2).
constexpr int tile_kernel_waves_per_simd(int bytes, int coded) { return (coded <= 1 && bytes <= 4) ? 8 : 4; }

template <int BYTES, int CODED, int ILP>
__global__ __launch_bounds__(1024, tile_kernel_waves_per_simd(BYTES, CODED)) void tile_ans_tile_kernel(TileAnsArgs a, int num_pairs) {
  extern __shared__ __align__(16) uint8_t smem[];
  using Word = typename ElementWord<BYTES>::type;
  constexpr int RAW = BYTES - CODED;
  static_assert(ILP == 1 || (ILP == 2 && CODED == 1), "two tile pairs per wave are for single coded lanes");
  constexpr int CHAINS = CODED * ILP;                                      // chain k = coded lane k % CODED of pair k / CODED
  constexpr int NC = CODED > 0 ? CODED : 1, NR = RAW > 0 ? RAW : 1, NK = CHAINS > 0 ? CHAINS : 1;       // array sizes
  typedef __attribute__((address_space(3))) uint8_t* lds_ptr;
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const uint32_t pb = uniform(static_cast<uint32_t>(a.prob_bits));
  const uint32_t table_bytes = 4u << pb;
  const int waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr)smem));
  const uint32_t windows0 = CODED * table_bytes;
  const uint32_t stages0 = windows0 + static_cast<uint32_t>(waves) * 2 * CHAINS * kRingBytes;
  const uint32_t flag0 = stages0 + static_cast<uint32_t>(waves) * 2 * CHAINS * kTileChunk;

  // Byte positions inside an element: the coded lanes and the raw lanes, each ascending.
  int coded_pos[NC], raw_pos[NR];
  {
    int c = 0, r = 0;
#pragma unroll
    for (int b = 0; b < BYTES; ++b) {
      const bool is_raw = __builtin_amdgcn_readfirstlane(static_cast<int>(a.raw[b])) != 0;
#pragma unroll
      for (int i = 0; i < NC; ++i) if (CODED > 0 && !is_raw && c == i) coded_pos[i] = b;
#pragma unroll
      for (int i = 0; i < NR; ++i) if (RAW > 0 && is_raw && r == i) raw_pos[i] = b;
      c += is_raw ? 0 : 1;
      r += is_raw ? 1 : 0;
    }
  }

  // One word behind the staging areas says whether a table holds a frequency the 12-bit field cannot.
  volatile uint32_t* wide_flag = reinterpret_cast<volatile uint32_t*>(smem + flag0);
  if (threadIdx.x == 0) *wide_flag = 0u;
  __syncthreads();
#pragma unroll
  for (int c = 0; c < CODED; ++c) {
    const uint32_t* table = a.tables + (static_cast<size_t>(coded_pos[c]) << pb);
    uint32_t* dst = reinterpret_cast<uint32_t*>(smem + c * table_bytes);
    for (uint32_t slot = threadIdx.x; slot < (1u << pb); slot += blockDim.x) {
      const uint32_t entry = table[slot];
      const uint32_t freq = (entry >> 8) & 0xFFFu;
      if (freq == 0) *wide_flag = 1u;
      dst[slot] = freq | (((slot - (entry >> 20)) & 0xFFFu) << 12) | (entry << 24);
    }
  }
  __syncthreads();
  const bool wide = *wide_flag != 0u;
  if (lds0 != 0) {      // the step addresses the tables from LDS offset 0
    if (threadIdx.x == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
    return;
  }
  const int stride = static_cast<int>(gridDim.x) * waves * ILP;
  const int first_pair = (static_cast<int>(blockIdx.x) * waves + wave) * ILP;
  if (wide) {
    for (int pair0 = first_pair; pair0 < num_pairs; pair0 += stride) {
      for (int j = 0; j < ILP; ++j) {
        const int64_t tile = 2 * static_cast<int64_t>(pair0 + j) + half;
        const bool there = pair0 + j < num_pairs && tile < a.tiles;
        for (int b = 0; b < BYTES; ++b) decode_stream(a, static_cast<int64_t>(b) * a.tiles + tile, there, half, l32);
      }
    }
    return;
  }

  const uint32_t kslot = table_bytes - 4u;
  uint32_t shv = half ? 16u : 0u;
  uint32_t table_at[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) table_at[c] = static_cast<uint32_t>(c) * table_bytes;
  asm volatile("" : "+v"(shv));                           // the step names it as a vector operand
#pragma unroll
  for (int c = 0; c < NC; ++c) asm volatile("" : "+v"(table_at[c]));
  const uint8_t* payload8 = reinterpret_cast<const uint8_t*>(a.payload);
  const uint32_t mine_at = static_cast<uint32_t>(wave * 2 + half) * CHAINS;
  const int tile_elements = static_cast<int>(a.tile_elements);
  auto stage_of = [&](int k) { return lds0 + stages0 + (mine_at + static_cast<uint32_t>(k)) * kTileChunk; };

  for (int pair0 = first_pair; pair0 < num_pairs; pair0 += stride) {
    Pair st[NK];
    uint32_t raw_at[ILP][NR];  // a raw lane's bytes of a tile are consecutive payload bytes: the tile's first
    int count[ILP];
    bool full = true;
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      const int64_t tile = 2 * static_cast<int64_t>(pair0 + j) + half;
      uint32_t begin[NC], end[NC];
      count[j] = 0;
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        begin[c] = end[c] = 0;
        st[j * NC + c].x = kStateMin;
      }
#pragma unroll
      for (int r = 0; r < NR; ++r) raw_at[j][r] = 0;
      if (pair0 + j < num_pairs && tile < a.tiles) {
        const int64_t left = a.elements - tile * a.tile_elements;
        count[j] = static_cast<int>(left < a.tile_elements ? left : a.tile_elements);
        bool good = true;
#pragma unroll
        for (int c = 0; c < CODED; ++c) {
          const int64_t stream = static_cast<int64_t>(coded_pos[c]) * a.tiles + tile;
          begin[c] = a.offsets[stream];
          end[c] = a.offsets[stream + 1];
          good = good && begin[c] <= end[c] && end[c] <= a.payload_words;
        }
#pragma unroll
        for (int r = 0; r < RAW; ++r) {
          const int64_t stream = static_cast<int64_t>(raw_pos[r]) * a.tiles + tile;
          const uint32_t from = a.offsets[stream], to = a.offsets[stream + 1];
          good = good && from <= to && to <= a.payload_words && to - from == static_cast<uint32_t>((count[j] + 1) >> 1);
          raw_at[j][r] = 2u * from;                              // the launcher keeps the payload below 4 GiB
        }
        if (!good) {
          if (l32 == 0) tile_ans_flag(a.error, EP_DECODE_BAD_OFFSETS);
          count[j] = 0;
#pragma unroll
          for (int c = 0; c < NC; ++c) begin[c] = end[c] = 0;
        } else {
#pragma unroll
          for (int c = 0; c < CODED; ++c) st[j * NC + c].x = a.states[(static_cast<int64_t>(c) * a.tiles + tile) * kStatesPerTile + l32];
        }
      }
#pragma unroll
      for (int c = 0; c < CODED; ++c) {
        open_window(st[j * NC + c], lds0 + windows0 + (mine_at + static_cast<uint32_t>(j * NC + c)) * kRingBytes, begin[c], end[c], count[j] > 0,
                    a.payload, a.payload_words, a.offsets, l32);
      }
      full = full && count[j] == tile_elements;
    }
    // Wave-uniform bases, 32-bit lane offsets: the addresses cost one vector add per access.
    auto out_of = [&](int j) { return reinterpret_cast<Word*>(a.out) + 2 * static_cast<int64_t>(pair0 + j) * a.tile_elements; };
    const uint32_t out_half = static_cast<uint32_t>(half * tile_elements);

    full = full && (tile_elements % kTileChunk) == 0 && a.wide_stores != 0;
    const bool all_full = __builtin_amdgcn_readfirstlane(__all(full) ? 1 : 0) != 0;
    if (all_full) {
      // Chunks of eight groups. The steps leave their symbols in LDS; then lane l takes elements 8 l .. 8 l + 7 of
      // the chunk: their symbols from LDS, 8 bytes of each raw lane from the payload (requested before the steps),
      // and stores the 8 elements as one piece. One memory instruction per raw lane and per 16 bytes of output for a
      // whole chunk, instead of one per group: the per-CU address path is the bottleneck otherwise.
      const uint32_t mine = 8u * static_cast<uint32_t>(l32);
#pragma unroll 1
      for (int at = tile_elements - kTileChunk; at >= 0; at -= kTileChunk) {
        u32x2 raw[ILP][NR], symbols[NK];
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
#pragma unroll
          for (int r = 0; r < RAW; ++r) __builtin_memcpy(&raw[j][r], payload8 + (raw_at[j][r] + static_cast<uint32_t>(at) + mine), 8);
        }
        __builtin_amdgcn_s_setprio(1);      // the dependent steps go before other waves' independent work (below)
#pragma unroll
        for (int g = kTileChunk / 32 - 1; g >= 0; --g) {
          auto leave = [&](int k, uint32_t symbol) {
            *reinterpret_cast<__attribute__((address_space(3))) uint8_t*>(static_cast<uintptr_t>(stage_of(k) + 32u * g + l32)) = static_cast<uint8_t>(symbol);
          };
#pragma unroll
          for (int k = 0; k + 1 < CHAINS; k += 2) {
            uint32_t symbol0, symbol1;
            tile_ans_step_dual<false>(st[k], st[k + 1], pb, kslot, table_at[k % NC], table_at[(k + 1) % NC], shv, ~0ull, symbol0, symbol1);
            leave(k, symbol0);
            leave(k + 1, symbol1);
            if ((g & 1) == 0) {                          // a step takes at most 32 words, the window holds 64
              slide_window(st[k]);
              slide_window(st[k + 1]);
            }
          }
          if constexpr (CHAINS % 2 == 1) {
            constexpr int k = CHAINS - 1;
            leave(k, tile_ans_step<false>(st[k], pb, kslot, table_at[k % NC], shv, ~0ull));
            if ((g & 1) == 0) slide_window(st[k]);
          }
        }
        __builtin_amdgcn_s_setprio(0);
        if constexpr (CODED > 0) {
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int k = 0; k < CHAINS; ++k) {
            symbols[k] = *reinterpret_cast<__attribute__((address_space(3))) const u32x2*>(static_cast<uintptr_t>(stage_of(k) + mine));
          }
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
#pragma unroll
        for (int j = 0; j < ILP; ++j) {
          const u32x2* sym = symbols + j * NC;
          Word* to = out_of(j) + (out_half + static_cast<uint32_t>(at) + mine);
          if constexpr (BYTES == 1) {
            __builtin_nontemporal_store(CODED == 1 ? sym[0] : raw[j][0], reinterpret_cast<u32x2*>(to));
          } else if constexpr (BYTES == 2 && CODED == 1) {
            // v_perm_b32 picks bytes from {second operand: 0..3, first operand: 4..7}.
            u32x4 v;
#pragma unroll
            for (int d = 0; d < 4; ++d) {
              const uint32_t low = coded_pos[0] == 0 ? sym[0][d >> 1] : raw[j][0][d >> 1];
              const uint32_t high = coded_pos[0] == 0 ? raw[j][0][d >> 1] : sym[0][d >> 1];
              v[d] = __builtin_amdgcn_perm(high, low, (d & 1) ? 0x07030602u : 0x05010400u);
            }
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(to));
          } else {
            Word e[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
              e[i] = 0;
#pragma unroll
              for (int c = 0; c < CODED; ++c) e[i] |= static_cast<Word>(static_cast<Word>((sym[c][i >> 2] >> (8 * (i & 3))) & 0xFFu) << (8 * coded_pos[c]));
#pragma unroll
              for (int r = 0; r < RAW; ++r) e[i] |= static_cast<Word>(static_cast<Word>((raw[j][r][i >> 2] >> (8 * (i & 3))) & 0xFFu) << (8 * raw_pos[r]));
            }
            if constexpr (BYTES == 2) {
              const u32x4 v = {static_cast<uint32_t>(e[0]) | static_cast<uint32_t>(e[1]) << 16, static_cast<uint32_t>(e[2]) | static_cast<uint32_t>(e[3]) << 16,
                               static_cast<uint32_t>(e[4]) | static_cast<uint32_t>(e[5]) << 16, static_cast<uint32_t>(e[6]) | static_cast<uint32_t>(e[7]) << 16};
              __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(to));
            } else {
#pragma unroll
              for (int q = 0; q < BYTES / 2; ++q) {
                u32x4 v;
                if constexpr (BYTES == 4) {
                  v = u32x4{static_cast<uint32_t>(e[4 * q]), static_cast<uint32_t>(e[4 * q + 1]), static_cast<uint32_t>(e[4 * q + 2]), static_cast<uint32_t>(e[4 * q + 3])};
                } else {
                  v = u32x4{static_cast<uint32_t>(e[2 * q]), static_cast<uint32_t>(static_cast<uint64_t>(e[2 * q]) >> 32),
                            static_cast<uint32_t>(e[2 * q + 1]), static_cast<uint32_t>(static_cast<uint64_t>(e[2 * q + 1]) >> 32)};
                }
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(to) + q);
              }
            }
          }
        }
      }
    } else {
      // Short, missing or unaligned tiles: one tile pair after the other, one group per round, on its own lane mask.
#pragma unroll
      for (int j = 0; j < ILP; ++j) {
        const int groups = (count[j] + 31) >> 5;
        const int other = __shfl_xor(groups, 32);
        const int rounds = __builtin_amdgcn_readfirstlane(groups > other ? groups : other);
        const int rem = count[j] & 31;
        Word* out = out_of(j);
#pragma unroll 1
        for (int round = 0; round < rounds; ++round) {
          const int lanes_now = (round == 0 && rem != 0) ? rem : 32;
          const bool valid_lane = round < groups && l32 < lanes_now;
          const uint32_t at = static_cast<uint32_t>((groups - 1 - round) << 5) + static_cast<uint32_t>(l32);
          Word value = 0;
#pragma unroll
          for (int r = 0; r < RAW; ++r) {
            const uint32_t byte = valid_lane ? payload8[raw_at[j][r] + at] : 0u;
            value |= static_cast<Word>(static_cast<Word>(byte) << (8 * raw_pos[r]));
          }
          const uint64_t valid = __builtin_amdgcn_ballot_w64(valid_lane);
#pragma unroll
          for (int c = 0; c < CODED; ++c) {
            Pair& chain = st[j * NC + c];
            const uint32_t symbol = tile_ans_step<true>(chain, pb, kslot, table_at[c], shv, valid);
            value |= static_cast<Word>(static_cast<Word>(symbol) << (8 * coded_pos[c]));
            slide_window(chain);
          }
          if (valid_lane) __builtin_nontemporal_store(value, out + (out_half + at));
        }
      }
    }

    // A valid stream ends with every word consumed.
#pragma unroll
    for (int j = 0; j < ILP; ++j) {
      const uint64_t live = __builtin_amdgcn_ballot_w64(count[j] > 0);
      const bool liveA = (live & 1u) != 0, liveB = ((live >> 32) & 1u) != 0;
#pragma unroll
      for (int c = 0; c < CODED; ++c) {
        const Pair& chain = st[j * NC + c];
        const int ptrA = window_pointer_a(chain), ptrB = window_pointer_b(chain);
        if (((liveA && ptrA != chain.beginA) || (liveB && ptrB != chain.beginB)) && lane == 0) {
          const bool over = (liveA && ptrA < chain.beginA) || (liveB && ptrB < chain.beginB);
          tile_ans_flag(a.error, over ? EP_DECODE_OVERREAD : EP_DECODE_NOT_CONSUMED);
        }
      }
    }
  }
}

constexpr size_t kLdsLimitBytes = 160 * 1024;

static size_t tile_kernel_lds_bytes(int prob_bits, int coded, int ilp, int waves) {
  const int chains = coded * ilp;
  return static_cast<size_t>(coded) * (size_t{4} << prob_bits) + static_cast<size_t>(waves) * 2 * chains * (kRingBytes + kTileChunk) + 16;
}

// The workgroup size for `ilp` tile pairs per wave. A pair is one long serial chain, so the grid walks the pairs in
// passes, and a pass costs about as much as it has waves per SIMD: among the workgroup sizes that fit LDS and
// registers, the one whose passes are fullest. Returns the number of passes (0: nothing fits).
struct TileLaunch {
  int waves, resident;
  int64_t passes;
};
static TileLaunch plan_tile_launch(int prob_bits, int bytes, int coded, int ilp, int64_t pairs, int compute_units) {
  const int waves_per_cu = 4 * tile_kernel_waves_per_simd(bytes, coded);
  TileLaunch plan{0, 0, 0};
  int64_t best = INT64_MAX;
  for (int w = 16; w >= 1; --w) {
    const size_t lds = tile_kernel_lds_bytes(prob_bits, coded, ilp, w);
    if (lds > kLdsLimitBytes) continue;
    int blocks_per_cu = static_cast<int>(kLdsLimitBytes / lds);
    if (blocks_per_cu > 2) blocks_per_cu = 2;
    if (blocks_per_cu * w > waves_per_cu) blocks_per_cu = waves_per_cu / w;
    if (blocks_per_cu < 1) continue;
    const int64_t slots = static_cast<int64_t>(blocks_per_cu) * w * compute_units * ilp;
    const int64_t passes = (pairs + slots - 1) / slots;
    const int64_t cost = passes * blocks_per_cu * w;
    if (cost < best) {
      best = cost;
      plan = TileLaunch{w, blocks_per_cu, passes};
    }
  }
  return plan;
}

template <int BYTES, int CODED, int ILP>
static hipError_t launch_tile_kernel_as(const TileAnsArgs& args, const TileLaunch& plan, int compute_units, hipStream_t stream) {
  static thread_local int configured_for = -1;
  const int64_t pairs = (args.tiles + 1) / 2;
  const int64_t per_block = static_cast<int64_t>(plan.waves) * ILP;
  const int64_t wanted = (pairs + per_block - 1) / per_block;
  const int64_t most = static_cast<int64_t>(plan.resident) * compute_units;
  const unsigned blocks = static_cast<unsigned>(wanted < most ? wanted : most);
  const size_t lds = tile_kernel_lds_bytes(args.prob_bits, CODED, ILP, plan.waves);
  int device = 0;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) return status;
  if (configured_for != device) {
    status = hipFuncSetAttribute(reinterpret_cast<const void*>(tile_ans_tile_kernel<BYTES, CODED, ILP>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                 static_cast<int>(kLdsLimitBytes));
    if (status != hipSuccess) return status;
    configured_for = device;
  }
  hipLaunchKernelGGL((tile_ans_tile_kernel<BYTES, CODED, ILP>), dim3(blocks), dim3(plan.waves * 64), lds, stream, args, static_cast<int>(pairs));
  return hipGetLastError();
}

template <int BYTES, int CODED>
static hipError_t launch_tile_kernel(const TileAnsArgs& args, int compute_units, hipStream_t stream) {
  const int64_t pairs = (args.tiles + 1) / 2;
  const TileLaunch single = plan_tile_launch(args.prob_bits, BYTES, CODED, 1, pairs, compute_units);
  if (single.waves == 0) return hipErrorInvalidConfiguration;
  if constexpr (CODED == 1 && BYTES >= 2) {
    // More pairs than one pass of waves holds: two pairs per wave keep twice the chains in flight (measured 6-8 %
    // faster on two-byte elements; single-byte elements measure a few percent slower that way).
    if (single.passes > 1) {
      const TileLaunch twice = plan_tile_launch(args.prob_bits, BYTES, CODED, 2, pairs, compute_units);
      if (twice.waves != 0) return launch_tile_kernel_as<BYTES, CODED, 2>(args, twice, compute_units, stream);
    }
  }
  return launch_tile_kernel_as<BYTES, CODED, 1>(args, single, compute_units, stream);
}

// Containers the tile kernel is built for: up to four coded lanes (more: registers and LDS run out; the general
// kernel takes those).
constexpr int kMaxTileCodedLanes = 4;

template <int BYTES>
static hipError_t launch_tile_kernel_for(int coded, const TileAnsArgs& args, int compute_units, hipStream_t stream) {
  switch (coded) {
    case 0: return launch_tile_kernel<BYTES, 0>(args, compute_units, stream);
    case 1: return launch_tile_kernel<BYTES, 1>(args, compute_units, stream);
    case 2: if constexpr (BYTES >= 2) return launch_tile_kernel<BYTES, 2>(args, compute_units, stream); break;
    case 3: if constexpr (BYTES >= 4) return launch_tile_kernel<BYTES, 3>(args, compute_units, stream); break;
    case 4: if constexpr (BYTES >= 4) return launch_tile_kernel<BYTES, 4>(args, compute_units, stream); break;
    default: break;
  }
  return hipErrorInvalidValue;
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
  args.wide_stores = reinterpret_cast<uintptr_t>(out_dev) % 16 == 0;
  args.error = error_dev;
  int coded = 0;
  for (int b = 0; b < kMaxByteLanes; ++b) {
    args.raw[b] = 0;
    args.coded_before[b] = coded;
    if (b < num_lanes) {
      if (lane_modes_host[b] > 1) return EP_HIP_EINVAL;
      args.raw[b] = lane_modes_host[b];
      if (!args.raw[b]) ++coded;
    }
  }
  if (coded > 0 && states_dev == nullptr) return EP_HIP_EINVAL;
  const int64_t streams = args.tiles * num_lanes;
  if (streams >= (int64_t{1} << 31)) return EP_HIP_EUNSUPPORTED;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // The tile kernel counts a stream's window slides (one per 64 words, at most one word per element) in 16 bits.
  if (coded <= kMaxTileCodedLanes && args.tile_elements <= (int64_t{1} << 22) && payload_words < (uint64_t{1} << 31)) {
    int device = 0, compute_units = 0;
    EP_HIP_TRY(hipGetDevice(&device));
    EP_HIP_TRY(hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device));
    switch (num_lanes) {
      case 1: EP_HIP_TRY(launch_tile_kernel_for<1>(coded, args, compute_units, s)); break;
      case 2: EP_HIP_TRY(launch_tile_kernel_for<2>(coded, args, compute_units, s)); break;
      case 4: EP_HIP_TRY(launch_tile_kernel_for<4>(coded, args, compute_units, s)); break;
      default: EP_HIP_TRY(launch_tile_kernel_for<8>(coded, args, compute_units, s)); break;
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
