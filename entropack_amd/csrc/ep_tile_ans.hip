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
//                            f32: three raw + one coded, 1-byte types): one tile per half, table in LDS, raw bytes
//                            fetched alongside, whole elements stored (coalesced).
#include "ep_common.hpp"

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
  int* error;
  uint8_t raw[kMaxByteLanes];            // 1 = raw lane
  int coded_before[kMaxByteLanes];       // coded lanes before lane b (row block of `states`)
};

__device__ __forceinline__ void tile_ans_flag(int* error, int code) { atomicCAS(error, 0, code); }

__global__ __launch_bounds__(256) void tile_ans_stream_kernel(TileAnsArgs a) {
  const int lane = threadIdx.x & 63;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t stream = 2 * (static_cast<int64_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6)) + half;
  const bool live = stream < a.tiles * a.lanes;
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
  const int waves_per_block = 4;
  const int64_t pairs = (streams + 1) / 2;
  const int64_t blocks = (pairs + waves_per_block - 1) / waves_per_block;
  hipLaunchKernelGGL(tile_ans_stream_kernel, dim3(static_cast<unsigned>(blocks)), dim3(waves_per_block * 64), 0, s, args);
  EP_HIP_TRY(hipGetLastError());
  return EP_HIP_OK;
}
